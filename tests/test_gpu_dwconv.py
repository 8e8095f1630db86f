"""GPU parity tests of DWConv / DWConvWGRAD: the HIP kernels, called through the C ABI by the
drop-in ops, against the CPU oracle, the golden vectors, closed forms and, at the full README
shape, size-independent properties.  Tolerances are the reference's own test criteria
(tests/ops/test_conv.py:28-36,75-83) plus tighter ones that fp32 accumulation makes possible."""
import itertools
import math

import pytest
import torch

import oracle
from conftest import cpu_gen, from_bits, rand_cl3d, rand_dw_weight
from kerops_amd.ops.conv import DWConv, DWConvStats, DWConvWGRAD
from kerops_amd.utils import allclose_two_stage, weight_grad_similarity

pytestmark = pytest.mark.gpu
DEV = 'cuda'

# odd / prime extents exercise every edge mask (the reference sweeps {2,3,7,13,16,32,37,53,111,128})
SHAPES = [
    (1, 8, 5, 4, 3), (2, 8, 7, 13, 37), (1, 8, 64, 64, 32), (3, 8, 2, 2, 2), (1, 8, 3, 111, 16),
    (1, 16, 13, 16, 32), (2, 16, 37, 3, 53), (1, 16, 2, 128, 7),
    (1, 32, 16, 7, 53), (2, 32, 3, 37, 13), (1, 32, 53, 2, 33),
    (1, 64, 9, 11, 35), (2, 64, 3, 2, 2), (1, 64, 33, 10, 40), (1, 64, 7, 53, 17),
    (1, 128, 6, 9, 18), (2, 128, 13, 3, 37),
]


def check_fwd(x, wk, y):
    ref16, ref32 = oracle.dwconv_fwd(x, wk, wide=True, return_fp32=True)
    y = y.cpu()
    assert y.shape == x.shape and y.dtype == torch.float16
    assert y.stride() == x.stride()
    # the reference's criterion (oracle plays the role of torch's conv3d there)
    assert allclose_two_stage(ref16, y, rtol_strict=1e-4, atol_strict=1e-3, rtol_narrow=1e-3, atol_narrow=2e-3)
    # fp32 accumulation: never more than one fp16 rounding away from the exact sum
    err = (y.float() - ref32).abs()
    assert (err <= 2.0 ** -11 * ref32.abs().clamp(min=2.0 ** -14) * 1.01 + 1e-6).all()
    # ... and almost always the same fp16 value as the rounded wide sum: the two differ where the fp32 sum's own
    # error (a few 2^-24 of the largest term) crosses a rounding boundary of fp16, about 0.15 % of the outputs
    same = (y.contiguous().view(torch.int16) == ref16.contiguous().view(torch.int16)).float().mean().item()
    assert same >= 0.998 - 3.0 * math.sqrt(0.002 / y.numel()), same


@pytest.mark.parametrize('shape', SHAPES)
def test_dwconv_matches_oracle(shape):
    g = cpu_gen()
    x = rand_cl3d(g, *shape)
    _, wk = rand_dw_weight(g, shape[1])
    check_fwd(x, wk, DWConv(x.to(DEV), wk.to(DEV)))


@pytest.mark.parametrize('shape', SHAPES)
def test_dwconv_wgrad_matches_oracle(shape):
    g = cpu_gen()
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    ref = oracle.dwconv_wgrad(x, grad)
    gw32 = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.float32).cpu()
    assert list(gw32.shape) == [3, 3, 3, shape[1]] and gw32.dtype == torch.float32
    rel = ((gw32.double() - ref).norm() / ref.norm()).item()
    assert rel < 2e-6, rel
    # drop-in result type (fp16) and the reference's own criterion
    gw16 = DWConvWGRAD(x.to(DEV), grad.to(DEV)).cpu()
    assert gw16.dtype == torch.float16
    # the fp16 result is written by the reduction kernel: the fp32 sum rounded once, as a cast of it rounds
    assert torch.equal(gw16.view(torch.int16), gw32.to(torch.float16).view(torch.int16))
    gwbf = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.bfloat16).cpu()  # any other type: cast from fp32
    assert gwbf.dtype == torch.bfloat16 and torch.equal(gwbf.view(torch.int16), gw32.bfloat16().view(torch.int16))
    if ref.abs().max() < 6e4:
        assert weight_grad_similarity(ref.float(), gw16.float(), rtol_cos=1e-4, atol_cos=1e-4,
                                      rtol_len=1e-3 * shape[0], atol_len=1e-3)


@pytest.mark.parametrize('shape', SHAPES + [(1, 64, 40, 70, 33), (2, 16, 30, 64, 64), (1, 8, 50, 40, 64)])
def test_dwconv_stats_equals_dwconv_then_stats(shape):
    g = cpu_gen(5)
    x = rand_cl3d(g, *shape) * 1.5 + 0.25
    _, wk = rand_dw_weight(g, shape[1])
    xd, wd = x.to(DEV), wk.to(DEV)
    y, mean, sq = DWConvStats(xd, wd)
    assert torch.equal(y, DWConv(xd, wd))  # same kernel body, same rounding
    assert mean.dtype == sq.dtype == torch.float32 and mean.shape == sq.shape == (shape[1],)
    rm, rs = oracle.stats(y.cpu())  # the statistics of the tensor as stored
    assert torch.allclose(mean.cpu().double(), rm, rtol=2e-6, atol=2e-6)
    assert torch.allclose(sq.cpu().double(), rs, rtol=2e-6, atol=2e-6)
    y2, mean2, sq2 = DWConvStats(xd, wd)
    assert torch.equal(mean, mean2) and torch.equal(sq, sq2)  # fixed summation order


@pytest.mark.parametrize('shape', [(1, 8, 1, 1, 1), (1, 16, 1, 5, 1), (2, 64, 4, 1, 9), (1, 32, 1, 1, 70), (3, 128, 1, 2, 1),
                                   (1, 8, 300, 1, 1)])
def test_extents_of_one(shape):
    # below the smallest extent of the reference's grid (2): whole taps fall outside the volume
    g = cpu_gen(11)
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    _, wk = rand_dw_weight(g, shape[1])
    check_fwd(x, wk, DWConv(x.to(DEV), wk.to(DEV)))
    ref = oracle.dwconv_wgrad(x, grad)
    gw32 = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.float32).cpu()
    assert ((gw32.double() - ref).norm() / max(ref.norm().item(), 1e-30)).item() < 2e-6
    assert torch.equal(gw32 == 0, ref == 0)  # taps that never meet the volume stay exactly zero
    y, mean, sq = DWConvStats(x.to(DEV), wk.to(DEV))
    rm, rs = oracle.stats(y.cpu())
    assert torch.allclose(mean.cpu().double(), rm, rtol=2e-6, atol=2e-6)
    assert torch.allclose(sq.cpu().double(), rs, rtol=2e-6, atol=2e-6)


def fixture_grid_sample(n, channels, max_voxels, seed):
    """A deterministic sample of the grid the reference's tests sweep (tests/conftest.py:4-36): batch 1-4, three
    extents from {2,3,7,13,16,32,37,53,111,128}, bounded so that the oracle stays fast."""
    import random
    rng = random.Random(seed)
    extents = [2, 3, 7, 13, 16, 32, 37, 53, 111, 128]
    out = []
    while len(out) < n:
        shape = (rng.choice([1, 2, 3, 4]), rng.choice(channels), rng.choice(extents), rng.choice(extents),
                 rng.choice(extents))
        if shape[0] * shape[2] * shape[3] * shape[4] * shape[1] <= max_voxels * 8 and shape not in out:
            out.append(shape)
    return out


# batch 4 with the two largest extents of the reference's grid (111, 128) at 64 and 128 channels: rare in a random
# sample of bounded size, so they are listed; the third extent is kept small to bound the oracle's work
FORCED_GRID = [(4, 64, 111, 128, 2), (4, 128, 128, 111, 3), (4, 64, 2, 111, 128), (4, 128, 3, 128, 111),
               (4, 64, 128, 2, 111), (4, 128, 111, 3, 128), (4, 64, 128, 128, 2), (4, 128, 111, 111, 2),
               (3, 64, 7, 128, 111), (4, 128, 2, 128, 128)]


@pytest.mark.parametrize('shape', fixture_grid_sample(500, [8, 16, 32, 64, 128], 150_000, seed=322) + FORCED_GRID)
def test_reference_fixture_grid_sample(shape):
    g = cpu_gen(sum(shape))
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    _, wk = rand_dw_weight(g, shape[1])
    check_fwd(x, wk, DWConv(x.to(DEV), wk.to(DEV)))
    ref = oracle.dwconv_wgrad(x, grad)
    gw32 = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.float32).cpu()
    rel = ((gw32.double() - ref).norm() / ref.norm()).item()
    assert rel < 2e-6, rel


from kerops_amd.ops.conv.variants import FWD_VARIANTS, WGRAD_VARIANTS as WG_VARIANTS  # noqa: E402


@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
def test_every_built_launch_shape(c):
    """Every (W_block, D_block, lane_channels) the library is built with, with several H_chunk
    values (chunk borders inside the volume, chunk of one row, chunk larger than H)."""
    g = cpu_gen(7)
    shape = (2, c, 11, 19, 37)
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    _, wk = rand_dw_weight(g, c)
    ref_gw = oracle.dwconv_wgrad(x, grad)
    xd, gd, wd = x.to(DEV), grad.to(DEV), wk.to(DEV)
    for (tw, td, cl), hc in itertools.product(FWD_VARIANTS[c], (0, 1, 4, 100)):
        check_fwd(x, wk, DWConv(xd, wd, W_block=tw, D_block=td, lane_channels=cl, H_chunk=hc))
    for (tw, td, cl), hc in itertools.product(WG_VARIANTS[c], (0, 1, 4, 100)):
        gw = DWConvWGRAD(xd, gd, W_block=tw, D_block=td, lane_channels=cl, H_chunk=hc, out_dtype=torch.float32)
        rel = ((gw.cpu().double() - ref_gw).norm() / ref_gw.norm()).item()
        assert rel < 2e-6, (tw, td, cl, hc, rel)


@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
def test_balanced_split_small(c):
    """The balanced split of the H march (H_chunk = 0, and explicit group sizes -g): shares that end inside a
    bundle of patches, a partly filled last bundle, groups larger than the tensor, group sizes that do not divide
    the resident workgroup count, several samples.  The forward result does not depend on the split (bit-identical
    to one uniform chunk, itself checked against the oracle); the weight gradient is checked against the oracle."""
    g = cpu_gen(11)
    shape = (3, c, 13, 21, 37)
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    _, wk = rand_dw_weight(g, c)
    xd, gd, wd = x.to(DEV), grad.to(DEV), wk.to(DEV)
    one_chunk = DWConv(xd, wd, H_chunk=100)
    check_fwd(x, wk, one_chunk)
    for hc in (0, -1, -2, -3, -4, -7, -16, -64, -600):
        assert torch.equal(DWConv(xd, wd, H_chunk=hc), one_chunk), hc
    ref_gw = oracle.dwconv_wgrad(x, grad)
    for hc in (0, -2, -4, -6, -16, -64, -600):
        gw = DWConvWGRAD(xd, gd, H_chunk=hc, out_dtype=torch.float32)
        rel = ((gw.cpu().double() - ref_gw).norm() / ref_gw.norm()).item()
        assert rel < 2e-6, (hc, rel)
        assert torch.equal(gw, DWConvWGRAD(xd, gd, H_chunk=hc, out_dtype=torch.float32)), hc  # deterministic


@pytest.mark.parametrize('shape', [(1, 8, 9, 300, 1000), (1, 16, 9, 300, 600), (1, 32, 9, 200, 400),
                                   (1, 64, 9, 260, 260), (1, 128, 9, 130, 260), (2, 64, 5, 260, 130)])
def test_balanced_split_many_patches(shape):
    """More patches than resident workgroups: every group owns several bundles and crosses from one into the next
    in the middle of its share (for 128 channels with both slabs in a bundle); the last bundle holds a single
    patch.  Compared on the GPU with uniform chunks of the whole height, which the tests above pin to the oracle."""
    g = torch.Generator(DEV).manual_seed(sum(shape))
    n, c, h, w, d = shape
    xd = torch.randn(n, h, w, d, c, device=DEV, dtype=torch.float16, generator=g).permute(0, 4, 1, 2, 3)
    gd = torch.randn(n, h, w, d, c, device=DEV, dtype=torch.float16, generator=g).permute(0, 4, 1, 2, 3)
    wd = (torch.randn(3, 3, 3, c, device=DEV, generator=g) / 5).half()
    y_uniform = DWConv(xd, wd, H_chunk=h)
    gw_uniform = DWConvWGRAD(xd, gd, H_chunk=h, out_dtype=torch.float32)
    for hc in (0, -64, -128, -34):
        assert torch.equal(DWConv(xd, wd, H_chunk=hc), y_uniform), hc
        gw = DWConvWGRAD(xd, gd, H_chunk=hc, out_dtype=torch.float32)
        rel = ((gw.double() - gw_uniform.double()).norm() / gw_uniform.double().norm()).item()
        assert rel < 2e-6, (hc, rel)


def test_golden_vectors(golden):
    x = from_bits(golden['x']).to(memory_format=torch.channels_last_3d)
    grad = from_bits(golden['grad']).to(memory_format=torch.channels_last_3d)
    wk = from_bits(golden['weight_c13x3x3'])[:, 0].permute(1, 2, 3, 0).contiguous()
    y = DWConv(x.to(DEV), wk.to(DEV)).cpu()
    y32 = torch.from_numpy(golden['dwconv_y_f32'])
    assert (y.float() - y32).abs().max() <= 2.0 ** -11 * max(1.0, y32.abs().max().item()) * 1.01
    assert torch.allclose(y.float(), y32, rtol=1e-2, atol=1e-2)  # the tolerance stated for the README-shape forward
    gw = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.float32).cpu().double()
    ref = torch.from_numpy(golden['dwconv_wgrad_f64'])
    assert ((gw - ref).norm() / ref.norm()).item() < 1e-6


def test_config1_golden_fixture(golden_config1):
    """The CPU-runnable target configuration, x (1,8,64,64,32) ~ N(0,1), weight ~ N(0,1/27): the committed vectors were
    written by torch's CPU conv3d(groups=C) in fp32 (output cast to fp16) and its fp64 autograd."""
    x = from_bits(golden_config1['x']).to(memory_format=torch.channels_last_3d)
    wk = from_bits(golden_config1['weight_c13x3x3'])[:, 0].permute(1, 2, 3, 0).contiguous()
    y = DWConv(x.to(DEV), wk.to(DEV)).cpu()
    ref = from_bits(golden_config1['dwconv_y'])
    assert y.shape == ref.shape == (1, 8, 64, 64, 32)
    assert torch.allclose(y.float(), ref.float(), rtol=1e-2, atol=1e-2)  # the configuration's stated tolerance
    # both sides round an fp32 sum of the same 27 products once: at most one fp16 step apart, and almost always equal
    assert allclose_two_stage(ref, y.contiguous(), rtol_strict=1e-4, atol_strict=1e-3, rtol_narrow=1e-3, atol_narrow=2e-3)
    same = (y.contiguous().view(torch.int16) == ref.view(torch.int16)).float().mean().item()
    assert same >= 0.998, same
    grad = torch.flip(x, dims=(2, 3, 4)).contiguous(memory_format=torch.channels_last_3d)  # as the generator defines it
    gw = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.float32).cpu().double()
    gref = torch.from_numpy(golden_config1['dwconv_wgrad_f64'])
    assert ((gw - gref).norm() / gref.norm()).item() < 1e-6


def test_single_taps_copy_every_fp16_value():
    """Weight = one 1.0 at a tap: the output is the input shifted, bit for bit, for every finite
    fp16 pattern including subnormals (no flush to zero, no rounding in the fp32 path)."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    fin = bits[torch.isfinite(bits)]
    H, W, D, c = 31, 16, 16, 8
    flat = torch.zeros(H * W * D * c, dtype=torch.float16)
    flat[:fin.numel()] = fin
    x = flat.view(1, H, W, D, c).permute(0, 4, 1, 2, 3)
    xd = x.to(DEV)
    for kh, kw, kd in [(1, 1, 1), (0, 0, 0), (2, 2, 2), (0, 1, 2), (2, 1, 0), (1, 2, 1)]:
        wk = torch.zeros(3, 3, 3, c, dtype=torch.float16)
        wk[kh, kw, kd] = 1.0
        y = DWConv(xd, wk.to(DEV)).cpu()
        exp = torch.zeros_like(x)
        sh, sw, sd = kh - 1, kw - 1, kd - 1
        src = x[:, :, max(sh, 0):H + min(sh, 0), max(sw, 0):W + min(sw, 0), max(sd, 0):D + min(sd, 0)]
        exp[:, :, max(-sh, 0):H + min(-sh, 0), max(-sw, 0):W + min(-sw, 0), max(-sd, 0):D + min(-sd, 0)] = src
        same = (y.view(torch.int16) == exp.view(torch.int16)) | ((y == 0) & (exp == 0))
        assert same.all(), (kh, kw, kd)


def test_ones_count_neighbours_and_wgrad_closed_form():
    c, H, W, D = 64, 5, 9, 21
    ones = torch.ones(1, c, H, W, D, dtype=torch.float16).to(memory_format=torch.channels_last_3d).to(DEV)
    y = DWConv(ones, torch.ones(3, 3, 3, c, dtype=torch.float16, device=DEV)).cpu()

    def cnt(n):
        v = torch.full((n,), 3.0)
        v[0] = v[-1] = 2.0
        return v

    exp = cnt(H).view(H, 1, 1) * cnt(W).view(1, W, 1) * cnt(D).view(1, 1, D)
    assert torch.equal(y[0, 0].float(), exp) and torch.equal(y[0, c - 1].float(), exp)
    gw = DWConvWGRAD(ones, ones, out_dtype=torch.float32).cpu()
    for kh, kw, kd in itertools.product(range(3), repeat=3):
        assert gw[kh, kw, kd, 0].item() == (H - abs(kh - 1)) * (W - abs(kw - 1)) * (D - abs(kd - 1))


def test_wgrad_is_deterministic():
    g = cpu_gen(21)
    x, grad = rand_cl3d(g, 2, 64, 23, 17, 40).to(DEV), rand_cl3d(g, 2, 64, 23, 17, 40).to(DEV)
    a = DWConvWGRAD(x, grad, out_dtype=torch.float32)
    b = DWConvWGRAD(x, grad, out_dtype=torch.float32)
    assert torch.equal(a, b)


def test_config3_wgrad_crop_fp64():
    """Weight-gradient target configuration: rel L2 error <= 1e-3 against an fp64 CPU reduction on (1,64,96,96,64)."""
    g = cpu_gen()
    shape = (1, 64, 96, 96, 64)
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    ref = oracle.dwconv_wgrad(x, grad)
    gw = DWConvWGRAD(x.to(DEV), grad.to(DEV), out_dtype=torch.float32).cpu().double()
    rel = ((gw - ref).norm() / ref.norm()).item()
    assert rel <= 1e-3 and rel < 1e-5, rel
    gw16 = DWConvWGRAD(x.to(DEV), grad.to(DEV)).cpu().double()
    assert ((gw16 - ref).norm() / ref.norm()).item() <= 1e-3


@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
def test_readme_shape_properties(c):
    """Full (1, C, 350, 350, 128): (a) slabs of the output, including every border, equal the
    oracle run on the matching input slab; (b) the adjoint identity
    <DWConv(x, w), g> = <w, DWConvWGRAD(x, g)> ties forward and weight gradient together at a
    size the CPU oracle cannot sweep."""
    gen = torch.Generator(DEV).manual_seed(322)
    H, W, D = 350, 350, 128
    x = torch.randn(1, H, W, D, c, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    grad = torch.randn(1, H, W, D, c, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    _, wk = rand_dw_weight(cpu_gen(), c)
    wd = wk.to(DEV)
    y = DWConv(x, wd)
    gw = DWConvWGRAD(x, grad, out_dtype=torch.float32)

    lhs = torch.zeros((), dtype=torch.float64, device=DEV)
    for h0 in range(0, H, 50):  # chunked fp64 reduction keeps temporaries small
        lhs += (y[:, :, h0:h0 + 50].double() * grad[:, :, h0:h0 + 50].double()).sum()
    rhs = (wd.double() * gw.double()).sum()
    assert abs(lhs.item() - rhs.item()) <= 1e-3 * max(abs(rhs.item()), 1e3), (lhs.item(), rhs.item())

    # slabs: (h range, w range, d range) of the output; the input slab carries a halo of one
    for (h0, h1), (w0, w1), (d0, d1) in [((0, 6), (0, 9), (0, 20)), ((344, 350), (341, 350), (108, 128)),
                                         ((170, 176), (0, 9), (50, 90)), ((57, 63), (170, 182), (0, 128))]:
        ha, hb = max(h0 - 1, 0), min(h1 + 1, H)
        wa, wb = max(w0 - 1, 0), min(w1 + 1, W)
        da, db = max(d0 - 1, 0), min(d1 + 1, D)
        xs = x[:, :, ha:hb, wa:wb, da:db].cpu().contiguous(memory_format=torch.channels_last_3d)
        ref16, ref32 = oracle.dwconv_fwd(xs, wk, wide=True, return_fp32=True)
        sl = (slice(None), slice(None), slice(h0 - ha, h0 - ha + h1 - h0), slice(w0 - wa, w0 - wa + w1 - w0),
              slice(d0 - da, d0 - da + d1 - d0))
        got = y[:, :, h0:h1, w0:w1, d0:d1].cpu()
        # a slab border that is not a volume border sees zero padding in the oracle run: the
        # halo removes exactly those rows from the comparison
        assert torch.allclose(got.float(), ref32[sl], rtol=1e-2, atol=1e-2)  # tolerance stated for the README-shape forward
        assert (got.float() - ref32[sl]).abs().max() <= 2.0 ** -11 * max(1.0, ref32.abs().max().item()) * 1.01


@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
@pytest.mark.parametrize('shape_hc', [((2, 11, 19, 37), 0), ((1, 5, 3, 2), 0), ((1, 13, 9, 70), 4), ((1, 9, 8, 8), 1),
                                      ((1, 7, 20, 130), 100)])
def test_fused_backward_matches_oracle_and_separate_ops(c, shape_hc):
    """DWConvBackward = (DWConv(grad, flipped weight), DWConvWGRAD(x, grad)), every plane of grad staged once."""
    from kerops_amd.ops.conv import DWConvBackward
    (n, h, w, d), hc = shape_hc
    g = cpu_gen(c + h)
    x, grad = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    _, wk = rand_dw_weight(g, c)
    xd, gd, wd = x.to(DEV), grad.to(DEV), wk.to(DEV)
    dx, gw = DWConvBackward(xd, gd, wd, H_chunk=hc, out_dtype=torch.float32)
    assert dx.shape == x.shape and dx.stride() == x.stride() and gw.shape == (3, 3, 3, c)
    ref_gw = oracle.dwconv_wgrad(x, grad)
    rel = ((gw.cpu().double() - ref_gw).norm() / ref_gw.norm()).item()
    assert rel < 2e-6, rel
    wflip = torch.flip(wk, dims=(0, 1, 2)).contiguous()
    check_fwd(grad, wflip, dx)
    # same arithmetic as the separate matrix-core kernels: the input gradient agrees to the last bit
    dx2 = DWConv(gd, wflip.to(DEV))
    assert torch.equal(dx, dx2)
    gw2 = DWConvWGRAD(xd, gd, out_dtype=torch.float32)
    assert ((gw - gw2).norm() / gw2.norm()).item() < 2e-6  # other patch shape, other summation order
    # determinism
    dx3, gw3 = DWConvBackward(xd, gd, wd, H_chunk=hc, out_dtype=torch.float32)
    assert torch.equal(dx, dx3) and torch.equal(gw, gw3)
    # default result type fp16, written by the reduction kernel = the fp32 sum rounded once
    dx4, gw4 = DWConvBackward(xd, gd, wd, H_chunk=hc)
    assert gw4.dtype == torch.float16 and torch.equal(dx, dx4)
    assert torch.equal(gw4.view(torch.int16), gw.to(torch.float16).view(torch.int16))


@pytest.mark.parametrize('c', [8, 64])
@pytest.mark.parametrize('h', [4, 5, 6, 7, 8, 9])
@pytest.mark.parametrize('hc', [0, 3, 4, 5])
def test_march_period_of_four_every_step_count(c, h, hc):
    """The marching kernels run their plane steps in groups of four (the accumulator registers of a tile are a
    ring of four planes): every residue of the step count mod 4, with chunk borders inside the volume (hc rows per
    chunk) and without (0: balanced split), for the forward kernel, the statistics mode and the fused backward."""
    from kerops_amd.ops.conv import DWConvBackward
    g = cpu_gen(17 * c + 5 * h + hc)
    x, grad = rand_cl3d(g, 1, c, h, 9, 12), rand_cl3d(g, 1, c, h, 9, 12)
    _, wk = rand_dw_weight(g, c)
    xd, gd, wd = x.to(DEV), grad.to(DEV), wk.to(DEV)
    y = DWConv(xd, wd, H_chunk=hc)
    check_fwd(x, wk, y)
    assert torch.equal(y, DWConv(xd, wd))
    ys, mean, sqmean = DWConvStats(xd, wd)
    assert torch.equal(ys, y)
    yf = y.float()
    assert torch.allclose(mean.cpu(), yf.mean(dim=(0, 2, 3, 4)).cpu(), rtol=1e-5, atol=1e-6)
    assert torch.allclose(sqmean.cpu(), (yf * yf).mean(dim=(0, 2, 3, 4)).cpu(), rtol=1e-5, atol=1e-6)
    dx, gw = DWConvBackward(xd, gd, wd, H_chunk=hc, out_dtype=torch.float32)
    wflip = torch.flip(wk, dims=(0, 1, 2)).contiguous()
    check_fwd(grad, wflip, dx)
    ref_gw = oracle.dwconv_wgrad(x, grad)
    assert ((gw.cpu().double() - ref_gw).norm() / ref_gw.norm()).item() < 2e-6
