"""Full README shape (1, C, 350, 350, 128): every value of the weight gradient and every voxel of the forward
output, checked on the GPU against independent restatements that torch evaluates there in chunks.

The CPU oracle cannot sweep 15.7 M voxels per channel in a test, so the references here are torch expressions whose
meaning does not depend on any kernel of this library:

  * weight gradient: the 27 taps as 27 sliced dot products, gw[kh,kw,kd,c] = sum g[h,w,d,c] * x[h+kh-1,w+kw-1,d+kd-1,c]
    over the overlapping boxes of g and the shifted x, accumulated in fp64 over chunks of H (the restatement the
    oracle itself is pinned with on small shapes, tests/test_oracle_pin.py);
  * forward: the 27 shifted products summed in fp32 per chunk of H, and torch's own conv3d(groups=C) on the GPU
    under the reference's criterion (tests/ops/test_conv.py:25-36 of the reference).
"""
import pytest
import torch

from conftest import cpu_gen, rand_dw_weight
from kerops_amd.ops.conv import DWConv, DWConvBackward, DWConvWGRAD
from kerops_amd.utils import allclose_two_stage

DEV = 'cuda'
H, W, D = 350, 350, 128


def make(c, seed=322):
    gen = torch.Generator(DEV).manual_seed(seed + c)
    x = torch.randn(1, H, W, D, c, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    g = torch.randn(1, H, W, D, c, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    return x, g


def box(n, k):
    """Index ranges of g and of x along an axis of extent n for tap offset k - 1 (x index = g index + k - 1)."""
    s = k - 1
    return slice(max(0, -s), n - max(0, s)), slice(max(0, s), n - max(0, -s))


def wgrad_by_sliced_dots(x, g, rows=10):
    """[3,3,3,C] fp64: every tap as a dot product over the box where g and the shifted x overlap, in chunks of
    `rows` planes of g (each chunk converts its planes of g and the planes of x around them to fp64 once)."""
    _, c, H, W, D = x.shape
    xv, gv = x[0].permute(1, 2, 3, 0), g[0].permute(1, 2, 3, 0)  # [H, W, D, C] views of the channels-last memory
    out = torch.zeros(3, 3, 3, c, dtype=torch.float64, device=x.device)
    for h0 in range(0, H, rows):
        h1 = min(h0 + rows, H)
        g64 = gv[h0:h1].double()
        xa, xb = max(h0 - 1, 0), min(h1 + 1, H)
        x64 = xv[xa:xb].double()
        for kh in range(3):
            # planes of g in [h0, h1) whose partner plane h + kh - 1 exists
            ga, gb = max(h0, 1 - kh), min(h1, H + 1 - kh)
            if ga >= gb:
                continue
            gs = g64[ga - h0:gb - h0]
            xs = x64[ga + kh - 1 - xa:gb + kh - 1 - xa]
            for kw in range(3):
                gw_, xw_ = box(W, kw)
                for kd in range(3):
                    gd_, xd_ = box(D, kd)
                    out[kh, kw, kd] += (gs[:, gw_, gd_] * xs[:, xw_, xd_]).sum(dim=(0, 1, 2))
    return out


def check_gw(gw, ref, what):
    gw = gw.double()
    rel = ((gw - ref).norm() / ref.norm()).item()
    assert rel <= 1e-5, (what, rel)
    # per tap and channel: relative error 1e-4, with a floor for taps whose sum happens to fall near zero
    floor = 1e-5 * ref.pow(2).mean().sqrt().item()
    worst = ((gw - ref).abs() / (ref.abs() + floor / 1e-4)).max().item()
    assert worst <= 1e-4, (what, worst)


def test_restatements_agree_with_the_oracle():
    """CPU: the two torch restatements used below, on a shape with chunk borders inside the volume, against the
    oracle (which tests/test_oracle_pin.py pins to torch's conv3d and its autograd)."""
    import oracle
    from conftest import rand_cl3d
    gen = cpu_gen(5)
    x, g = rand_cl3d(gen, 1, 8, 23, 6, 9), rand_cl3d(gen, 1, 8, 23, 6, 9)
    _, wk = rand_dw_weight(gen, 8)
    ref = oracle.dwconv_wgrad(x, g)
    assert torch.allclose(wgrad_by_sliced_dots(x, g, rows=10), ref, rtol=1e-12, atol=1e-9)
    _, ref32 = oracle.dwconv_fwd(x, wk, wide=True, return_fp32=True)
    got = forward_by_shifted_products(x, wk, rows=10).permute(3, 0, 1, 2).unsqueeze(0)
    assert torch.allclose(got, ref32, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
def test_full_shape_weight_gradient_every_tap(c):
    x, g = make(c)
    ref = wgrad_by_sliced_dots(x, g)
    check_gw(DWConvWGRAD(x, g, out_dtype=torch.float32), ref, 'DWConvWGRAD')
    # the drop-in result type: one fp16 rounding of the fp32 sums (|gw| stays far below the fp16 maximum here)
    gw16 = DWConvWGRAD(x, g)
    assert gw16.dtype == torch.float16
    assert torch.allclose(gw16.double(), ref, rtol=2.0 ** -10, atol=1e-2)
    # the other built kernel families sum in other orders: same bound
    check_gw(DWConvWGRAD(x, g, lane_channels=16, W_block=8, D_block={8: 32, 16: 16, 32: 16}.get(c, 8),
                         out_dtype=torch.float32), ref, 'register-staged matrix-core kernel')
    _, wk = rand_dw_weight(cpu_gen(), c)
    dx, gw_b = DWConvBackward(x, g, wk.to(DEV), out_dtype=torch.float32)
    check_gw(gw_b, ref, 'DWConvBackward')
    # its input gradient is the forward kernel's arithmetic on (g, flipped weight): bit-identical
    assert torch.equal(dx, DWConv(g, torch.flip(wk, dims=(0, 1, 2)).contiguous().to(DEV)))


def forward_by_shifted_products(x, wk, rows=25):
    """fp32 [H, W, D, C]: sum over the 27 taps of the shifted input times the tap's weight vector, chunked over H."""
    _, c, H, W, D = x.shape
    xv = x[0].permute(1, 2, 3, 0)
    w32 = wk.float()
    out = torch.empty(H, W, D, c, dtype=torch.float32, device=x.device)
    for h0 in range(0, H, rows):
        h1 = min(h0 + rows, H)
        xa, xb = max(h0 - 1, 0), min(h1 + 1, H)
        x32 = xv[xa:xb].float()
        acc = torch.zeros(h1 - h0, W, D, c, dtype=torch.float32, device=x.device)
        for kh in range(3):
            ya, yb = max(h0, 1 - kh), min(h1, H + 1 - kh)  # output planes whose input plane y + kh - 1 exists
            if ya >= yb:
                continue
            xs = x32[ya + kh - 1 - xa:yb + kh - 1 - xa]
            for kw in range(3):
                yw, xw = box(W, kw)
                for kd in range(3):
                    yd, xd = box(D, kd)
                    acc[ya - h0:yb - h0, yw, yd] += xs[:, xw, xd] * w32[kh, kw, kd]
        out[h0:h1] = acc
    return out


@pytest.mark.gpu
@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
def test_full_shape_forward_every_voxel(c):
    x, _ = make(c, seed=7)
    _, wk = rand_dw_weight(cpu_gen(), c)
    wd = wk.to(DEV)
    y = DWConv(x, wd)
    ref32 = forward_by_shifted_products(x, wd)
    yv = y[0].permute(1, 2, 3, 0)
    assert torch.allclose(yv.float(), ref32, rtol=1e-2, atol=1e-2)  # the tolerance stated for the README-shape forward
    # both sides add the same 27 fp32 products (in different orders) and the kernel rounds once to fp16: the
    # difference stays within one fp16 step of the sum
    err = (yv.float() - ref32).abs()
    bound = 2.0 ** -10 * ref32.abs() + 4e-6  # (27 fp32 additions in another order: a few 2^-24 of the largest term)
    assert bool((err <= bound).all()), (err / bound).max().item()
    del err, bound
    same = (yv == ref32.half()).float().mean().item()
    assert same >= 0.998, same
    if c == 64:
        # torch's own depthwise conv3d on the GPU under the reference's criterion (its tests compare with exactly
        # this call, tests/ops/test_conv.py:25-36)
        wt = wk.permute(3, 0, 1, 2).unsqueeze(1).contiguous().to(DEV)
        ref16 = torch.nn.functional.conv3d(x, wt, None, stride=1, padding=1, groups=c)
        assert ref16.dtype == torch.float16 and ref16.shape == y.shape
        assert allclose_two_stage(y, ref16, rtol_strict=1e-4, atol_strict=1e-3, percentile_strict=0.99,
                                  rtol_narrow=1e-3, atol_narrow=2e-3)
