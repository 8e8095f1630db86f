"""GPU parity tests of the pointwise MFMA kernel, the ReLULinearAdd drop-in and the fused
depthwise-separable block with its int8 output (the fused-block target configuration: x (1,64,128,128,128), 64 -> 128 channels)."""
import math

import pytest
import torch
from torch.nn import functional as F

import oracle
from conftest import cpu_gen, rand_cl3d, rand_dw_weight
from kerops_amd.ops.fused import DWSepBlock, DWSepBlockInt8, PointwiseLinear
from kerops_amd.ops.bnrelu import ApplyBNReLU
from kerops_amd.ops.linear import (ApplyBNReLULinearAdd, LinBReLULinAdd, LinBReLULinBackward, ReLULinearAdd,
                               ReLULinearBackward)
from kerops_amd.utils import allclose_two_stage, weight_grad_similarity

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def rand_pw(g, cin, cout):
    return (torch.randn(cin, cout, generator=g) / math.sqrt(cin)).half()


@pytest.mark.parametrize('cin,cout', [(16, 16), (16, 32), (32, 16), (32, 32), (64, 64), (64, 128), (128, 128),
                                      (128, 32), (16, 128)])
@pytest.mark.parametrize('spatial', [(1, 3, 5, 7), (2, 4, 4, 4), (1, 1, 1, 1), (3, 2, 13, 37)])
def test_relu_linear_add_matches_oracle(cin, cout, spatial):
    g = cpu_gen(cin * 1000 + cout)
    n, h, w, d = spatial
    x = rand_cl3d(g, n, cin, h, w, d)
    add = rand_cl3d(g, n, cout, h, w, d)
    Wm = rand_pw(g, cin, cout)
    out = ReLULinearAdd(x.to(DEV), Wm.to(DEV), add.to(DEV)).cpu()
    ref = oracle.pointwise(x, Wm, add=add, relu_in=True)
    assert out.shape == add.shape and out.stride() == add.stride()
    # fp32 MFMA accumulation vs the oracle's fp64: at most one fp16 rounding apart before the add
    assert allclose_two_stage(ref.contiguous(), out.contiguous(), rtol_strict=1e-4, atol_strict=1e-3,
                              rtol_narrow=1e-3, atol_narrow=2e-3)
    assert (out.float() - ref.float()).abs().max() <= 2.0 ** -9 * max(1.0, ref.abs().max().item())
    same = (out.contiguous().view(torch.int16) == ref.contiguous().view(torch.int16)).float().mean().item()
    assert same > 0.99, same
    # the reference's own ground truth: 1x1x1 conv3d of relu(x) plus the residual
    conv = F.conv3d(F.relu(x.float()), Wm.float().t().reshape(cout, cin, 1, 1, 1)).half() + add
    assert torch.allclose(out.float(), conv.float(), rtol=1e-3, atol=2e-3)


@pytest.mark.parametrize('cin,cout', [(16, 16), (32, 32), (32, 16), (64, 128), (128, 64), (16, 128)])
@pytest.mark.parametrize('spatial', [(1, 3, 5, 7), (2, 4, 4, 4), (1, 1, 1, 1), (3, 5, 13, 37)])
def test_bnrelu_linear_add_equals_composition(cin, cout, spatial):
    g = cpu_gen(cin * 7 + cout)
    n, h, w, d = spatial
    x = rand_cl3d(g, n, cin, h, w, d) * 2 + 0.3
    add = rand_cl3d(g, n, cout, h, w, d)
    Wm = rand_pw(g, cin, cout)
    bw = torch.rand(cin, generator=g) + 0.5
    bb = torch.randn(cin, generator=g) * 0.5
    dev = [t_.to(DEV) for t_ in (x, bw, bb, Wm, add)]
    fused = ApplyBNReLULinearAdd(*dev)
    composed = ReLULinearAdd(ApplyBNReLU(dev[0], dev[1], dev[2]), dev[3], dev[4])
    assert fused.shape == add.shape and fused.stride() == add.stride()
    assert torch.equal(fused.view(torch.int16), composed.view(torch.int16))  # bit for bit
    ref = oracle.pointwise(oracle.bnrelu_fwd(x, bw, bb), Wm, add=add, relu_in=True)
    # fp32 MFMA sums against the oracle's fp64: one fp16 rounding of the product apart before the residual add
    assert (fused.cpu().float() - ref.float()).abs().max() <= 2.0 ** -9 * max(1.0, ref.abs().max().item())


@pytest.mark.parametrize('cin,cout', [(16, 16), (16, 32), (32, 16), (32, 32), (32, 64), (64, 64), (64, 128),
                                      (128, 128), (128, 32), (16, 128), (128, 16), (64, 16)])
@pytest.mark.parametrize('spatial', [(1, 3, 5, 7), (2, 4, 4, 4), (1, 1, 1, 1), (3, 5, 13, 37)])
def test_relu_linear_backward_matches_oracle(cin, cout, spatial):
    g = cpu_gen(cin * 1000 + cout + 1)
    n, h, w, d = spatial
    x = rand_cl3d(g, n, cin, h, w, d)
    grad = rand_cl3d(g, n, cout, h, w, d)
    Wm = rand_pw(g, cin, cout)
    dx, dw = ReLULinearBackward(x.to(DEV), grad.to(DEV), Wm.to(DEV), out_dtype=torch.float32)
    # default result type fp16, written by the reduction kernel = the fp32 result rounded once; same dx
    dx16, dw16 = ReLULinearBackward(x.to(DEV), grad.to(DEV), Wm.to(DEV))
    assert dw16.dtype == torch.float16 and torch.equal(dx16, dx)
    assert torch.equal(dw16.view(torch.int16), dw.to(torch.float16).view(torch.int16))
    dx, dw = dx.cpu(), dw.cpu()
    ref_dx, ref_dw = oracle.relu_linear_bwd(x, grad, Wm)
    assert dx.shape == x.shape and dx.stride() == x.stride() and dw.shape == (cin, cout)
    # the mask is exact; the values are fp32 MFMA sums vs the oracle's fp64, one rounding to fp16 each
    assert torch.equal(dx == 0, ref_dx == 0) or ((dx == 0) != (ref_dx == 0)).float().mean() < 1e-3
    assert torch.equal(dx[x <= 0], torch.zeros_like(dx[x <= 0]))
    assert (dx.float() - ref_dx.float()).abs().max() <= 2.0 ** -9 * max(1.0, ref_dx.abs().max().item())
    same = (dx.contiguous().view(torch.int16) == ref_dx.contiguous().view(torch.int16)).float().mean().item()
    assert same > 0.99, same
    rel = ((dw.double() - ref_dw).norm() / max(ref_dw.norm().item(), 1e-30)).item()
    assert rel < 2e-6, rel
    # the reference's own criteria (tests/ops/test_linear.py:60-78)
    assert allclose_two_stage(ref_dx.contiguous(), dx.contiguous(), rtol_strict=1e-4, atol_strict=1e-4,
                              rtol_narrow=1e-3, atol_narrow=1e-3)
    if ref_dw.norm() > 0:
        assert weight_grad_similarity(ref_dw.float(), dw, rtol_cos=1e-4, atol_cos=1e-4, rtol_len=1e-3, atol_len=1e-3)


def test_relu_linear_backward_default_dtype_determinism_and_large():
    g = cpu_gen(77)
    x = rand_cl3d(g, 2, 32, 37, 53, 16)   # V = 62 752: many tiles per workgroup, ragged last tile
    grad = rand_cl3d(g, 2, 16, 37, 53, 16)
    Wm = rand_pw(g, 32, 16)
    xd, gd, wd = x.to(DEV), grad.to(DEV), Wm.to(DEV)
    dx1, dw1 = ReLULinearBackward(xd, gd, wd)
    dx2, dw2 = ReLULinearBackward(xd, gd, wd)
    assert dw1.dtype == torch.float16 and dx1.dtype == torch.float16
    assert torch.equal(dx1, dx2) and torch.equal(dw1, dw2)  # no atomics: bit-reproducible
    ref_dx, ref_dw = oracle.relu_linear_bwd(x, grad, Wm)
    same = (dx1.cpu().contiguous().view(torch.int16) == ref_dx.contiguous().view(torch.int16)).float().mean().item()
    assert same > 0.99, same
    _, dw32 = ReLULinearBackward(xd, gd, wd, out_dtype=torch.float32)
    assert ((dw32.cpu().double() - ref_dw).norm() / ref_dw.norm()).item() < 2e-6
    with pytest.raises(AssertionError):
        ReLULinearBackward(xd, gd, wd.t().contiguous())


@pytest.mark.parametrize('c', [16, 32, 64])
@pytest.mark.parametrize('spatial', [(1, 3, 5, 7), (2, 4, 4, 4), (1, 1, 1, 1), (3, 5, 13, 37), (1, 37, 53, 16)])
def test_lin_brelu_lin_add_matches_oracle(c, spatial):
    g = cpu_gen(c * 77 + spatial[1])
    n, h, w, d = spatial
    x, add = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    Wup, Wdown = rand_pw(g, c, 2 * c), rand_pw(g, 2 * c, c)
    bias = (torch.randn(2 * c, generator=g) * 0.5).half()
    out = LinBReLULinAdd(x.to(DEV), Wup.to(DEV), Wdown.to(DEV), bias.to(DEV), add.to(DEV)).cpu()
    ref = oracle.lin_brelu_lin_add(x, Wup, Wdown, bias, add)
    assert out.shape == x.shape and out.stride() == x.stride()
    # fp32 MFMA sums vs the oracle's fp64: a hidden value may round differently once in a while
    assert allclose_two_stage(ref.contiguous(), out.contiguous(), rtol_strict=1e-4, atol_strict=5e-4,
                              rtol_narrow=1e-3, atol_narrow=2e-3)
    assert (out.float() - ref.float()).abs().max() <= 2.0 ** -8 * max(1.0, ref.abs().max().item())
    same = (out.contiguous().view(torch.int16) == ref.contiguous().view(torch.int16)).float().mean().item()
    assert same > 0.98, same
    # the reference's own ground truth (tests/ops/test_linear.py:101-116)
    base = F.conv3d(x.float(), Wup.float().t().reshape(2 * c, c, 1, 1, 1), bias.float())
    base = F.conv3d(F.relu(base), Wdown.float().t().reshape(c, 2 * c, 1, 1, 1)) + add.float()
    assert allclose_two_stage(base.half().contiguous(), out.contiguous(), rtol_strict=1e-4, atol_strict=5e-4,
                              rtol_narrow=1e-3, atol_narrow=2e-3) or torch.allclose(out.float(), base, rtol=2e-3,
                                                                                    atol=4e-3)


def test_lin_brelu_lin_add_closed_form_and_contract():
    g = cpu_gen(31)
    c = 32
    x, add = rand_cl3d(g, 1, c, 5, 6, 7), rand_cl3d(g, 1, c, 5, 6, 7)
    eye_up = torch.cat([torch.eye(c), torch.zeros(c, c)], 1).half()
    eye_dn = torch.cat([torch.eye(c), torch.zeros(c, c)], 0).half()
    zero_b = torch.zeros(2 * c, dtype=torch.float16)
    out = LinBReLULinAdd(x.to(DEV), eye_up.to(DEV), eye_dn.to(DEV), zero_b.to(DEV), add.to(DEV)).cpu()
    assert torch.equal(out, (F.relu(x).float() + add.float()).half())  # one nonzero product per sum: exact
    with pytest.raises(AssertionError):
        LinBReLULinAdd(x.to(DEV), eye_dn.to(DEV), eye_up.to(DEV), zero_b.to(DEV), add.to(DEV))
    from kerops_amd.settings import CongiguratorError
    x128 = rand_cl3d(g, 1, 128, 2, 2, 2)
    with pytest.raises(CongiguratorError):
        LinBReLULinAdd(x128.to(DEV), rand_pw(g, 128, 256).to(DEV), rand_pw(g, 256, 128).to(DEV),
                       torch.zeros(256, dtype=torch.float16, device=DEV), x128.to(DEV))


@pytest.mark.parametrize('c', [16, 32, 64])
@pytest.mark.parametrize('spatial', [(1, 3, 5, 7), (2, 4, 4, 4), (1, 1, 1, 1), (3, 5, 13, 37), (1, 37, 53, 16)])
def test_lin_brelu_lin_backward_matches_oracle(c, spatial):
    g = cpu_gen(c * 91 + spatial[1])
    n, h, w, d = spatial
    x, grad = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    Wup, Wdown = rand_pw(g, c, 2 * c), rand_pw(g, 2 * c, c)
    bias = (torch.randn(2 * c, generator=g) * 0.5).half()
    dev = [t_.to(DEV) for t_ in (x, grad, Wup, Wdown, bias)]
    dx, dup, ddn, db = (t_.cpu() for t_ in LinBReLULinBackward(*dev, out_dtype=torch.float32))
    # default result type fp16, written by the reduction kernel = the fp32 results rounded once; same dx
    got16 = [t_.cpu() for t_ in LinBReLULinBackward(*dev)]
    assert torch.equal(got16[0], dx)
    for h16, f32 in zip(got16[1:], (dup, ddn, db)):
        assert h16.dtype == torch.float16 and h16.shape == f32.shape
        assert torch.equal(h16.view(torch.int16), f32.to(torch.float16).view(torch.int16))
    rdx, rup, rdn, rdb = oracle.lin_brelu_lin_bwd(x, grad, Wup, Wdown, bias)
    assert dx.shape == x.shape and dx.stride() == x.stride()
    assert dup.shape == (c, 2 * c) and ddn.shape == (2 * c, c) and db.shape == (2 * c,)
    # fp32 MFMA sums vs the oracle's fp64: an intermediate fp16 value may round differently once in a while, and where
    # a hidden pre-activation lies within a rounding of zero its ReLU mask may flip.  The reference's test rechecks
    # such voxels by hand (tests/ops/test_linear.py:203-219); here the error a flip can cause is bounded per voxel:
    # sum over the hidden units next to zero of |Wdown g|_j * |Wup[ci, j]|.
    x2, g2 = (t_.permute(0, 2, 3, 4, 1).reshape(-1, c).double() for t_ in (x, grad))
    up64 = x2 @ Wup.double()
    linup = up64 + bias.double()
    # the pre-activation is fp16(up) + bias (exact next to zero); its sign can only differ from the oracle's where it
    # lies within one fp16 step of the product: 2^-10 |up| covers the step of every binade
    near = (linup.abs() <= 2.0 ** -10 * up64.abs() + 1e-7).double()
    flip_bound = ((near * (g2 @ Wdown.double().t()).abs()) @ Wup.double().abs().t()).float()
    flip_bound = flip_bound.reshape(n, h, w, d, c).permute(0, 4, 1, 2, 3)
    err = (dx.float() - rdx.float()).abs()
    assert (err <= 2.0 ** -7 * max(1.0, rdx.abs().max().item()) + 1.01 * flip_bound).all()
    kink = (near.sum(dim=1) > 0).reshape(n, 1, h, w, d).expand_as(dx)
    # 2c hidden units per voxel, each within a step of zero with probability of a few 1e-4
    if n * h * w * d >= 500:
        assert kink.float().mean().item() <= 0.08, kink.float().mean().item()
    same = (dx.contiguous().view(torch.int16) == rdx.contiguous().view(torch.int16)).float().mean().item()
    assert same > 0.97, same
    for got, ref in ((dup, rup), (ddn, rdn), (db, rdb)):
        rel = ((got.double() - ref).norm() / max(ref.norm().item(), 1e-30)).item()
        assert rel < 1e-3, rel
    # the reference's own criteria (tests/ops/test_linear.py:153-200)
    assert weight_grad_similarity(rdn.float(), ddn, rtol_cos=1e-4, atol_cos=1e-4, rtol_len=1e-3, atol_len=1e-3)
    assert weight_grad_similarity(rup.float(), dup, rtol_cos=1e-4, atol_cos=1e-4, rtol_len=2e-3, atol_len=1e-3)
    assert weight_grad_similarity(rdb.float(), db, rtol_cos=1e-3, atol_cos=1e-3, rtol_len=2e-3, atol_len=1e-3)
    keep = (~kink).to(dx.dtype)  # voxels away from every kink: the reference's criterion without its manual recheck
    assert allclose_two_stage((rdx * keep).contiguous(), (dx * keep).contiguous(), rtol_strict=1e-4, atol_strict=1e-3,
                              rtol_narrow=1e-3, atol_narrow=4e-3)


@pytest.mark.parametrize('c', [16, 32])
def test_lin_brelu_lin_backward_several_tiles_per_wavefront(c):
    # more 32-voxel tiles than resident wavefronts, ragged end: the loop-carried prefetch, the store of a tile
    # one iteration late and the accumulation over tiles are all on the path
    g = cpu_gen(1000 + c)
    n, h, w, d = 1, 61, 67, 29
    x, grad = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    Wup, Wdown = rand_pw(g, c, 2 * c), rand_pw(g, 2 * c, c)
    bias = (torch.randn(2 * c, generator=g) * 0.5).half()
    dev = [t_.to(DEV) for t_ in (x, grad, Wup, Wdown, bias)]
    dx, dup, ddn, db = (t_.cpu() for t_ in LinBReLULinBackward(*dev, out_dtype=torch.float32))
    rdx, rup, rdn, rdb = oracle.lin_brelu_lin_bwd(x, grad, Wup, Wdown, bias)
    assert (dx.float() - rdx.float()).abs().max() <= 2.0 ** -7 * max(1.0, rdx.abs().max().item())
    same = (dx.contiguous().view(torch.int16) == rdx.contiguous().view(torch.int16)).float().mean().item()
    assert same > 0.97, same
    for got, ref in ((dup, rup), (ddn, rdn), (db, rdb)):
        rel = ((got.double() - ref).norm() / max(ref.norm().item(), 1e-30)).item()
        assert rel < 1e-3, rel


@pytest.mark.parametrize('c', [16, 32, 64])
def test_lin_brelu_lin_backward_mask_at_zero(c):
    # linup == 0 exactly (x = 0, bias = +0 or -0) must not pass the gradient, a positive bias must
    g = cpu_gen(7 + c)
    n, h, w, d = 1, 5, 6, 7
    x = torch.zeros(n, c, h, w, d, dtype=torch.float16).contiguous(memory_format=torch.channels_last_3d)
    grad = rand_cl3d(g, n, c, h, w, d)
    Wup, Wdown = rand_pw(g, c, 2 * c), rand_pw(g, 2 * c, c)
    bias = torch.zeros(2 * c, dtype=torch.float16)
    bias[1::4] = -0.0
    bias[2::4] = 0.25
    bias[3::4] = -0.25
    dev = [t_.to(DEV) for t_ in (x, grad, Wup, Wdown, bias)]
    dx, dup, ddn, db = (t_.cpu() for t_ in LinBReLULinBackward(*dev, out_dtype=torch.float32))
    rdx, rup, rdn, rdb = oracle.lin_brelu_lin_bwd(x, grad, Wup, Wdown, bias)
    assert torch.all(db[0::4] == 0) and torch.all(db[1::4] == 0) and torch.all(db[3::4] == 0)
    assert torch.all(db[2::4] != 0)
    assert torch.all(dup == 0)  # x = 0
    assert torch.all(ddn[0::4] == 0) and torch.all(ddn[1::4] == 0) and torch.all(ddn[3::4] == 0)
    for got, ref in ((ddn, rdn), (db, rdb)):
        assert ((got.double() - ref).norm() / ref.norm()).item() < 1e-3
    assert (dx.float() - rdx.float()).abs().max() <= 2.0 ** -7 * max(1.0, rdx.abs().max().item())


def _spatial_sample(n, seed, max_voxels=200_000):
    """Deterministic sample of the spatial grid of the reference's linear tests (tests/conftest.py:14-36)."""
    import random
    rng = random.Random(seed)
    extents = [2, 3, 7, 13, 16, 32, 37, 53, 111, 128]
    out = []
    while len(out) < n:
        sp = (rng.choice([1, 2, 3, 4]), rng.choice(extents), rng.choice(extents), rng.choice(extents))
        if sp[0] * sp[1] * sp[2] * sp[3] <= max_voxels and sp not in out:
            out.append(sp)
    return out


# batch 4 with the largest extents of the reference's grid, listed because a bounded random sample rarely holds them
FORCED_SPATIAL = [(4, 111, 128, 2), (4, 128, 111, 3), (4, 2, 111, 128), (4, 3, 128, 111), (4, 128, 2, 111),
                  (4, 128, 128, 2)]


@pytest.mark.parametrize('spatial', _spatial_sample(250, seed=322) + FORCED_SPATIAL)
@pytest.mark.parametrize('cout', [16, 32])
def test_linear_family_on_reference_fixture_grid_sample(cout, spatial):
    # the reference's parameters: 32 input channels, channels_out in {16, 32} (tests/ops/test_linear.py:11-78) and
    # channels in {16, 32} for the bottleneck block (:81-200)
    test_relu_linear_add_matches_oracle(32, cout, spatial)
    test_relu_linear_backward_matches_oracle(32, cout, spatial)
    test_lin_brelu_lin_add_matches_oracle(cout, spatial)
    test_lin_brelu_lin_backward_matches_oracle(cout, spatial)


def test_lin_brelu_lin_backward_defaults_and_determinism():
    g = cpu_gen(41)
    c = 32
    x, grad = rand_cl3d(g, 2, c, 37, 53, 16), rand_cl3d(g, 2, c, 37, 53, 16)
    Wup, Wdown = rand_pw(g, c, 2 * c), rand_pw(g, 2 * c, c)
    bias = (torch.randn(2 * c, generator=g) * 0.5).half()
    dev = [t_.to(DEV) for t_ in (x, grad, Wup, Wdown, bias)]
    r1 = LinBReLULinBackward(*dev)
    r2 = LinBReLULinBackward(*dev)
    assert all(t_.dtype == torch.float16 for t_ in r1)
    assert all(torch.equal(a_, b_) for a_, b_ in zip(r1, r2))  # no atomics: bit-reproducible
    rdx, rup, rdn, rdb = oracle.lin_brelu_lin_bwd(x, grad, Wup, Wdown, bias)
    got = LinBReLULinBackward(*dev, out_dtype=torch.float32)
    for a_, b_ in zip(got[1:], (rup, rdn, rdb)):
        assert ((a_.cpu().double() - b_).norm() / b_.norm()).item() < 1e-3
    with pytest.raises(AssertionError):
        LinBReLULinBackward(dev[0], dev[1], dev[3], dev[2], dev[4])


def test_pointwise_identity_and_no_relu():
    g = cpu_gen(5)
    x = rand_cl3d(g, 1, 64, 5, 6, 7)
    eye = torch.eye(64, dtype=torch.float16)
    y = PointwiseLinear(x.to(DEV), eye.to(DEV)).cpu()
    assert torch.equal(y, x)  # exact: one nonzero product per output
    y = PointwiseLinear(x.to(DEV), eye.to(DEV), relu_in=True).cpu()
    assert torch.equal(y, F.relu(x))
    perm = torch.randperm(64, generator=g)
    P = torch.zeros(64, 64, dtype=torch.float16)
    P[torch.arange(64), perm] = 1.0  # out[:, perm[i]] = x[:, i]
    y = PointwiseLinear(x.to(DEV), P.to(DEV)).cpu()
    assert torch.equal(y[:, perm], x)


@pytest.mark.parametrize('shape', [(1, 64, 9, 11, 13), (2, 64, 3, 17, 8), (1, 64, 16, 16, 16)])
@pytest.mark.parametrize('cout', [128, 32])
def test_dwsep_block_matches_oracle(shape, cout):
    g = cpu_gen(31)
    x = rand_cl3d(g, *shape)
    _, wk = rand_dw_weight(g, 64)
    scale = torch.rand(64, generator=g) + 0.5
    shift = torch.randn(64, generator=g) * math.sqrt(0.1)
    Wm = rand_pw(g, 64, cout)
    y, amax = DWSepBlock(x.to(DEV), wk.to(DEV), scale.to(DEV), shift.to(DEV), Wm.to(DEV))
    ref = oracle.dwsep_block(x, wk, scale, shift, Wm)
    assert torch.allclose(y.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)  # config 5 tolerance
    assert (y.cpu().float() - ref.float()).abs().max() <= 2.0 ** -8 * max(1.0, ref.abs().max().item())
    assert amax.item() == y.abs().max().item()
    q, qscale, y2 = DWSepBlockInt8(x.to(DEV), wk.to(DEV), scale.to(DEV), shift.to(DEV), Wm.to(DEV))
    assert torch.equal(y2, y)
    # int8 bit-exact given the identical pre-quant tensor
    assert torch.equal(q.cpu(), oracle.quant_i8_sym(y.cpu(), amax.item()))
    assert qscale.item() == torch.tensor(amax.item(), dtype=torch.float32).div(127.0).item()


@pytest.mark.parametrize('cout', [128, 32])
def test_dwsep_block_noncontiguous_weights(cout):
    """Both weights handed over as non-contiguous views (the torch (C,1,3,3,3) layout permuted, a transposed linear
    weight): the op's contiguous copies must stay alive until the launch, the result equals the contiguous call."""
    g = cpu_gen(77)
    x = rand_cl3d(g, 1, 64, 6, 9, 10).to(DEV)
    wt, wk = rand_dw_weight(g, 64)
    scale = (torch.rand(64, generator=g) + 0.5).to(DEV)
    shift = (torch.randn(64, generator=g) * math.sqrt(0.1)).to(DEV)
    Wm = rand_pw(g, 64, cout)
    dw_view = wt.to(DEV)[:, 0].permute(1, 2, 3, 0)
    pw_view = Wm.t().contiguous().to(DEV).t()
    assert not dw_view.is_contiguous() and not pw_view.is_contiguous()
    y0, a0 = DWSepBlock(x, wk.to(DEV), scale, shift, Wm.to(DEV))
    for _ in range(3):
        y1, a1 = DWSepBlock(x, dw_view, scale, shift, pw_view)
        assert torch.equal(y1, y0) and a1.item() == a0.item()
    p0 = PointwiseLinear(x, Wm.to(DEV))
    assert torch.equal(PointwiseLinear(x, pw_view), p0)


def test_config5_full_shape():
    """(1,64,128,128,128) -> y (1,128,128,128,128) -> int8: slab comparison with the oracle,
    absmax against torch, int8 against the closed form on the build's own y."""
    gen = torch.Generator(DEV).manual_seed(322)
    x = torch.randn(1, 128, 128, 128, 64, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    g = cpu_gen()
    _, wk = rand_dw_weight(g, 64)
    scale = torch.rand(64, generator=g) + 0.5
    shift = torch.randn(64, generator=g) * math.sqrt(0.1)
    Wm = (torch.randn(64, 128, generator=g) / 8.0).half()
    q, qscale, y = DWSepBlockInt8(x, wk.to(DEV), scale.to(DEV), shift.to(DEV), Wm.to(DEV))
    assert list(y.shape) == [1, 128, 128, 128, 128] and q.dtype == torch.int8
    amax = y.abs().max().float()
    assert qscale.item() == (amax / 127.0).item()
    for (h0, h1) in [(0, 5), (61, 66), (123, 128)]:
        ha, hb = max(h0 - 1, 0), min(h1 + 1, 128)
        xs = x[:, :, ha:hb].cpu().contiguous(memory_format=torch.channels_last_3d)
        ref = oracle.dwsep_block(xs, wk, scale, shift, Wm)[:, :, h0 - ha:h0 - ha + h1 - h0]
        assert torch.allclose(y[:, :, h0:h1].cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
    ys = y[:, :, 40:44].cpu()
    assert torch.equal(q[:, :, 40:44].cpu(), oracle.quant_i8_sym(ys, amax.item()))
    # every element: the closed form rint(fp32(y / scale)) with the quotient taken in fp64 and rounded once to fp32
    # (the library's quotient is the correctly rounded fp32 quotient; a double rounding could only matter for a
    # quotient within 2^-29 of a fp32 midpoint that is also within one fp32 step of a tie of rint), and torch's own
    # fp32 division by the same scale, which is correctly rounded as well: both bit for bit
    ref_q = torch.empty_like(q)
    for h0 in range(0, 128, 32):
        ys = y[:, :, h0:h0 + 32]
        ref_q[:, :, h0:h0 + 32] = torch.round((ys.double() / qscale.double()).float()).clamp(-127, 127).to(torch.int8)
    assert torch.equal(ref_q, q)
    assert torch.equal(torch.round(y.float() / qscale).clamp(-127, 127).to(torch.int8), q)
