"""GPU tests of the autograd.Function wrappers: gradients of a small depthwise block through the
HIP ops against torch autograd of the same mathematics in fp32."""
import math

import pytest
import torch
from torch.nn import functional as F

import oracle
from conftest import cpu_gen, rand_cl3d, rand_dw_weight
from kerops_amd.autograd import (AddStatsFn, ApplyBNReLUFn, ApplyBNReLULinearAddFn, AvgPoolCeilStatsFn, DWConvFn,
                                 DWConvStatsFn, ReLULinearAddFn, StatsFn)
from kerops_amd.utils import allclose_two_stage, weight_grad_similarity

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.mark.parametrize('shape', [(1, 8, 5, 6, 7), (2, 64, 9, 4, 13), (1, 32, 3, 3, 3)])
def test_dwconv_input_and_weight_gradients(shape):
    g = cpu_gen(41)
    c = shape[1]
    x = rand_cl3d(g, *shape)
    go = rand_cl3d(g, *shape)
    wt, wk = rand_dw_weight(g, c)
    xd = x.to(DEV).requires_grad_(True)
    wd = wk.to(DEV).requires_grad_(True)
    y = DWConvFn.apply(xd, wd)
    y.backward(go.to(DEV))
    # reference: fp64 autograd on the CPU
    x64 = x.double().requires_grad_(True)
    w64 = wt.double().requires_grad_(True)
    F.conv3d(x64, w64, None, 1, 1, 1, c).backward(go.double())
    ref_gx = x64.grad
    ref_gw = w64.grad[:, 0].permute(1, 2, 3, 0)
    assert xd.grad.dtype == torch.float16 and xd.grad.shape == x.shape
    assert (xd.grad.cpu().double() - ref_gx).abs().max() <= 2.0 ** -10 * max(1.0, ref_gx.abs().max().item())
    # input gradient = forward kernel on the flipped weight: check it against the oracle too
    flipped = torch.flip(wk, dims=(0, 1, 2)).contiguous()
    _, gx32 = oracle.dwconv_fwd(go, flipped, wide=True, return_fp32=True)
    assert torch.allclose(gx32.double(), ref_gx, rtol=1e-5, atol=1e-5)
    assert weight_grad_similarity(ref_gw.float(), wd.grad.cpu().float(), rtol_len=2e-3, atol_len=1e-2)


def test_block_gradients_against_torch_autograd():
    g = cpu_gen(43)
    n, c, h, w, d = 2, 16, 7, 6, 9
    x, r = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    wt, wk = rand_dw_weight(g, c)
    gamma = torch.rand(c, generator=g) + 0.5
    beta = torch.randn(c, generator=g) * 0.3
    up = torch.randn(n, c, 4, 3, 5, generator=g)

    def run(mod):
        xd = x.to(DEV).requires_grad_(True)
        wd = wk.to(DEV).requires_grad_(True)
        gd = gamma.to(DEV).requires_grad_(True)
        bd = beta.to(DEV).requires_grad_(True)
        if mod == 'hip':
            y = DWConvFn.apply(xd, wd)
            z, mean, sq = AddStatsFn.apply(y, r.to(DEV))
            rv = torch.rsqrt(sq - mean ** 2 + 1e-5)
            a = ApplyBNReLUFn.apply(z, gd * rv, bd - mean * rv * gd)
            p, pm, ps = AvgPoolCeilStatsFn.apply(a)
            loss = (p.float() * up.to(DEV)).sum() + pm.sum() + 0.5 * ps.sum()
        else:
            wfull = wd.float().permute(3, 0, 1, 2)[:, None]
            y = F.conv3d(xd.float(), wfull, None, 1, 1, 1, c)
            z = y + r.to(DEV).float()
            mean, sq = z.mean(dim=(0, 2, 3, 4)), (z * z).mean(dim=(0, 2, 3, 4))
            rv = torch.rsqrt(sq - mean ** 2 + 1e-5)
            a = F.relu(z * (gd * rv).view(1, c, 1, 1, 1) + (bd - mean * rv * gd).view(1, c, 1, 1, 1))
            p = F.avg_pool3d(a, 2, ceil_mode=True)
            loss = (p * up.to(DEV)).sum() + p.mean(dim=(0, 2, 3, 4)).sum() + 0.5 * (p * p).mean(dim=(0, 2, 3, 4)).sum()
        loss.backward()
        return loss.item(), xd.grad.float().cpu(), wd.grad.float().cpu(), gd.grad.cpu(), bd.grad.cpu()

    lh, gxh, gwh, ggh, gbh = run('hip')
    lt, gxt, gwt, ggt, gbt = run('torch')
    assert abs(lh - lt) <= 2e-3 * abs(lt) + 1e-2
    # fp16 tensors between the ops limit the agreement; direction and size of every gradient must match
    for a, b in ((gxh, gxt), (gwh, gwt), (ggh, ggt), (gbh, gbt)):
        cos = F.cosine_similarity(a.flatten(), b.flatten(), dim=0).item()
        assert cos > 0.999, cos
        assert abs(a.norm().item() - b.norm().item()) <= 2e-2 * b.norm().item()


def test_stats_fn_gradient():
    g = cpu_gen(47)
    x = rand_cl3d(g, 2, 8, 5, 4, 3)
    xd = x.to(DEV).requires_grad_(True)
    mean, sq = StatsFn.apply(xd)
    um, us = torch.randn(8, generator=g), torch.randn(8, generator=g)
    ((mean * um.to(DEV)).sum() + (sq * us.to(DEV)).sum()).backward()
    assert torch.equal(xd.grad.cpu().contiguous().view(torch.int16),
                       oracle.stats_bwd(x, um, us).contiguous().view(torch.int16))


def test_linear_family_gradients_against_torch_autograd():
    """ReLULinearAddFn and LinBReLULinAddFn against fp32 torch autograd of the 1x1x1 convolutions they stand for
    (the ground truth of the reference's tests/ops/test_linear.py)."""
    from kerops_amd.autograd import LinBReLULinAddFn, ReLULinearAddFn
    g = cpu_gen(53)
    n, c, co, h, w, d = 2, 32, 16, 5, 6, 7
    x, add = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, co, h, w, d)
    Wm = (torch.randn(c, co, generator=g) / math.sqrt(c)).half()
    up = rand_cl3d(g, n, co, h, w, d)
    xd, ad, wd = (t_.to(DEV).requires_grad_(True) for t_ in (x, add, Wm))
    out = ReLULinearAddFn.apply(xd, wd, ad)
    out.backward(up.to(DEV))
    xr, ar, wr = (t_.float().requires_grad_(True) for t_ in (x, add, Wm))
    ref = F.conv3d(F.relu(xr), wr.t().reshape(co, c, 1, 1, 1)) + ar
    ref.backward(up.float())
    assert torch.allclose(out.float().cpu(), ref, rtol=2e-3, atol=4e-3)
    assert torch.allclose(xd.grad.float().cpu(), xr.grad, rtol=2e-3, atol=4e-3)
    assert torch.equal(ad.grad.cpu(), up)
    assert ((wd.grad.float().cpu() - wr.grad).norm() / wr.grad.norm()).item() < 2e-3

    add2, up2 = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    Wu = (torch.randn(c, 2 * c, generator=g) / math.sqrt(c)).half()
    Wd = (torch.randn(2 * c, c, generator=g) / math.sqrt(2 * c)).half()
    b = (torch.randn(2 * c, generator=g) * 0.5).half()
    dev = [t_.to(DEV).requires_grad_(True) for t_ in (x, Wu, Wd, b, add2)]
    out = LinBReLULinAddFn.apply(*dev)
    out.backward(up2.to(DEV))
    refs = [t_.float().requires_grad_(True) for t_ in (x, Wu, Wd, b, add2)]
    hid = F.relu(F.conv3d(refs[0], refs[1].t().reshape(2 * c, c, 1, 1, 1), refs[3]))
    ref = F.conv3d(hid, refs[2].t().reshape(c, 2 * c, 1, 1, 1)) + refs[4]
    ref.backward(up2.float())
    assert torch.allclose(out.float().cpu(), ref, rtol=4e-3, atol=8e-3)
    # a hidden unit whose pre-activation is within one fp16 rounding of zero may take the other side of the
    # ReLU: rare, but it moves that voxel's input gradient by a whole weight row
    bad = (dev[0].grad.float().cpu() - refs[0].grad).abs() > 2e-2 + 1e-2 * refs[0].grad.abs()
    assert bad.float().mean().item() < 2e-2
    for got, want in zip(dev[1:4], refs[1:4]):
        # (the same flips reach the weight gradients; the strict comparison is the one against the oracle)
        assert ((got.grad.float().cpu() - want.grad).norm() / want.grad.norm()).item() < 3e-2
    assert torch.equal(dev[4].grad.cpu(), up2)


def test_fused_forward_functions_have_the_gradients_of_their_compositions():
    # the one-pass forward ops do the arithmetic of the compositions they stand for (the conv output bit for bit; the
    # statistics are fp32 sums taken in another order); their backward runs the same backward ops
    g = cpu_gen(47)
    n, c, h, w, d = 2, 32, 6, 7, 9
    x = rand_cl3d(g, n, c, h, w, d)
    res = rand_cl3d(g, n, c, h, w, d)
    _, wk = rand_dw_weight(g, c)
    pw = (torch.randn(c, c, generator=g) / math.sqrt(c)).half()
    gamma = torch.rand(c, generator=g) + 0.5
    beta = torch.randn(c, generator=g) * 0.3
    go = rand_cl3d(g, n, c, h, w, d)

    def run(fused):
        leaves = [t.to(DEV).requires_grad_(True) for t in (x, wk, gamma, beta, pw, res)]
        xd, wd, gd, bd, pd, rd = leaves
        if fused:
            y, mean, sq = DWConvStatsFn.apply(xd, wd)
        else:
            y = DWConvFn.apply(xd, wd)
            mean, sq = StatsFn.apply(y)
        # batch-norm fold in torch autograd (fp32), as a user of the ops would write it
        inv = torch.rsqrt(sq - mean * mean + 1e-5)
        scale, shift = gd * inv, bd - mean * gd * inv
        if fused:
            out = ApplyBNReLULinearAddFn.apply(y, scale, shift, pd, rd)
        else:
            out = ReLULinearAddFn.apply(ApplyBNReLUFn.apply(y, scale, shift), pd, rd)
        out.backward(go.to(DEV))
        return [out.detach()] + [t.grad for t in leaves] + [y.detach(), mean.detach(), sq.detach()]

    a, b = run(True), run(False)
    assert torch.equal(a[7], b[7])  # the conv output: bit for bit
    for u, v in ((a[8], b[8]), (a[9], b[9])):  # per-channel sums of 756 values in two orders
        assert torch.allclose(u, v, rtol=1e-5, atol=1e-6)
    # scale and shift then differ in their last fp32 bits, which can move an fp16 activation by one step before
    # the pointwise layer and the output by one more
    assert (a[0].float() - b[0].float()).abs().max().item() <= 2.0 ** -8 * max(1.0, b[0].float().abs().max().item())
    # with the same scale and shift the fused second half is bit-identical to its composition
    yd, pd, rd = a[7], pw.to(DEV), res.to(DEV)
    sc, sh = (torch.rand(c, generator=g) + 0.5).to(DEV), (torch.randn(c, generator=g) * 0.3).to(DEV)
    assert torch.equal(ApplyBNReLULinearAddFn.apply(yd, sc, sh, pd, rd),
                       ReLULinearAddFn.apply(ApplyBNReLUFn.apply(yd, sc, sh), pd, rd))
    # backward: the same backward ops on the same tensors, except that the composition lets torch add the two fp16
    # gradients that reach y (one more rounding) where the fused Function adds them in fp32 inside AddStatsBackward
    for i, (u, v) in enumerate(zip(a[1:7], b[1:7])):
        assert u.dtype == v.dtype and u.shape == v.shape, i
        err = (u.float() - v.float()).abs().max().item()
        assert err <= 2.0 ** -8 * max(1.0, v.float().abs().max().item()), (i, err)
    assert torch.equal(a[6], b[6])  # the residual's gradient is the upstream gradient in both
