"""GPU tests of the autograd.Function wrappers: gradients of a small depthwise block through the
HIP ops against torch autograd of the same mathematics in fp32."""
import math

import pytest
import torch
from torch.nn import functional as F

import oracle
from conftest import cpu_gen, rand_cl3d, rand_dw_weight
from kerops_amd.autograd import AddStatsFn, ApplyBNReLUFn, AvgPoolCeilStatsFn, DWConvFn, StatsFn
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
