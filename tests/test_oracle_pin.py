"""Pins the CPU oracle (oracle/kerops_oracle.c) before anything is compared with it.

Each oracle function is checked against (i) the committed golden vectors, which were
produced by torch CPU library routines only, (ii) the same torch routines on fresh seeded
inputs with odd sizes, and (iii) closed forms / brute force chosen so that a flipped tap,
a transposed axis, a wrong divisor or a dropped term fails.  No GPU is involved.
"""
import itertools
import math

import numpy as np
import pytest
import torch
from torch import nn
from torch.nn import functional as F

import oracle
from conftest import cpu_gen, from_bits, rand_cl3d, rand_dw_weight

SHAPES = [(1, 8, 5, 4, 3), (2, 8, 7, 13, 2), (1, 16, 3, 16, 9), (3, 32, 2, 3, 7), (1, 64, 4, 5, 6)]


def torch_dwconv(x, w_torch, dtype=torch.float32):
    return F.conv3d(x.to(dtype), w_torch.to(dtype), None, stride=1, padding=1, groups=x.shape[1])


# ------------------------------------------------------------------ fp16 conversions
def test_fp16_conversions_exhaustive():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    h = bits.view(torch.float16)
    f = oracle.h2f(h)
    ref = h.float()
    ok = ~torch.isnan(ref)
    assert torch.equal(f[ok], ref[ok]) and torch.isnan(f[~ok]).all()
    g = cpu_gen(1)
    vals = [torch.randn(200000, generator=g) * s for s in (1e-8, 1e-6, 1e-4, 1e-2, 1.0, 300.0, 70000.0)]
    vals.append(h.float()[ok])
    # ties and range boundaries
    vals.append(torch.tensor([65504.0, 65519.99, 65520.0, -65520.0, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                              2.0 ** -24 * 1.5, 2.0 ** -24 * 2.5, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 0.0, -0.0]))
    r = torch.cat(vals)
    assert torch.equal(oracle.f2h(r).view(torch.int16), r.half().view(torch.int16))


# ------------------------------------------------------------------ golden vectors
def test_oracle_against_golden(golden):
    x = from_bits(golden['x']).to(memory_format=torch.channels_last_3d)
    grad = from_bits(golden['grad']).to(memory_format=torch.channels_last_3d)
    wt = from_bits(golden['weight_c13x3x3'])
    wk = wt[:, 0].permute(1, 2, 3, 0).contiguous()

    y16, y32 = oracle.dwconv_fwd(x, wk, wide=True, return_fp32=True)
    assert torch.allclose(y32, torch.from_numpy(golden['dwconv_y_f32']), rtol=1e-5, atol=1e-6)
    # fp64 vs fp32 summation may straddle an fp16 rounding tie: at most one fp16 ulp apart, rarely
    gold16 = from_bits(golden['dwconv_y'])
    same = (y16.contiguous().view(torch.int16) == gold16.view(torch.int16)).float().mean()
    assert same > 0.995
    assert (y16.float() - gold16.float()).abs().max() <= 2.0 ** -9
    # the fp32 flavour of the oracle adds the taps in the order torch's CPU kernel does
    y16n, y32n = oracle.dwconv_fwd(x, wk, wide=False, return_fp32=True)
    assert torch.allclose(y32n, torch.from_numpy(golden['dwconv_y_f32']), rtol=1e-6, atol=1e-6)

    gw = oracle.dwconv_wgrad(x, grad)
    assert torch.allclose(gw, torch.from_numpy(golden['dwconv_wgrad_f64']), rtol=1e-12, atol=1e-12)

    mean, sq = oracle.stats(x)
    assert torch.allclose(mean, torch.from_numpy(golden['stats_mean_f64']), rtol=1e-12, atol=1e-14)
    assert torch.allclose(sq, torch.from_numpy(golden['stats_sqmean_f64']), rtol=1e-12, atol=1e-14)

    # BN folding as the reference's test does it (tests/ops/test_bn_relu.py:27-29)
    gamma, beta = torch.from_numpy(golden['gamma']).double(), torch.from_numpy(golden['beta']).double()
    rvareps = torch.rsqrt(sq - mean ** 2 + 1e-5)
    W, B = gamma * rvareps, beta - mean * rvareps * gamma
    y = oracle.bnrelu_fwd(x, W, B)
    ref = torch.from_numpy(golden['bnrelu_y_f32'])
    assert torch.allclose(y.float(), ref, rtol=1e-3, atol=1e-3)  # fp16 output rounding only

    yp, pm, ps, yp32 = oracle.avgpool_ceil_stats(x, return_fp32=True)
    assert torch.equal(yp32.contiguous(), torch.from_numpy(golden['avgpool_y_f32']))
    assert torch.allclose(pm, torch.from_numpy(golden['avgpool_mean_f64']), rtol=1e-6, atol=1e-7)
    assert torch.allclose(ps, torch.from_numpy(golden['avgpool_sqmean_f64']), rtol=1e-6, atol=1e-7)


def test_oracle_against_config1_fixture(golden_config1):
    """The CPU-runnable DWConv configuration, x (1,8,64,64,32): the oracle against the committed torch results."""
    x = from_bits(golden_config1['x']).to(memory_format=torch.channels_last_3d)
    wk = from_bits(golden_config1['weight_c13x3x3'])[:, 0].permute(1, 2, 3, 0).contiguous()
    gold = from_bits(golden_config1['dwconv_y'])
    for wide in (True, False):
        y16 = oracle.dwconv_fwd(x, wk, wide=wide)
        assert torch.allclose(y16.float(), gold.float(), rtol=1e-2, atol=1e-2)  # the configuration's tolerance
        # torch rounded an fp32 sum, the oracle an fp64 (wide) or fp32 one: equal but for sums next to an fp16 tie
        same = (y16.contiguous().view(torch.int16) == gold.view(torch.int16)).float().mean().item()
        assert same >= 0.999, same
        assert (y16.float() - gold.float()).abs().max() <= 2.0 ** -10 * max(1.0, gold.abs().max().item())
    grad = torch.flip(x, dims=(2, 3, 4)).contiguous(memory_format=torch.channels_last_3d)
    gw = oracle.dwconv_wgrad(x, grad)
    assert torch.allclose(gw, torch.from_numpy(golden_config1['dwconv_wgrad_f64']), rtol=1e-11, atol=1e-11)


# ------------------------------------------------------------------ DWConv forward
@pytest.mark.parametrize('shape', SHAPES)
def test_dwconv_fwd_vs_torch(shape):
    g = cpu_gen()
    x = rand_cl3d(g, *shape)
    wt, wk = rand_dw_weight(g, shape[1])
    for wide in (False, True):
        y16, y32 = oracle.dwconv_fwd(x, wk, wide=wide, return_fp32=True)
        ref = torch_dwconv(x, wt, torch.float64)
        assert torch.allclose(y32.double(), ref, rtol=2e-6, atol=2e-6)
        assert y16.is_contiguous(memory_format=torch.channels_last_3d) or min(shape[2:]) == 1
        assert (y16.float() - ref.float()).abs().max() <= 2.0 ** -10 * max(1.0, ref.abs().max().item())


def test_dwconv_fwd_single_taps_are_shifts():
    """A weight with a single 1 at (kh,kw,kd) must copy x shifted by (kh-1,kw-1,kd-1) with a
    zero border: pins tap orientation (correlation, not convolution) and the axis order."""
    g = cpu_gen(3)
    n, c, H, W, D = 1, 8, 5, 6, 7
    x = rand_cl3d(g, n, c, H, W, D)
    for kh, kw, kd in itertools.product(range(3), repeat=3):
        wk = torch.zeros(3, 3, 3, c, dtype=torch.float16)
        wk[kh, kw, kd] = 1.0
        y = oracle.dwconv_fwd(x, wk)
        exp = torch.zeros_like(x)
        sh, sw, sd = kh - 1, kw - 1, kd - 1
        src = x[:, :, max(sh, 0):H + min(sh, 0), max(sw, 0):W + min(sw, 0), max(sd, 0):D + min(sd, 0)]
        exp[:, :, max(-sh, 0):H + min(-sh, 0), max(-sw, 0):W + min(-sw, 0), max(-sd, 0):D + min(-sd, 0)] = src
        assert torch.equal(y, exp), (kh, kw, kd)


def test_dwconv_fwd_ones_counts_neighbours():
    c, H, W, D = 8, 4, 5, 3
    x = torch.ones(1, c, H, W, D, dtype=torch.float16).to(memory_format=torch.channels_last_3d)
    wk = torch.ones(3, 3, 3, c, dtype=torch.float16)
    y = oracle.dwconv_fwd(x, wk)

    def cnt(i, n):
        return min(i + 1, n - 1) - max(i - 1, 0) + 1

    for h, w, d in itertools.product(range(H), range(W), range(D)):
        assert y[0, 0, h, w, d].item() == cnt(h, H) * cnt(w, W) * cnt(d, D)
    assert sorted(set(y.flatten().tolist())) == [8.0, 12.0, 18.0, 27.0]


def test_dwconv_fwd_brute_force_and_linearity():
    g = cpu_gen(5)
    n, c, H, W, D = 1, 8, 5, 4, 3
    x = rand_cl3d(g, n, c, H, W, D)
    _, wk = rand_dw_weight(g, c)
    _, y32 = oracle.dwconv_fwd(x, wk, wide=True, return_fp32=True)
    xf, wf = x.double(), wk.double()
    for h, w, d, ch in itertools.product(range(H), range(W), range(D), range(c)):
        s = 0.0
        for kh, kw, kd in itertools.product(range(3), repeat=3):
            hh, ww, dd = h + kh - 1, w + kw - 1, d + kd - 1
            if 0 <= hh < H and 0 <= ww < W and 0 <= dd < D:
                s += xf[0, ch, hh, ww, dd].item() * wf[kh, kw, kd, ch].item()
        assert abs(y32[0, ch, h, w, d].item() - s) < 1e-6
    x2 = rand_cl3d(g, n, c, H, W, D)
    _, a = oracle.dwconv_fwd(x, wk, return_fp32=True)
    _, b = oracle.dwconv_fwd(x2, wk, return_fp32=True)
    xs = (x.float() * 0.5 + x2.float() * 0.25).half().to(memory_format=torch.channels_last_3d)
    exact = (xs.float() == x.float() * 0.5 + x2.float() * 0.25).all()
    if exact:
        _, s = oracle.dwconv_fwd(xs, wk, return_fp32=True)
        assert torch.allclose(s, 0.5 * a + 0.25 * b, rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ DWConv wgrad
@pytest.mark.parametrize('shape', SHAPES)
def test_dwconv_wgrad_vs_autograd(shape):
    g = cpu_gen()
    x, grad = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    wt, wk = rand_dw_weight(g, shape[1])
    w64 = wt.double().clone().requires_grad_(True)
    torch_dwconv(x, w64, torch.float64).backward(grad.double())
    ref = w64.grad[:, 0].permute(1, 2, 3, 0)
    gw = oracle.dwconv_wgrad(x, grad)
    assert torch.allclose(gw, ref, rtol=1e-11, atol=1e-11)


def test_dwconv_wgrad_closed_forms():
    c, H, W, D = 8, 4, 5, 6
    ones = torch.ones(1, c, H, W, D, dtype=torch.float16).to(memory_format=torch.channels_last_3d)
    gw = oracle.dwconv_wgrad(ones, ones)
    for kh, kw, kd in itertools.product(range(3), repeat=3):
        assert gw[kh, kw, kd, 0].item() == (H - abs(kh - 1)) * (W - abs(kw - 1)) * (D - abs(kd - 1))
    g = cpu_gen(9)
    x, grad = rand_cl3d(g, 2, c, H, W, D), rand_cl3d(g, 2, c, H, W, D)
    gw = oracle.dwconv_wgrad(x, grad)
    centre = (x.double() * grad.double()).sum(dim=(0, 2, 3, 4))
    assert torch.allclose(gw[1, 1, 1], centre, rtol=1e-12)
    # 27 sliced dot products (independent restatement)
    xp = F.pad(x.double(), (1, 1, 1, 1, 1, 1))
    for kh, kw, kd in itertools.product(range(3), repeat=3):
        s = (grad.double() * xp[:, :, kh:kh + H, kw:kw + W, kd:kd + D]).sum(dim=(0, 2, 3, 4))
        assert torch.allclose(gw[kh, kw, kd], s, rtol=1e-12, atol=1e-12), (kh, kw, kd)
    # adjoint identity <DWConv(x, w), g> = <w, WGRAD(x, g)>
    _, wk = rand_dw_weight(g, c)
    _, y32 = oracle.dwconv_fwd(x, wk, wide=True, return_fp32=True)
    lhs = (y32.double() * grad.double()).sum()
    rhs = (wk.double() * gw).sum()
    assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(rhs))


# ------------------------------------------------------------------ stats / add
@pytest.mark.parametrize('shape', [(1, 2, 3, 3, 3), (2, 4, 7, 5, 3)] + SHAPES)
def test_stats_and_backward(shape):
    g = cpu_gen()
    x = rand_cl3d(g, *shape)
    mean, sq = oracle.stats(x)
    xd = x.double()
    assert torch.allclose(mean, xd.mean(dim=(0, 2, 3, 4)), rtol=1e-12, atol=1e-14)
    assert torch.allclose(sq, (xd ** 2).mean(dim=(0, 2, 3, 4)), rtol=1e-12, atol=1e-14)
    c = shape[1]
    um, us = torch.randn(c, generator=g) / 3, torch.randn(c, generator=g) / 3
    xg = x.float().clone().requires_grad_(True)
    loss = ((xg ** 2).mean(dim=(0, 2, 3, 4)) * us).sum() + (xg.mean(dim=(0, 2, 3, 4)) * um).sum()
    loss.backward()
    dx = oracle.stats_bwd(x, um, us)
    assert torch.allclose(dx.float(), xg.grad, rtol=2e-3, atol=1e-6)


def test_stats_closed_forms():
    x = torch.full((2, 8, 3, 5, 7), 1.5, dtype=torch.float16).to(memory_format=torch.channels_last_3d)
    mean, sq = oracle.stats(x)
    assert torch.all(mean == 1.5) and torch.all(sq == 2.25)
    ramp = torch.arange(8, dtype=torch.float16).view(1, 8, 1, 1, 1).expand(2, 8, 3, 5, 7).contiguous(
        memory_format=torch.channels_last_3d)
    mean, sq = oracle.stats(ramp)
    assert torch.equal(mean, torch.arange(8, dtype=torch.float64))
    assert torch.equal(sq, torch.arange(8, dtype=torch.float64) ** 2)


def test_add_stats_and_backward():
    g = cpu_gen(11)
    shape = (2, 8, 5, 3, 7)
    x, y = rand_cl3d(g, *shape), rand_cl3d(g, *shape)
    z, mean, sq = oracle.add_stats(x, y)
    r = x + y  # fp16 add in torch rounds once, like the reference kernel
    assert torch.equal(z, r)
    assert torch.allclose(mean, r.double().mean(dim=(0, 2, 3, 4)), rtol=1e-12)
    assert torch.allclose(sq, (r.double() ** 2).mean(dim=(0, 2, 3, 4)), rtol=1e-12)
    um, us = torch.randn(8, generator=g) / 3, torch.randn(8, generator=g) / 3
    ug = rand_cl3d(g, *shape)
    rg = r.float().clone().requires_grad_(True)
    loss = (rg * ug.float()).sum() + ((rg ** 2).mean(dim=(0, 2, 3, 4)) * us).sum() + (
        rg.mean(dim=(0, 2, 3, 4)) * um).sum()
    loss.backward()
    out = oracle.add_stats_bwd(ug, um, us, z)
    assert torch.allclose(out.float(), rg.grad, rtol=2e-3, atol=1e-3)


# ------------------------------------------------------------------ BN-ReLU
@pytest.mark.parametrize('shape', [(1, 2, 3, 3, 3)] + SHAPES)
def test_bnrelu_forward_backward(shape):
    g = cpu_gen()
    c = shape[1]
    x = rand_cl3d(g, *shape)
    W = torch.randn(c, generator=g) + 0.5
    B = torch.randn(c, generator=g) * 2
    y = oracle.bnrelu_fwd(x, W, B)
    ref = F.relu(x.float() * W.view(1, c, 1, 1, 1) + B.view(1, c, 1, 1, 1))
    assert (y.float() - ref).abs().max() <= 2.0 ** -10 * max(1.0, ref.abs().max().item())
    assert torch.equal(oracle.bnrelu_fwd(x, torch.ones(c), torch.zeros(c)), F.relu(x))
    zero_w = oracle.bnrelu_fwd(x, torch.zeros(c), B)
    assert torch.equal(zero_w, B.clamp(min=0).half().view(1, c, 1, 1, 1).expand_as(x))

    grad = rand_cl3d(g, *shape, std=0.1)
    xg = x.float().clone().requires_grad_(True)
    Wg = W.clone().view(1, c, 1, 1, 1).requires_grad_(True)
    Bg = B.clone().view(1, c, 1, 1, 1).requires_grad_(True)
    F.relu(xg * Wg + Bg).backward(grad.float())
    dx, dW, dB = oracle.bnrelu_bwd(x, W, B, grad)
    assert torch.allclose(dx.float(), xg.grad, rtol=1e-3, atol=1e-4)
    assert torch.allclose(dW.float(), Wg.grad.flatten(), rtol=1e-4, atol=1e-3)
    assert torch.allclose(dB.float(), Bg.grad.flatten(), rtol=1e-4, atol=5e-4)


def test_bnrelu_matches_train_mode_batchnorm():
    g = cpu_gen(13)
    shape = (2, 16, 7, 5, 3)
    x = rand_cl3d(g, *shape, mean=0.5, std=math.sqrt(2.0))
    gamma = torch.rand(16, generator=g) + 0.5
    beta = torch.randn(16, generator=g) * math.sqrt(0.1)
    bn = nn.BatchNorm3d(16, eps=1e-5)
    with torch.no_grad():
        bn.weight.copy_(gamma)
        bn.bias.copy_(beta)
        ref = F.relu(bn.train()(x.float()))
    mean, sq = oracle.stats(x)
    rvareps = torch.rsqrt(sq - mean ** 2 + 1e-5)
    y = oracle.bnrelu_fwd(x, gamma.double() * rvareps, beta.double() - mean * rvareps * gamma.double())
    assert torch.allclose(y.float(), ref, rtol=1e-3, atol=1e-3)


# ------------------------------------------------------------------ avg pool
@pytest.mark.parametrize('shape', [(1, 2, 3, 3, 3), (2, 4, 7, 5, 2), (1, 8, 2, 2, 2), (1, 8, 2, 3, 2)] + SHAPES)
def test_avgpool_vs_torch(shape):
    g = cpu_gen()
    x = rand_cl3d(g, *shape)
    yp, mean, sq, y32 = oracle.avgpool_ceil_stats(x, return_fp32=True)
    ref = nn.AvgPool3d(2, ceil_mode=True)(x.float())
    assert torch.equal(y32.contiguous(), ref)  # sums of <= 8 fp16 values are exact in fp32
    assert torch.equal(yp.contiguous(), ref.half())
    assert torch.allclose(mean, ref.double().mean(dim=(0, 2, 3, 4)), rtol=1e-12, atol=1e-14)
    assert torch.allclose(sq, (ref.double() ** 2).mean(dim=(0, 2, 3, 4)), rtol=1e-12, atol=1e-14)

    c = shape[1]
    up = rand_cl3d(g, *ref.shape)
    um, us = torch.randn(c, generator=g), torch.randn(c, generator=g)
    xg = x.float().clone().requires_grad_(True)
    o = nn.AvgPool3d(2, ceil_mode=True)(xg)
    loss = (up.float() * o).sum() + (um * o.mean(dim=(0, 2, 3, 4))).sum() + (us * (o ** 2).mean(dim=(0, 2, 3, 4))).sum()
    loss.backward()
    dx = oracle.avgpool_ceil_stats_bwd(up, um, us, yp, list(shape))
    # the op uses the fp16-rounded pooled output in the sqmean term, autograd the fp32 one
    assert torch.allclose(dx.float(), xg.grad, rtol=2e-3, atol=2e-3)


def test_avgpool_edge_windows():
    x = torch.arange(27, dtype=torch.float16).view(1, 1, 3, 3, 3).expand(1, 2, 3, 3, 3).contiguous(
        memory_format=torch.channels_last_3d)
    yp, mean, sq = oracle.avgpool_ceil_stats(x)
    v = torch.arange(27, dtype=torch.float64).view(3, 3, 3)
    assert yp[0, 0, 0, 0, 0].item() == v[:2, :2, :2].mean().item()      # full window of 8
    assert yp[0, 0, 1, 0, 0].item() == v[2:, :2, :2].mean().item()      # 4 voxels
    assert yp[0, 0, 1, 1, 0].item() == v[2:, 2:, :2].mean().item()      # 2 voxels
    assert yp[0, 0, 1, 1, 1].item() == 26.0                             # single voxel
    const = torch.full((1, 8, 5, 3, 7), 0.75, dtype=torch.float16).to(memory_format=torch.channels_last_3d)
    yp, mean, sq = oracle.avgpool_ceil_stats(const)
    assert torch.all(yp == 0.75) and torch.all(mean == 0.75) and torch.all(sq == 0.5625)


# ------------------------------------------------------------------ quantisers
@pytest.mark.parametrize('window', [1.0, 3.0, 0.37, 6.5, 100.0])
def test_quant_u8_window_exhaustive(window):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    x = bits[~torch.isnan(bits)]
    q = oracle.quant_u8_window(x, window)
    ref = oracle.np_quant_u8_window(x.float().numpy(), window)
    assert np.array_equal(q.numpy(), ref)
    q32 = oracle.quant_u8_window(x.float(), window)
    assert torch.equal(q, q32)
    w16 = torch.tensor([-window, window, 0.0], dtype=torch.float32)
    assert oracle.quant_u8_window(w16, window).tolist() == [0, 255, 127]
    order = torch.argsort(x.float())
    assert (np.diff(q[order].numpy().astype(np.int32)) >= 0).all()  # monotone
    big = torch.tensor([1e4, -1e4, float('inf'), float('-inf')], dtype=torch.float32)
    assert oracle.quant_u8_window(big, window).tolist() == [255, 0, 255, 0]
    for dt in (torch.float16, torch.float32):
        back = oracle.dequant_u8_window(q, dt, window).float()
        inside = x.float().abs() <= window
        tol = 2 * window / 255 * (1 + 1e-3) + (2.0 ** -10 * window if dt == torch.float16 else 0.0)
        assert ((back - x.float()).abs()[inside] <= tol).all()
    lo = oracle.dequant_u8_window(torch.tensor([0, 255], dtype=torch.uint8), torch.float32, window)
    assert lo[0].item() == -np.float32(window) and abs(lo[1].item() - window) <= 1e-6 * window


def test_quant_i8_sym_closed_forms():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    y = bits[torch.isfinite(bits)]
    for amax in (1.0, 127.0, 3.3, 65504.0):
        q = oracle.quant_i8_sym(y, amax)
        scale = np.float32(amax) / np.float32(127.0)
        ref = torch.round(torch.from_numpy((y.float().numpy() / scale).astype(np.float32))).clamp(-127, 127).to(
            torch.int8)
        assert torch.equal(q, ref)
    # scale = 1 exactly: ties go to even
    ties = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, -127.5], dtype=torch.float16)
    assert oracle.quant_i8_sym(ties, 127.0).tolist() == [0, 2, 2, 0, -2, -2, 126, 127, -127]
    assert oracle.absmax_f16(y) == 65504.0
    assert oracle.quant_i8_sym(torch.zeros(5, dtype=torch.float16), 0.0).tolist() == [0] * 5


# ------------------------------------------------------------------ pointwise / fused block
def test_pointwise_and_block_vs_torch():
    g = cpu_gen(17)
    n, cin, cout, h, w, d = 1, 16, 32, 3, 5, 4
    x = rand_cl3d(g, n, cin, h, w, d)
    Wm = (torch.randn(cin, cout, generator=g) / math.sqrt(cin)).half()
    add = rand_cl3d(g, n, cout, h, w, d)
    out = oracle.pointwise(x, Wm, add=add, relu_in=True)
    conv = F.conv3d(F.relu(x.double()), Wm.double().t().reshape(cout, cin, 1, 1, 1))
    ref = conv.half() + add
    assert torch.equal(out, ref)
    # fused block = dwconv -> affine -> relu -> fp16 -> pointwise
    _, wk = rand_dw_weight(g, cin)
    scale, shift = torch.rand(cin, generator=g) + 0.5, torch.randn(cin, generator=g) * 0.3
    y, mid = oracle.dwsep_block(x, wk, scale, shift, Wm, return_mid=True)
    _, acc = oracle.dwconv_fwd(x, wk, wide=True, return_fp32=True)
    t = F.relu(acc * scale.view(1, cin, 1, 1, 1) + shift.view(1, cin, 1, 1, 1)).half()
    assert (mid.float() - t.float()).abs().max() <= 2.0 ** -10 * max(1.0, t.abs().max().item())
    ref_y = oracle.pointwise(mid, Wm)
    assert torch.equal(y, ref_y)


def test_relu_linear_bwd_vs_torch_autograd():
    """Pinned by autograd of the 1x1x1 conv3d of relu(x) in fp64 (the ground truth of the reference's
    own test, tests/ops/test_linear.py:40-78) and by closed forms."""
    g = cpu_gen(23)
    n, cin, cout, h, w, d = 2, 16, 32, 3, 5, 4
    x = rand_cl3d(g, n, cin, h, w, d)
    grad = rand_cl3d(g, n, cout, h, w, d)
    Wm = (torch.randn(cin, cout, generator=g) / math.sqrt(cin)).half()
    dx, dw = oracle.relu_linear_bwd(x, grad, Wm)
    xd = x.double().requires_grad_(True)
    wd = Wm.double().requires_grad_(True)
    out = F.conv3d(F.relu(xd), wd.t().reshape(cout, cin, 1, 1, 1))
    out.backward(grad.double())
    assert torch.equal(dx, xd.grad.half())
    assert dx.stride() == x.stride()
    assert torch.allclose(dw, wd.grad, rtol=1e-12, atol=1e-12)
    # closed forms: identity weight passes grad through the mask; an all-negative x has no gradient at all
    eye = torch.eye(cin, dtype=torch.float16)
    grad_c = rand_cl3d(g, n, cin, h, w, d)
    dx, dw = oracle.relu_linear_bwd(x, grad_c, eye)
    assert torch.equal(dx, torch.where(x > 0, grad_c, torch.zeros_like(grad_c)))
    ref_dw = torch.einsum('nihwd,nohwd->io', F.relu(x.double()), grad_c.double())
    assert torch.allclose(dw, ref_dw, rtol=1e-12, atol=1e-12)
    dx, dw = oracle.relu_linear_bwd(-x.abs(), grad, Wm)
    assert dx.abs().max() == 0 and dw.abs().max() == 0


def test_lin_brelu_lin_add_vs_torch():
    """Pinned by the two 1x1x1 conv3d calls of the reference's own test (tests/ops/test_linear.py:101-106),
    with the fp16 roundings of the kernel (kerops/kernels/linear.py:139-141) made explicit."""
    g = cpu_gen(29)
    n, c, h, w, d = 2, 16, 3, 5, 4
    x, add = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    Wup = (torch.randn(c, 2 * c, generator=g) / math.sqrt(c)).half()
    Wdown = (torch.randn(2 * c, c, generator=g) / math.sqrt(2 * c)).half()
    bias = (torch.randn(2 * c, generator=g) * 0.5).half()
    out, hid = oracle.lin_brelu_lin_add(x, Wup, Wdown, bias, add, return_hidden=True)
    up = F.conv3d(x.double(), Wup.double().t().reshape(2 * c, c, 1, 1, 1)).half()
    hid_ref = F.relu((up.float() + bias.float().view(1, -1, 1, 1, 1)).half())
    assert torch.equal(hid, hid_ref)
    down = F.conv3d(hid_ref.double(), Wdown.double().t().reshape(c, 2 * c, 1, 1, 1)).half()
    assert torch.equal(out, (down.float() + add.float()).half())
    # closed form: Wup = [I 0], bias = 0, Wdown = [I; 0]  ->  out = relu(x) + add
    eye_up = torch.cat([torch.eye(c), torch.zeros(c, c)], 1).half()
    eye_dn = torch.cat([torch.eye(c), torch.zeros(c, c)], 0).half()
    out = oracle.lin_brelu_lin_add(x, eye_up, eye_dn, torch.zeros(2 * c, dtype=torch.float16), add)
    assert torch.equal(out, (F.relu(x).float() + add.float()).half())


def test_lin_brelu_lin_bwd_vs_torch():
    """Pinned by a torch restatement with the kernel's fp16 roundings made explicit
    (kerops/kernels/linear.py:196-214) and, loosely, by fp64 autograd of the two conv3d calls
    (the ground truth of tests/ops/test_linear.py:146-151)."""
    g = cpu_gen(37)
    n, c, h, w, d = 2, 16, 3, 5, 4
    x, grad = rand_cl3d(g, n, c, h, w, d), rand_cl3d(g, n, c, h, w, d)
    Wup = (torch.randn(c, 2 * c, generator=g) / math.sqrt(c)).half()
    Wdown = (torch.randn(2 * c, c, generator=g) / math.sqrt(2 * c)).half()
    bias = (torch.randn(2 * c, generator=g) * 0.5).half()
    dx, dup, ddn, db = oracle.lin_brelu_lin_bwd(x, grad, Wup, Wdown, bias)
    X = x.permute(0, 2, 3, 4, 1).reshape(-1, c).double()
    G = grad.permute(0, 2, 3, 4, 1).reshape(-1, c).double()
    lin = ((X @ Wup.double()).half().float() + bias.float()).half()
    hid = F.relu(lin).double()
    lg = torch.where(lin > 0, (G @ Wdown.double().t()).half(), torch.zeros_like(lin)).double()
    assert torch.allclose(ddn, hid.t() @ G, rtol=1e-12, atol=1e-12)
    assert torch.allclose(dup, X.t() @ lg, rtol=1e-12, atol=1e-12)
    assert torch.allclose(db, lg.sum(0), rtol=1e-12, atol=1e-12)
    ref_dx = (lg @ Wup.double().t()).half().reshape(n, h, w, d, c).permute(0, 4, 1, 2, 3)
    assert torch.equal(dx, ref_dx) and dx.stride() == x.stride()
    # fp64 autograd without the intermediate roundings agrees to fp16 accuracy
    xd = x.double().requires_grad_(True)
    wu, wd_, bd = (t_.double().requires_grad_(True) for t_ in (Wup, Wdown, bias))
    y = F.conv3d(F.relu(F.conv3d(xd, wu.t().reshape(2 * c, c, 1, 1, 1), bd)), wd_.t().reshape(c, 2 * c, 1, 1, 1))
    y.backward(grad.double())
    for a_, b_ in ((dup, wu.grad), (ddn, wd_.grad), (db, bd.grad)):
        assert ((a_ - b_).norm() / b_.norm()).item() < 2e-3
    assert (dx.double() - xd.grad).abs().max() < 2e-2
