"""Writes tests/golden/hotpath_small.npz (inputs and expected outputs for every op of the
hot path on one small odd-sized case) and tests/golden/config1_dwconv.npz (the CPU-runnable
DWConv configuration, x (1,8,64,64,32)), computed with the torch CPU routines that the
reference's own tests use as ground truth (tests/ops/test_conv.py:25,62-72,
test_stats.py:13-16, test_bn_relu.py:18-30, test_avgpool.py:12-16 of the reference).

The reference stores no vectors of its own (every test regenerates its inputs on the GPU),
and neither the reference package nor the oracle is imported here: the fixture is produced
by library routines only, so it pins the oracle and the HIP kernels independently.

    python tests/golden/make_golden.py
"""
import math
import os

import numpy as np
import torch
from torch import nn
from torch.nn import functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(t):
    """fp16 tensor -> uint16 numpy array in logical (N, C, H, W, D) order."""
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    g = torch.Generator('cpu').manual_seed(322)
    n, c, h, w, d = 2, 8, 7, 13, 5
    x = torch.randn(n, c, h, w, d, generator=g).half()
    grad = torch.randn(n, c, h, w, d, generator=g).half()
    wt = (torch.randn(c, 1, 3, 3, 3, generator=g) / math.sqrt(27)).half()
    gamma = torch.rand(c, generator=g) + 0.5
    beta = torch.randn(c, generator=g) * math.sqrt(0.1)

    out = {}
    out['x'] = bits(x)
    out['grad'] = bits(grad)
    out['weight_c13x3x3'] = bits(wt)

    # DWConv forward, fp32 on the CPU, one rounding to fp16
    y32 = F.conv3d(x.float(), wt.float(), None, stride=1, padding=1, groups=c)
    out['dwconv_y_f32'] = y32.numpy()
    out['dwconv_y'] = bits(y32.half())

    # weight gradient by fp64 autograd, reported as [3,3,3,C]
    w64 = wt.double().clone().requires_grad_(True)
    F.conv3d(x.double(), w64, None, stride=1, padding=1, groups=c).backward(grad.double())
    out['dwconv_wgrad_f64'] = w64.grad[:, 0].permute(1, 2, 3, 0).contiguous().numpy()

    # per-channel statistics
    xf = x.double()
    out['stats_mean_f64'] = xf.mean(dim=(0, 2, 3, 4)).numpy()
    out['stats_sqmean_f64'] = (xf ** 2).mean(dim=(0, 2, 3, 4)).numpy()

    # train-mode batch norm + ReLU in fp32, and the folded per-channel (W, B)
    bn = nn.BatchNorm3d(c, eps=1e-5)
    with torch.no_grad():
        bn.weight.copy_(gamma)
        bn.bias.copy_(beta)
    bn.train()
    with torch.no_grad():
        out['bnrelu_y_f32'] = F.relu(bn(x.float())).numpy()
    out['gamma'] = gamma.numpy()
    out['beta'] = beta.numpy()

    # 2x2x2 ceil-mode average pool of the fp16 tensor computed in fp32
    pooled = nn.AvgPool3d(2, ceil_mode=True)(x.float())
    out['avgpool_y_f32'] = pooled.numpy()
    out['avgpool_mean_f64'] = pooled.double().mean(dim=(0, 2, 3, 4)).numpy()
    out['avgpool_sqmean_f64'] = (pooled.double() ** 2).mean(dim=(0, 2, 3, 4)).numpy()

    np.savez_compressed(os.path.join(HERE, 'hotpath_small.npz'), **out)
    print('wrote', os.path.join(HERE, 'hotpath_small.npz'))
    config1()


def config1():
    """x fp16 channels_last_3d (1,8,64,64,32) ~ N(0,1), depthwise weight (8,1,3,3,3) ~ N(0,1/27), padding 1,
    stride 1, no bias: conv3d(groups=C) in fp32 on the CPU, output cast to fp16.  The weight gradient is taken by
    fp64 autograd against the upstream gradient grad = x flipped along H, W and D (N(0,1) as well, and derivable
    from x, which keeps the file to x, the weight and the two results)."""
    g = torch.Generator('cpu').manual_seed(322)
    n, c, h, w, d = 1, 8, 64, 64, 32
    x = torch.randn(n, c, h, w, d, generator=g).half()
    wt = (torch.randn(c, 1, 3, 3, 3, generator=g) / math.sqrt(27)).half()
    out = {'x': bits(x), 'weight_c13x3x3': bits(wt)}
    y32 = F.conv3d(x.float(), wt.float(), None, stride=1, padding=1, groups=c)
    out['dwconv_y'] = bits(y32.half())
    grad = torch.flip(x, dims=(2, 3, 4))
    w64 = wt.double().clone().requires_grad_(True)
    F.conv3d(x.double(), w64, None, stride=1, padding=1, groups=c).backward(grad.double())
    out['dwconv_wgrad_f64'] = w64.grad[:, 0].permute(1, 2, 3, 0).contiguous().numpy()
    np.savez_compressed(os.path.join(HERE, 'config1_dwconv.npz'), **out)
    print('wrote', os.path.join(HERE, 'config1_dwconv.npz'))


if __name__ == '__main__':
    main()
