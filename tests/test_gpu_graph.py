"""The library only launches kernels on the caller's stream (no allocation, no memset, no host
synchronisation), so a sequence of ops can be captured into a HIP graph and replayed.  Every replay is
checked against the eager result on the same inputs, with eager work and synchronisations between the
replays."""
import pytest
import torch

from conftest import cpu_gen, rand_cl3d, rand_dw_weight
from kerops_amd.ops.avgpool import AvgPoolCeilStats
from kerops_amd.ops.bnrelu import ApplyBNReLU
from kerops_amd.ops.conv import DWConv, DWConvStats, DWConvWGRAD
from kerops_amd.ops.linear import ReLULinearAdd
from kerops_amd.ops.stats import Stats

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def block(x, wk, scale, shift, pw):
    y = DWConv(x, wk)
    mean, sq = Stats(y)
    y2, mean2, sq2 = DWConvStats(x, wk)
    z = ApplyBNReLU(y, scale, shift)
    pooled, pm, pq = AvgPoolCeilStats(z)
    lin = ReLULinearAdd(y, pw, x)
    gw = DWConvWGRAD(x, y, out_dtype=torch.float32)
    return y, mean, sq, y2, mean2, sq2, z, pooled, pm, pq, lin, gw


def test_conv_bn_pool_block_replays_from_a_hip_graph():
    g = cpu_gen(2024)
    c = 32
    shape = (2, c, 9, 20, 33)
    _, wk = rand_dw_weight(g, c)
    wk = wk.to(DEV)
    scale = (torch.rand(c, generator=g) + 0.5).to(DEV)
    shift = (torch.randn(c, generator=g) * 0.3).to(DEV)
    pw = (torch.randn(c, c, generator=g) / c ** 0.5).half().to(DEV)
    xs = rand_cl3d(g, *shape).to(DEV)  # static input of the graph

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture
        block(xs, wk, scale, shift, pw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = block(xs, wk, scale, shift, pw)

    for rep in range(3):
        x_new = rand_cl3d(g, *shape).to(DEV)
        xs.copy_(x_new)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = block(x_new, wk, scale, shift, pw)  # eager, between the replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (rep, i)
