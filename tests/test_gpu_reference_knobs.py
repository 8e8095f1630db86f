"""Every op called with the reference's own default knob values passed explicitly.

The reference's launch knobs (`num_warps`, `D_block`, `ILP`, `ACCTYPE`, `l1_cache_bytes`) are part of each op's
signature; code written against the reference may pass any value the reference accepts.  The values below are
the reference's own tables and constants: kerops/ops/conv/dwconv.py:10-24, kerops/ops/conv/dwconv_wgrad.py:10-30,
kerops/ops/stats.py:11,34, kerops/ops/bnrelu.py:11,44, kerops/ops/avgpool.py:11-14,63, kerops/ops/addition.py:11,52,
kerops/ops/quantization.py:9,23, kerops/ops/linear/relu_linear_add.py:10-19,
kerops/ops/linear/relu_linear_backward.py:10-24, kerops/ops/linear/linear_bias_relu_linear_add.py:10-26,
kerops/ops/linear/linear_bias_relu_linear_backward.py:10-19.  Each call must run and return what the call
without knobs returns (the stream ops and the forward convolution bit for bit; sums whose addition order
follows the launch shape to rounding).
"""
import pytest
import torch

from conftest import cpu_gen, rand_cl3d, rand_dw_weight
from kerops_amd.ops._common import BUILT_WAVES, nearest_conv_shape, stream_waves
from kerops_amd.ops.conv.variants import FWD_VARIANTS, WGRAD_VARIANTS

DEV = 'cuda'

# the reference's launch tables
REF_DWCONV_WARPS = {8: 1, 16: 2, 32: 2, 64: 2, 128: 4}
REF_DWCONV_DBLOCK = {8: 32, 16: 32, 32: 16, 64: 8, 128: 8}
REF_WGRAD_WARPS = {8: 1, 16: 1, 32: 1, 64: 1, 128: 2}
REF_WGRAD_ILP = {8: 1, 16: 1, 32: 2, 64: 3, 128: 3}
REF_L1 = 65536


def test_stream_waves_maps_every_positive_count():
    assert stream_waves(0) == 0
    assert [stream_waves(n) for n in (1, 2, 3, 4, 5, 6, 7, 8, 12, 13, 16, 32, 64)] == \
        [4, 4, 4, 4, 4, 4, 8, 8, 8, 16, 16, 16, 16]
    assert all(stream_waves(w) == w for w in BUILT_WAVES)
    with pytest.raises(AssertionError):
        stream_waves(-1)


def test_nearest_conv_shape():
    for table in (FWD_VARIANTS, WGRAD_VARIANTS):
        for c, built in table.items():
            for shape in built:
                assert nearest_conv_shape(table, c, *shape) == shape
            for d_block in (1, 2, 4, 8, 16, 32, 64, 128, 256):
                for lane_c in (16, 2):
                    got = nearest_conv_shape(table, c, 8, d_block, lane_c)
                    assert got in built and got[2] == lane_c
    # the reference's own D_block of every channel count is a built shape or maps onto one of the same family
    assert nearest_conv_shape(FWD_VARIANTS, 64, 8, 16, 16) == (4, 16, 16)
    assert nearest_conv_shape(FWD_VARIANTS, 64, 8, 1, 16)[1] == 8
    # channel counts without a table entry go through untouched: the library reports them
    assert nearest_conv_shape(FWD_VARIANTS, 256, 8, 8, 16) == (8, 8, 16)


def bits(t):
    return t.contiguous().view(torch.int16) if t.dtype == torch.float16 else t


@pytest.mark.gpu
@pytest.mark.parametrize('c', [8, 16, 32, 64, 128])
def test_conv_pair_with_reference_defaults(c):
    from kerops_amd.ops.conv import DWConv, DWConvWGRAD

    g = cpu_gen(c)
    x, gr = rand_cl3d(g, 2, c, 9, 11, 37).to(DEV), rand_cl3d(g, 2, c, 9, 11, 37).to(DEV)
    _, wk = rand_dw_weight(g, c)
    wk = wk.to(DEV)
    y0 = DWConv(x, wk)
    gw0 = DWConvWGRAD(x, gr, out_dtype=torch.float32)
    for acctype in ('float32', 'float16'):
        y = DWConv(x, wk, ACCTYPE=acctype, num_warps=REF_DWCONV_WARPS[c], D_block=REF_DWCONV_DBLOCK[c])
        assert torch.equal(bits(y), bits(y0))
        gw = DWConvWGRAD(x, gr, ACCTYPE=acctype, num_warps=REF_WGRAD_WARPS[c], D_block=REF_DWCONV_DBLOCK[c],
                         ILP=REF_WGRAD_ILP[c], out_dtype=torch.float32)
        assert torch.allclose(gw, gw0, rtol=1e-4, atol=1e-3)
    # any power-of-two D_block and any warp count the reference would take
    for d_block in (1, 2, 4, 16, 64, 128):
        for warps in (1, 3, 16):
            assert torch.equal(bits(DWConv(x, wk, num_warps=warps, D_block=d_block)), bits(y0))
            gw = DWConvWGRAD(x, gr, num_warps=warps, D_block=d_block, ILP=5, out_dtype=torch.float32)
            assert torch.allclose(gw, gw0, rtol=1e-4, atol=1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize('c', [4, 64])
def test_stream_ops_with_reference_defaults(c):
    from kerops_amd.ops.addition import AddStats, AddStatsBackward
    from kerops_amd.ops.avgpool import AvgPoolCeilStats, AvgPoolCeilStatsBackward
    from kerops_amd.ops.bnrelu import ApplyBNReLU, ApplyBNReLUBackward
    from kerops_amd.ops.quantization import DequantUint8Window, QuantUint8Window
    from kerops_amd.ops.stats import Stats, StatsBackward

    g = cpu_gen(100 + c)
    shape = (2, c, 7, 9, 13)
    x, y = rand_cl3d(g, *shape).to(DEV), rand_cl3d(g, *shape).to(DEV)
    w, b = (torch.rand(c, generator=g) + 0.5).to(DEV), (torch.randn(c, generator=g) * 0.3).to(DEV)
    mg, sg = (torch.randn(c, generator=g) / 3).to(DEV), (torch.randn(c, generator=g) / 3).to(DEV)

    def same(a, b_, exact_float=False):
        a = a if isinstance(a, tuple) else (a,)
        b_ = b_ if isinstance(b_, tuple) else (b_,)
        for u, v in zip(a, b_):
            if u.dtype == torch.float32 and not exact_float:
                assert torch.allclose(u, v, rtol=1e-5, atol=1e-5)  # sums: the addition order follows the launch shape
            else:
                assert torch.equal(bits(u), bits(v))

    # (op, positional arguments, the reference's num_warps)
    pooled, _, _ = AvgPoolCeilStats(x)
    gp = rand_cl3d(g, *pooled.shape).to(DEV)
    q = QuantUint8Window(x, 2.5)
    cases = [
        (Stats, (x,), 4), (StatsBackward, (x, mg, sg), 4),
        (ApplyBNReLU, (x, w, b), 8), (ApplyBNReLUBackward, (x, w, b, y), 8),
        (AddStats, (x, y), 8), (AddStatsBackward, (y, mg, sg, x), 8),
        (AvgPoolCeilStats, (x,), 2), (AvgPoolCeilStatsBackward, (gp, mg, sg, pooled, list(shape)), 4),
        (QuantUint8Window, (x, 2.5), 4), (DequantUint8Window, (q, torch.float16, 2.5), 4),
    ]
    for op, args, ref_warps in cases:
        base = op(*args)
        same(op(*args, num_warps=ref_warps, l1_cache_bytes=REF_L1), base)
        for warps in (1, 2, 4, 8, 16, 32):
            same(op(*args, num_warps=warps), base)
        # reconfigure, the reference's other way of setting a knob (kerops/settings/wrapper.py:74-77)
        saved = dict(op.configurators)
        try:
            op.reconfigure(**dict(saved, num_warps=ref_warps))
            same(op(*args), base)
        finally:
            op.reconfigure(**saved)


@pytest.mark.gpu
def test_linear_ops_with_reference_defaults():
    from kerops_amd.ops.linear import LinBReLULinAdd, LinBReLULinBackward, ReLULinearAdd, ReLULinearBackward

    g = cpu_gen(7)
    for c in (16, 32):
        shape = (1, c, 5, 6, 19)
        x, gr = rand_cl3d(g, *shape).to(DEV), rand_cl3d(g, *shape).to(DEV)
        wt = (torch.randn(c, c, generator=g) / c ** 0.5).half().to(DEV)
        up = (torch.randn(c, 2 * c, generator=g) / c ** 0.5).half().to(DEV)
        down = (torch.randn(2 * c, c, generator=g) / (2 * c) ** 0.5).half().to(DEV)
        bias = (torch.randn(2 * c, generator=g) * 0.1).half().to(DEV)
        ref_ilp = {16: 8, 32: 8}[c]
        assert torch.equal(bits(ReLULinearAdd(x, wt, gr, num_warps=4, D_block=16, ILP=ref_ilp)),
                           bits(ReLULinearAdd(x, wt, gr)))
        a = ReLULinearBackward(x, gr, wt, num_warps={16: 4, 32: 8}[c], D_block={16: 16, 32: 32}[c], ILP=16)
        b = ReLULinearBackward(x, gr, wt)
        assert torch.equal(bits(a[0]), bits(b[0])) and torch.equal(bits(a[1]), bits(b[1]))
        assert torch.equal(bits(LinBReLULinAdd(x, up, down, bias, gr, num_warps=4, D_block={16: 32, 32: 16}[c],
                                               ILP={16: 1, 32: 2}[c])),
                           bits(LinBReLULinAdd(x, up, down, bias, gr)))
        a = LinBReLULinBackward(x, gr, up, down, bias, num_warps=2, D_block=32, ILP={16: 8, 32: 9}[c])
        b = LinBReLULinBackward(x, gr, up, down, bias)
        for u, v in zip(a, b):
            assert torch.equal(bits(u), bits(v))
