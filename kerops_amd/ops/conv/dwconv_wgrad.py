"""DWConvWGRAD: weight gradient of the depthwise 3x3x3 convolution.

Host side of kerops_dwconv_wgrad_f16; same name, positional arguments and asserts as
kerops/ops/conv/dwconv_wgrad.py:25-79 of the reference.  The reference stores fp16
partials and returns an fp16 [3,3,3,C] tensor; here the sum is fp32 end to end and is
rounded once to `out_dtype` (fp16 by default so the result type matches the reference;
fp16 and fp32 are written by the reduction kernel itself).
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import nearest_conv_shape, next_power_of_2, require_cuda
from .variants import WGRAD_VARIANTS

# gfx950 launch table, keyed by channel count like the reference's (kerops/ops/conv/dwconv_wgrad.py:10-22):
# wavefronts per workgroup, tile extents along D and W, kernel family (32 = matrix-core kernel with LDS-direct
# staging, 16 = matrix-core kernel staged through registers, 2 = vector kernel)
_WAVES = {8: 4, 16: 4, 32: 4, 64: 4, 128: 4}
_TILE_D = {8: 64, 16: 32, 32: 16, 64: 8, 128: 8}
_TILE_W = {8: 8, 16: 8, 32: 8, 64: 8, 128: 8}
_LANE_C = {8: 32, 16: 32, 32: 32, 64: 32, 128: 32}


@confexc(KeyError)
def warps(channels):
    return _WAVES[channels]


@confexc(KeyError)
def dblock(channels):
    return _TILE_D[channels]


@confexc(KeyError)
def wtile(channels):
    return _TILE_W[channels]


@confexc(KeyError)
def lanec(channels):
    return _LANE_C[channels]


@confexc(KeyError)
def ilp(channels):
    # the reference's ILP (2*ILP rows of H per program, kerops/ops/conv/dwconv_wgrad.py:20-22)
    # has no separate meaning here: a workgroup marches over H_chunk rows
    return {8: 1, 16: 1, 32: 1, 64: 1, 128: 1}[channels]


@configure(
    ACCTYPE='float32',
    num_warps=lambda x: warps(x.shape[1]),
    D_block=lambda x: dblock(x.shape[1]),
    ILP=lambda x: ilp(x.shape[1]),
    W_block=lambda x: wtile(x.shape[1]),
    H_chunk=0,
    lane_channels=lambda x: lanec(x.shape[1]),
    out_dtype=torch.float16,
)
def DWConvWGRAD(
    x,
    grad,
    *,
    ACCTYPE: ConfigurableArg,
    num_warps: ConfigurableArg,
    D_block: ConfigurableArg,
    ILP: ConfigurableArg,
    W_block: ConfigurableArg,
    H_chunk: ConfigurableArg,
    lane_channels: ConfigurableArg,
    out_dtype: ConfigurableArg,
):
    """grad_w[kh,kw,kd,c] = sum_{n,h,w,d} grad[n,c,h,w,d] * x[n,c,h+kh-1,w+kw-1,d+kd-1].

    ACCTYPE, num_warps, D_block and ILP accept every value the reference accepts
    (kerops/ops/conv/dwconv_wgrad.py:10-22,42): accumulation is always fp32; num_warps and ILP (any positive
    count) are accepted and not used (the library fixes the wavefronts per workgroup with the patch shape, and
    a workgroup marches over rows of H instead of 2*ILP of them); a (W_block, D_block) pair the library is not
    built with runs on the nearest built patch shape of the same kernel family.
    H_chunk > 0: rows one workgroup marches over; 0: the balanced split (groups of workgroups share out the
    rows of all patches evenly); -g: that split with groups of g workgroups.  The split fixes the order of the
    fp32 additions: the same call always returns the same bits, different splits differ in the last bits.
    """
    channels = x.shape[1]

    assert x.ndim == grad.ndim == 5
    assert x.shape == grad.shape
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert grad.is_contiguous(memory_format=torch.channels_last_3d)
    assert x.dtype == grad.dtype == torch.float16
    assert channels == next_power_of_2(channels)
    assert D_block == next_power_of_2(D_block)
    {'float32': None, 'float16': None}[ACCTYPE]
    assert int(num_warps) > 0 and int(ILP) > 0
    require_cuda(x, grad)

    bsize, _, H, W, D = x.shape
    w_block, d_block, lane_c = nearest_conv_shape(WGRAD_VARIANTS, channels, W_block, D_block, lane_channels)
    cfg = (w_block, d_block, int(H_chunk), lane_c)
    ws_bytes = _lib.query('kerops_dwconv_wgrad_workspace_bytes', bsize, H, W, D, channels, *cfg)
    ws = _lib.workspace(ws_bytes, x.device)
    # fp32 and fp16 results are written by the library's reduction kernel; any other type is cast from fp32
    direct = out_dtype in _lib.GW_DTYPES
    grad_w = torch.empty([3, 3, 3, channels], device=x.device, dtype=out_dtype if direct else torch.float32)

    _lib.call(
        'kerops_dwconv_wgrad_f16_out', x.data_ptr(), grad.data_ptr(), grad_w.data_ptr(),
        _lib.GW_DTYPES[grad_w.dtype], ws.data_ptr(), ws_bytes, bsize, H, W, D, channels, *cfg, _lib.stream_of(x),
    )
    return grad_w if direct else grad_w.to(out_dtype)
