"""DWConvBackward: input gradient and weight gradient of DWConv in one pass over x and grad.

Host side of kerops_dwconv_bwd_f16.  The reference has no counterpart: it lacks the input gradient
(a TODO at kerops/kernels/dw_conv.py:145) and computes the weight gradient with DWConvWGRAD
(kerops/ops/conv/dwconv_wgrad.py:25-79).  The result equals
(DWConv(grad, weight flipped along the three spatial axes), DWConvWGRAD(x, grad)).
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import next_power_of_2, require_cuda


@confexc(KeyError)
def served(channels):
    # the channel counts of the reference's launch tables (kerops/ops/conv/dwconv.py:10-17)
    return {8: 0, 16: 0, 32: 0, 64: 0, 128: 0}[channels]


@configure(H_chunk=lambda x: served(x.shape[1]), out_dtype=torch.float16)
def DWConvBackward(x, grad, weight, *, H_chunk: ConfigurableArg, out_dtype: ConfigurableArg):
    """x, grad (N,C,H,W,D) fp16 channels_last_3d, weight [3,3,3,C] fp16 -> (grad_x like x, grad_w [3,3,3,C]).

    H_chunk as in DWConvWGRAD: 0 = balanced split, > 0 = uniform chunks of that many rows, -g = groups of g."""
    channels = x.shape[1]

    assert x.ndim == grad.ndim == 5
    assert x.shape == grad.shape
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert grad.is_contiguous(memory_format=torch.channels_last_3d)
    assert x.dtype == grad.dtype == weight.dtype == torch.float16
    assert channels == next_power_of_2(channels)
    assert list(weight.shape) == [3, 3, 3, channels]
    require_cuda(x, grad, weight)

    weight = weight.contiguous()
    bsize, _, H, W, D = x.shape
    ws_bytes = _lib.query('kerops_dwconv_bwd_workspace_bytes', bsize, H, W, D, channels, int(H_chunk))
    ws = _lib.workspace(ws_bytes, x.device)
    grad_x = torch.empty_like(x)
    # fp32 and fp16 results are written by the library's reduction kernel; any other type is cast from fp32
    direct = out_dtype in _lib.GW_DTYPES
    grad_w = torch.empty([3, 3, 3, channels], device=x.device, dtype=out_dtype if direct else torch.float32)
    _lib.call('kerops_dwconv_bwd_f16_out', x.data_ptr(), grad.data_ptr(), weight.data_ptr(), grad_x.data_ptr(),
              grad_w.data_ptr(), _lib.GW_DTYPES[grad_w.dtype], ws.data_ptr(), ws_bytes, bsize, H, W, D, channels,
              int(H_chunk), _lib.stream_of(x))
    return grad_x, (grad_w if direct else grad_w.to(out_dtype))
