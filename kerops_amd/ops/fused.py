"""Fused depthwise-separable block of the int8 configuration (no single reference counterpart):

    t = fp16(relu(DWConv(x, dw_weight) * scale[c] + shift[c]))
    y = fp16(t @ pw_weight)                  (1x1x1 conv on the matrix cores)
    q = symmetric per-tensor int8 of y       (scale = max|y| / 127, round half to even)

`PointwiseLinear` is the bare 1x1x1 GEMM; `DWSepBlock` returns (y, max|y|); `DWSepBlockInt8`
adds the quantisation pass and returns (q, scale).  Host side of kerops_dwsep_block_f16,
kerops_pointwise_f16 and kerops_quant_i8_sym_f16.
"""
import torch

from .. import _lib
from ..settings import ConfigurableArg, configure
from ._common import require_cuda
from .quantization import QuantInt8Sym


def PointwiseLinear(x, weight, relu_in=False):
    """x (N,Cin,H,W,D) fp16 channels_last_3d, weight [Cin, Cout] fp16 -> (N,Cout,H,W,D) fp16."""
    assert x.ndim == 5 and x.dtype == weight.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    cin, cout = weight.shape
    assert x.shape[1] == cin
    require_cuda(x, weight)
    n, _, h, w, d = x.shape
    weight = weight.contiguous()  # bound to a name: a copy must outlive the launch
    out = torch.empty([n, h, w, d, cout], dtype=torch.float16, device=x.device).permute(0, 4, 1, 2, 3)
    _lib.call('kerops_pointwise_f16', x.data_ptr(), weight.data_ptr(), None, out.data_ptr(),
              n * h * w * d, cin, cout, 1 if relu_in else 0, _lib.stream_of(x))
    return out


@configure(reserved=0)
def DWSepBlock(x, dw_weight, scale, shift, pw_weight, *, reserved: ConfigurableArg):
    """Returns (y fp16 (N,Cout,H,W,D) channels_last_3d, absmax fp32 1-element device tensor)."""
    assert x.ndim == 5 and x.dtype == dw_weight.dtype == pw_weight.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    n, cin, h, w, d = x.shape
    assert list(dw_weight.shape) == [3, 3, 3, cin]
    assert pw_weight.shape[0] == cin
    assert scale.numel() == shift.numel() == cin
    cout = pw_weight.shape[1]
    require_cuda(x, dw_weight, scale, shift, pw_weight)

    scale = scale.to(torch.float32).contiguous()
    shift = shift.to(torch.float32).contiguous()
    # bound to names: copies of non-contiguous weights must outlive the launch
    dw_weight = dw_weight.contiguous()
    pw_weight = pw_weight.contiguous()
    ws_bytes = _lib.query('kerops_dwsep_block_workspace_bytes', n, h, w, d, cin, cout)
    ws = _lib.workspace(ws_bytes, x.device)
    y = torch.empty([n, h, w, d, cout], dtype=torch.float16, device=x.device).permute(0, 4, 1, 2, 3)
    absmax = torch.empty(1, dtype=torch.float32, device=x.device)
    _lib.call('kerops_dwsep_block_f16', x.data_ptr(), dw_weight.data_ptr(), scale.data_ptr(),
              shift.data_ptr(), pw_weight.data_ptr(), y.data_ptr(), absmax.data_ptr(), n, h, w, d, cin,
              cout, ws.data_ptr(), ws_bytes, _lib.stream_of(x))
    return y, absmax


def DWSepBlockInt8(x, dw_weight, scale, shift, pw_weight):
    """Returns (q int8 like y, quantisation scale fp32 1-element tensor, y)."""
    y, absmax = DWSepBlock(x, dw_weight, scale, shift, pw_weight)
    q, qscale = QuantInt8Sym(y, absmax)
    return q, qscale, y
