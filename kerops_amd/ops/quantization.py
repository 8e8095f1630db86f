"""QuantUint8Window / DequantUint8Window (reference formula) and the symmetric per-tensor
int8 quantiser of the fused depthwise-separable block.

Host side of kerops_quant_u8_window / kerops_dequant_u8_window / kerops_absmax_f16 /
kerops_quant_i8_sym_f16.  The first two keep names, positional arguments and results of
kerops/ops/quantization.py:9-35 of the reference.  There `DequantUint8Window` declares its
configurable arguments without the `*` marker, which the reference's own signature check
(kerops/settings/utils.py:12-15) rejects at import; they are keyword-only here, as in
`QuantUint8Window`.
"""
import torch

from .. import _lib
from ..settings import ConfigurableArg, configure, get_l1_cache
from ..settings.stream_table import stream_knob
from ._common import require_cuda, stream_waves


def _dense(x):
    """The kernels are flat streams: any dense layout works, strides are kept by empty_like."""
    return x.is_contiguous() or (x.ndim == 5 and x.is_contiguous(memory_format=torch.channels_last_3d)) or (
        x.ndim == 4 and x.is_contiguous(memory_format=torch.channels_last)
    )


@configure(num_warps=stream_knob('QuantUint8Window', 'num_warps'), l1_cache_bytes=get_l1_cache,
           blocks=stream_knob('QuantUint8Window', 'blocks'), segment=stream_knob('QuantUint8Window', 'segment'))
def QuantUint8Window(x, window, *, num_warps: ConfigurableArg, l1_cache_bytes: ConfigurableArg,
                     blocks: ConfigurableArg, segment: ConfigurableArg):
    """u8 = trunc((clip(x, -window, window) + window) / (2*window) * 255), fp32 arithmetic; x fp16, bf16 or fp32.

    Launch knobs: `num_warps` = wavefronts per workgroup (built: 4, 8, 16; any other positive value runs on the
    nearest built count), `blocks` = workgroups, `segment` = walk of the stream (1 interleaved, 4 / 8 contiguous
    pieces per thread); 0 = the library's choice.  `l1_cache_bytes` is accepted and not used."""
    require_cuda(x)
    assert x.dtype in _lib.DTYPE_TAGS, 'fp16, bf16 or fp32 input'
    assert _dense(x)
    output = torch.empty_like(x, dtype=torch.uint8)
    _lib.call('kerops_quant_u8_window', x.data_ptr(), _lib.DTYPE_TAGS[x.dtype], output.data_ptr(), x.numel(),
              float(window), int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(x))
    return output


@configure(num_warps=stream_knob('DequantUint8Window', 'num_warps'), l1_cache_bytes=get_l1_cache,
           blocks=stream_knob('DequantUint8Window', 'blocks'), segment=stream_knob('DequantUint8Window', 'segment'))
def DequantUint8Window(x, init_dtype, window, *, num_warps: ConfigurableArg, l1_cache_bytes: ConfigurableArg,
                       blocks: ConfigurableArg, segment: ConfigurableArg):
    """x_hat = float(u8) * (2*window/255) - window, stored as `init_dtype` (fp16, bf16 or fp32).
    Launch knobs as for QuantUint8Window."""
    require_cuda(x)
    assert x.dtype == torch.uint8
    assert init_dtype in _lib.DTYPE_TAGS, 'fp16, bf16 or fp32 output'
    assert _dense(x)
    output = torch.empty_like(x, dtype=init_dtype)
    _lib.call('kerops_dequant_u8_window', x.data_ptr(), output.data_ptr(), _lib.DTYPE_TAGS[init_dtype], x.numel(),
              float(window), int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(x))
    return output


@configure(blocks=0)
def AbsMax(y, *, blocks: ConfigurableArg):
    """max |y| of an fp16 tensor as a 1-element fp32 device tensor (no host sync)."""
    require_cuda(y)
    assert y.dtype == torch.float16
    assert _dense(y)
    ws_bytes = _lib.query('kerops_absmax_workspace_bytes', int(blocks))
    ws = _lib.workspace(ws_bytes, y.device)
    out = torch.empty(1, dtype=torch.float32, device=y.device)
    _lib.call('kerops_absmax_f16', y.data_ptr(), out.data_ptr(), y.numel(), ws.data_ptr(), ws_bytes, int(blocks),
              _lib.stream_of(y))
    return out


@configure(blocks=stream_knob('QuantInt8Sym', 'blocks', 'y'), num_warps=stream_knob('QuantInt8Sym', 'num_warps', 'y'),
           segment=stream_knob('QuantInt8Sym', 'segment', 'y'))
def QuantInt8Sym(y, absmax=None, *, blocks: ConfigurableArg, num_warps: ConfigurableArg, segment: ConfigurableArg):
    """Symmetric per-tensor int8: scale = absmax/127, q = clamp(rint(y/scale), -127, 127).

    Rounding is half-to-even.  `absmax` is a 1-element fp32 device tensor (computed with
    AbsMax when omitted).  Returns (q int8 with y's strides, scale fp32 1-element tensor).
    """
    require_cuda(y)
    assert y.dtype == torch.float16
    assert _dense(y)
    if absmax is None:
        absmax = AbsMax(y)
    assert absmax.dtype == torch.float32 and absmax.numel() == 1 and absmax.is_cuda
    q = torch.empty_like(y, dtype=torch.int8)
    scale = torch.empty_like(absmax)  # absmax / 127, written by the quantising kernel
    _lib.call('kerops_quant_i8_sym_f16', y.data_ptr(), absmax.data_ptr(), q.data_ptr(), scale.data_ptr(), y.numel(),
              int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(y))
    return q, scale
