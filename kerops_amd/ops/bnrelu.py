"""ApplyBNReLU / ApplyBNReLUBackward: y = relu(x * weight[c] + bias[c]) and its gradient.

Host side of kerops_bnrelu_fwd_f16 / kerops_bnrelu_bwd_f16; names, positional
arguments, asserts and results as kerops/ops/bnrelu.py:11-82 of the reference.  Folding
the batch statistics into (weight, bias) stays the caller's job, as in the reference's
own test (tests/ops/test_bn_relu.py:27-29).
"""
import torch

from .. import _lib
from ..settings import ConfigurableArg, configure, get_l1_cache
from ..settings.stream_table import stream_knob
from ._common import next_power_of_2, numel_no_channels, require_cuda, stream_waves


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('ApplyBNReLU', 'num_warps'),
           blocks=stream_knob('ApplyBNReLU', 'blocks'), segment=stream_knob('ApplyBNReLU', 'segment'))
def ApplyBNReLU(
    x, weight, bias, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg,
    segment: ConfigurableArg
):
    """y = fp16(max(x * weight[c] + bias[c], 0)).

    Launch knobs: `num_warps` = 64-wide wavefronts per workgroup (built: 4, 8, 16; any other positive value runs
    on the nearest built count), `blocks` = workgroups, `segment` = walk of the stream (1 interleaved, 4 / 8
    contiguous chunks per thread); 0 = the library's choice.
    `l1_cache_bytes` is accepted for compatibility and not used: the reference sized its blocks with it."""
    num_channels = x.shape[1]
    assert x.ndim == 5
    assert num_channels == next_power_of_2(num_channels)
    assert x.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert weight.numel() == bias.numel() == num_channels
    require_cuda(x, weight, bias)

    weight = weight.to(torch.float32).contiguous()
    bias = bias.to(torch.float32).contiguous()
    output = torch.empty_like(x)
    _lib.call('kerops_bnrelu_fwd_f16', x.data_ptr(), weight.data_ptr(), bias.data_ptr(), output.data_ptr(),
              numel_no_channels(x), num_channels, int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(x))
    return output


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('ApplyBNReLUBackward', 'num_warps'),
           blocks=stream_knob('ApplyBNReLUBackward', 'blocks'), segment=stream_knob('ApplyBNReLUBackward', 'segment'))
def ApplyBNReLUBackward(
    x, weight, bias, grad, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg,
    segment: ConfigurableArg
):
    """Returns (dx fp16, weight_grad fp32, bias_grad fp32); the two gradients keep weight's shape.
    Launch knobs as for ApplyBNReLU (`l1_cache_bytes` accepted, not used)."""
    num_channels = x.shape[1]
    assert x.ndim == 5
    assert x.shape == grad.shape
    assert num_channels == next_power_of_2(num_channels)
    assert x.dtype == grad.dtype == torch.float16
    assert weight.dtype == bias.dtype == torch.float32
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert grad.is_contiguous(memory_format=torch.channels_last_3d)
    assert weight.numel() == bias.numel() == num_channels
    require_cuda(x, weight, bias, grad)

    m = numel_no_channels(x)
    wflat = weight.detach().contiguous()
    bflat = bias.detach().contiguous()
    outgrad = torch.empty_like(x)
    weight_grad = torch.empty_like(wflat)
    bias_grad = torch.empty_like(bflat)
    ws_bytes = _lib.query('kerops_stats_workspace_bytes', m, num_channels, int(blocks))
    ws = _lib.workspace(ws_bytes, x.device)
    _lib.call('kerops_bnrelu_bwd_f16', x.data_ptr(), wflat.data_ptr(), bflat.data_ptr(), grad.data_ptr(),
              outgrad.data_ptr(), weight_grad.data_ptr(), bias_grad.data_ptr(), m, num_channels, ws.data_ptr(),
              ws_bytes, int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(x))
    return outgrad, weight_grad, bias_grad
