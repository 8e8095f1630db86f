"""AddStats / AddStatsBackward: fp16 residual add fused with per-channel statistics.

Host side of kerops_add_stats_f16 / kerops_add_stats_bwd_f16; names, positional
arguments, asserts and results as kerops/ops/addition.py:11-88 of the reference.
"""
import torch

from .. import _lib
from ..settings import ConfigurableArg, configure, get_l1_cache
from ..settings.stream_table import stream_knob
from ._common import next_power_of_2, numel_no_channels, require_cuda, stream_waves


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('AddStats', 'num_warps'),
           blocks=stream_knob('AddStats', 'blocks'), segment=stream_knob('AddStats', 'segment'))
def AddStats(
    x, y, inplace=False, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg,
    segment: ConfigurableArg
):
    """Returns (x + y as fp16, mean, sqmean); with inplace=True the sum overwrites x.
    Launch knobs: `num_warps` = wavefronts per workgroup (built: 4, 8, 16; any other positive value runs on the
    nearest built count), `blocks` = workgroups, `segment` = walk of the stream (1 interleaved, 4 / 8 contiguous
    chunks per thread); 0 = the library's choice.  `l1_cache_bytes` is accepted and not used."""
    num_channels = x.shape[1]
    assert x.shape == y.shape
    assert x.ndim == y.ndim == 5
    assert num_channels == next_power_of_2(num_channels)
    assert x.dtype == y.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert y.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(x, y)

    m = numel_no_channels(x)
    output = x if inplace else torch.empty_like(x)
    ws_bytes = _lib.query('kerops_stats_workspace_bytes', m, num_channels, int(blocks))
    ws = _lib.workspace(ws_bytes, x.device)
    mean = torch.empty(num_channels, dtype=torch.float32, device=x.device)
    sqmean = torch.empty(num_channels, dtype=torch.float32, device=x.device)
    _lib.call('kerops_add_stats_f16', x.data_ptr(), y.data_ptr(), output.data_ptr(), mean.data_ptr(),
              sqmean.data_ptr(), m, num_channels, ws.data_ptr(), ws_bytes, int(blocks), stream_waves(num_warps),
              int(segment), _lib.stream_of(x))
    return output, mean, sqmean


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('AddStatsBackward', 'num_warps', 'add_grad'),
           blocks=stream_knob('AddStatsBackward', 'blocks', 'add_grad'),
           segment=stream_knob('AddStatsBackward', 'segment', 'add_grad'))
def AddStatsBackward(
    add_grad,
    mean_grad,
    sqmean_grad,
    add_result,
    *,
    l1_cache_bytes: ConfigurableArg,
    num_warps: ConfigurableArg,
    blocks: ConfigurableArg,
    segment: ConfigurableArg,
):
    """grad = add_grad + 2*add_result*sqmean_grad/M + mean_grad/M as fp16.  Launch knobs as for AddStats."""
    num_channels = add_grad.shape[1]
    assert add_result.shape == add_grad.shape
    assert add_grad.ndim == add_result.ndim == 5
    assert num_channels == next_power_of_2(num_channels)
    assert add_grad.dtype == add_result.dtype == torch.float16
    assert mean_grad.numel() == sqmean_grad.numel() == num_channels
    assert add_grad.is_contiguous(memory_format=torch.channels_last_3d)
    assert add_result.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(add_grad, add_result, mean_grad, sqmean_grad)

    mean_grad = mean_grad.to(torch.float32).contiguous()
    sqmean_grad = sqmean_grad.to(torch.float32).contiguous()
    output_grad = torch.empty_like(add_grad)
    _lib.call('kerops_add_stats_bwd_f16', add_grad.data_ptr(), mean_grad.data_ptr(), sqmean_grad.data_ptr(),
              add_result.data_ptr(), output_grad.data_ptr(), numel_no_channels(add_grad), num_channels, int(blocks),
              stream_waves(num_warps), int(segment), _lib.stream_of(add_grad))
    return output_grad
