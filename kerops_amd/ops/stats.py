"""Stats / StatsBackward: per-channel mean and mean of squares, and their gradient.

Host side of kerops_stats_f16 / kerops_stats_bwd_f16; names, positional arguments,
asserts and results as kerops/ops/stats.py:11-63 of the reference.
"""
import torch

from .. import _lib
from ..settings import ConfigurableArg, configure, get_l1_cache
from ..settings.stream_table import stream_knob
from ._common import next_power_of_2, numel_no_channels, require_cuda, stream_waves


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('Stats', 'num_warps'),
           blocks=stream_knob('Stats', 'blocks'), segment=stream_knob('Stats', 'segment'))
def Stats(x, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg,
          segment: ConfigurableArg):
    """Returns (mean, sqmean), fp32 [C], over every axis but channels.

    Launch knobs: `num_warps` = 64-wide wavefronts per workgroup (built: 4, 8, 16; any other positive value runs
    on the nearest built count), `blocks` = workgroups of the persistent loop, `segment` = walk of the stream
    (1 interleaved, 4 / 8 contiguous chunks per thread);
    0 = the library's choice.  `l1_cache_bytes` keeps the reference's name, is accepted and not used.
    """
    num_channels = x.shape[1]
    assert x.ndim == 5
    assert num_channels == next_power_of_2(num_channels)
    assert x.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(x)

    m = numel_no_channels(x)
    ws_bytes = _lib.query('kerops_stats_workspace_bytes', m, num_channels, int(blocks))
    ws = _lib.workspace(ws_bytes, x.device)
    mean = torch.empty(num_channels, dtype=torch.float32, device=x.device)
    sqmean = torch.empty(num_channels, dtype=torch.float32, device=x.device)
    _lib.call('kerops_stats_f16', x.data_ptr(), mean.data_ptr(), sqmean.data_ptr(), m, num_channels, ws.data_ptr(),
              ws_bytes, int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(x))
    return mean, sqmean


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('StatsBackward', 'num_warps'),
           blocks=stream_knob('StatsBackward', 'blocks'), segment=stream_knob('StatsBackward', 'segment'))
def StatsBackward(
    x, mean_grad, sqmean_grad, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg,
    segment: ConfigurableArg
):
    """dx = 2*x*sqmean_grad/M + mean_grad/M as fp16, M = numel / C.  Launch knobs as for Stats."""
    num_channels = x.shape[1]
    assert x.ndim == 5
    assert num_channels == next_power_of_2(num_channels)
    assert x.dtype == torch.float16
    assert mean_grad.numel() == sqmean_grad.numel() == num_channels
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(x, mean_grad, sqmean_grad)

    mean_grad = mean_grad.to(torch.float32).contiguous()
    sqmean_grad = sqmean_grad.to(torch.float32).contiguous()
    output_grad = torch.empty_like(x)
    _lib.call('kerops_stats_bwd_f16', x.data_ptr(), mean_grad.data_ptr(), sqmean_grad.data_ptr(),
              output_grad.data_ptr(), numel_no_channels(x), num_channels, int(blocks), stream_waves(num_warps),
              int(segment), _lib.stream_of(x))
    return output_grad
