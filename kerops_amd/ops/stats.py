"""Stats / StatsBackward: per-channel mean and mean of squares, and their gradient.

Host side of kerops_stats_f16 / kerops_stats_bwd_f16; names, positional arguments,
asserts and results as kerops/ops/stats.py:11-63 of the reference.
"""
import torch

from .. import _lib
from ..settings import ConfigurableArg, configure, get_l1_cache
from ._common import next_power_of_2, numel_no_channels, require_cuda


@configure(l1_cache_bytes=get_l1_cache, num_warps=4, blocks=0)
def Stats(x, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg):
    """Returns (mean, sqmean), fp32 [C], over every axis but channels.

    l1_cache_bytes / num_warps keep the reference's names; the gfx950 kernel is a
    persistent grid-stride stream of 4-wavefront workgroups and `blocks` (0 = one
    full wave of workgroups over the chip) is its only launch knob.
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
              ws_bytes, int(blocks), _lib.stream_of(x))
    return mean, sqmean


@configure(l1_cache_bytes=get_l1_cache, num_warps=4, blocks=0)
def StatsBackward(
    x, mean_grad, sqmean_grad, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg
):
    """dx = 2*x*sqmean_grad/M + mean_grad/M as fp16, M = numel / C."""
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
              output_grad.data_ptr(), numel_no_channels(x), num_channels, int(blocks), _lib.stream_of(x))
    return output_grad
