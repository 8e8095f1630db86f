"""AvgPoolCeilStats / AvgPoolCeilStatsBackward: 2x2x2 ceil-mode average pooling fused with
per-channel statistics of the pooled tensor.

Host side of kerops_avgpool_ceil_stats_f16 / kerops_avgpool_ceil_stats_bwd_f16; names,
positional arguments, asserts and results as kerops/ops/avgpool.py:11-122 of the reference.
"""
from math import ceil

import torch

from .. import _lib
from ..settings import ConfigurableArg, configure, get_l1_cache
from ..settings.stream_table import stream_knob, stream_shape
from ._common import next_power_of_2, require_cuda, stream_waves


@configure(l1_cache_bytes=get_l1_cache, num_warps=stream_knob('AvgPoolCeilStats', 'num_warps'),
           blocks=stream_knob('AvgPoolCeilStats', 'blocks'), segment=stream_knob('AvgPoolCeilStats', 'segment'))
def AvgPoolCeilStats(x, *, l1_cache_bytes: ConfigurableArg, num_warps: ConfigurableArg, blocks: ConfigurableArg,
                     segment: ConfigurableArg):
    """Returns (pooled fp16 (N,C,ceil(H/2),ceil(W/2),ceil(D/2)) channels_last_3d, mean, sqmean).

    Launch knobs: `num_warps` = 64-wide wavefronts per workgroup (built: 4, 8, 16; any other positive value, such
    as the reference's own 2, runs on the nearest built count), `blocks` = workgroups, `segment` = pooled chunks
    per thread and step (1 or 2); 0 = the library's choice.  `l1_cache_bytes` only feeds the
    reference's row-size assert below."""
    num_channels = x.shape[1]
    input_d = x.shape[-1]
    MAX_SIZE = l1_cache_bytes // x.element_size()

    # the reference's kernel holds a whole D row per program; the limit is kept so the
    # same inputs are rejected (kerops/ops/avgpool.py:20), the gfx950 kernel has none
    assert input_d * num_channels <= MAX_SIZE
    assert num_channels == next_power_of_2(num_channels)
    assert x.ndim == 5
    assert x.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(x)

    n, _, h, w, d = x.shape
    out_shape = [n] + [ceil(sh / 2) for sh in x.shape[2:]] + [num_channels]
    output = torch.empty(out_shape, dtype=torch.float16, device=x.device).permute(0, 4, 1, 2, 3)
    mean = torch.empty(num_channels, device=x.device, dtype=torch.float32)
    sqmean = torch.empty(num_channels, device=x.device, dtype=torch.float32)
    ws_bytes = _lib.query('kerops_avgpool_ceil_stats_workspace_bytes', n, h, w, d, num_channels, int(blocks))
    ws = _lib.workspace(ws_bytes, x.device)
    _lib.call('kerops_avgpool_ceil_stats_f16', x.data_ptr(), output.data_ptr(), mean.data_ptr(), sqmean.data_ptr(),
              n, h, w, d, num_channels, ws.data_ptr(), ws_bytes, int(blocks), stream_waves(num_warps), int(segment),
              _lib.stream_of(x))
    return output, mean, sqmean


@configure(blocks=stream_knob('ApplyBNReLUAvgPoolCeilStats', 'blocks'),
           num_warps=stream_knob('ApplyBNReLUAvgPoolCeilStats', 'num_warps'),
           segment=stream_knob('ApplyBNReLUAvgPoolCeilStats', 'segment'))
def ApplyBNReLUAvgPoolCeilStats(x, weight, bias, *, blocks: ConfigurableArg, num_warps: ConfigurableArg,
                                segment: ConfigurableArg):
    """ApplyBNReLU(x, weight, bias) followed by AvgPoolCeilStats in one pass over x (no reference counterpart:
    the reference composes kerops/ops/bnrelu.py:11-41 and kerops/ops/avgpool.py:11-60).  Bit-identical to the
    composition; the full-size activation is neither written nor read.  Returns (pooled, mean, sqmean)."""
    num_channels = x.shape[1]
    assert num_channels == next_power_of_2(num_channels)
    assert x.ndim == 5
    assert x.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert weight.numel() == bias.numel() == num_channels
    require_cuda(x, weight, bias)

    n, _, h, w, d = x.shape
    weight = weight.float().contiguous()
    bias = bias.float().contiguous()
    out_shape = [n] + [ceil(sh / 2) for sh in x.shape[2:]] + [num_channels]
    output = torch.empty(out_shape, dtype=torch.float16, device=x.device).permute(0, 4, 1, 2, 3)
    mean = torch.empty(num_channels, device=x.device, dtype=torch.float32)
    sqmean = torch.empty(num_channels, device=x.device, dtype=torch.float32)
    ws_bytes = _lib.query('kerops_avgpool_ceil_stats_workspace_bytes', n, h, w, d, num_channels, int(blocks))
    ws = _lib.workspace(ws_bytes, x.device)
    _lib.call('kerops_bnrelu_avgpool_ceil_stats_f16', x.data_ptr(), weight.data_ptr(), bias.data_ptr(),
              output.data_ptr(), mean.data_ptr(), sqmean.data_ptr(), n, h, w, d, num_channels, ws.data_ptr(),
              ws_bytes, int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(x))
    return output, mean, sqmean


def _backward_knob(key):
    """Table value for the gradient tensor the op writes: its tensor arguments are all of the pooled size (an eighth),
    so the class is taken from `outgrad_shape`."""
    def knob(outgrad_shape):
        voxels = 1
        for extent in outgrad_shape:
            voxels *= int(extent)
        return stream_shape('AvgPoolCeilStatsBackward', int(outgrad_shape[1]), 2 * voxels)[key]

    knob.__name__ = f'AvgPoolCeilStatsBackward_{key}'
    return knob


@configure(l1_cache_bytes=get_l1_cache, num_warps=_backward_knob('num_warps'), blocks=_backward_knob('blocks'),
           segment=_backward_knob('segment'))
def AvgPoolCeilStatsBackward(
    inpgrad,
    meangrad,
    sqmeangrad,
    output,
    outgrad_shape,
    *,
    l1_cache_bytes: ConfigurableArg,
    num_warps: ConfigurableArg,
    blocks: ConfigurableArg,
    segment: ConfigurableArg,
):
    """Gradient w.r.t. the pooling input, fp16, shape `outgrad_shape`, channels_last_3d.
    Launch knobs as for AvgPoolCeilStats."""
    MAX_SIZE = l1_cache_bytes // inpgrad.element_size()
    bsize, num_channels, h_outgrad, w_outgrad, d_outgrad = outgrad_shape

    assert d_outgrad * num_channels <= MAX_SIZE
    assert inpgrad.shape[1] == num_channels
    assert inpgrad.shape == output.shape
    assert meangrad.numel() == sqmeangrad.numel() == num_channels
    assert inpgrad.ndim == 5
    assert inpgrad.is_contiguous(memory_format=torch.channels_last_3d)
    assert output.is_contiguous(memory_format=torch.channels_last_3d)
    assert num_channels == next_power_of_2(num_channels)
    assert inpgrad.dtype == output.dtype == torch.float16
    assert meangrad.dtype == sqmeangrad.dtype == torch.float32
    assert list(inpgrad.shape[2:]) == [ceil(s / 2) for s in (h_outgrad, w_outgrad, d_outgrad)]
    assert inpgrad.shape[0] == bsize
    require_cuda(inpgrad, output, meangrad, sqmeangrad)

    outgrad = torch.empty(
        [bsize, h_outgrad, w_outgrad, d_outgrad, num_channels], dtype=torch.float16, device=inpgrad.device
    ).permute(0, 4, 1, 2, 3)
    meangrad = meangrad.contiguous()
    sqmeangrad = sqmeangrad.contiguous()
    _lib.call('kerops_avgpool_ceil_stats_bwd_f16', inpgrad.data_ptr(), meangrad.data_ptr(), sqmeangrad.data_ptr(),
              output.data_ptr(), outgrad.data_ptr(), bsize, h_outgrad, w_outgrad, d_outgrad, num_channels,
              int(blocks), stream_waves(num_warps), int(segment), _lib.stream_of(inpgrad))
    return outgrad
