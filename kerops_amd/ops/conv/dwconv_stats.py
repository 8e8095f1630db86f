"""DWConvStats: DWConv with the batch statistics of its output taken in the same pass.

Host side of kerops_dwconv_stats_f16.  An addition to the reference's op set: it returns what
DWConv (kerops/ops/conv/dwconv.py:20-63) followed by Stats (kerops/ops/stats.py:11-38) on the
result return, without reading the output again.
"""
import torch

from ... import _lib
from .._common import cl3d, next_power_of_2, require_cuda


def DWConvStats(x, weight):
    """Returns (y, mean, sqmean): y = DWConv(x, weight) (bit-identical), mean / sqmean = Stats(y)
    (fp32, per channel; fp32 partial sums per workgroup, added in fp64 in a fixed order)."""
    channels = x.shape[1]

    assert x.ndim == 5
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert x.dtype == weight.dtype == torch.float16
    assert channels == next_power_of_2(channels)
    assert list(weight.shape) == [3, 3, 3, channels]
    require_cuda(x, weight)

    bsize, _, H, W, D = x.shape
    weight = weight.contiguous()
    output = torch.empty_like(x)
    assert cl3d(output)
    mean = torch.empty(channels, dtype=torch.float32, device=x.device)
    sqmean = torch.empty(channels, dtype=torch.float32, device=x.device)
    nbytes = _lib.query('kerops_dwconv_stats_workspace_bytes', bsize, H, W, D, channels)
    workspace = _lib.workspace(nbytes, x.device)

    _lib.call(
        'kerops_dwconv_stats_f16', x.data_ptr(), weight.data_ptr(), output.data_ptr(), mean.data_ptr(),
        sqmean.data_ptr(), workspace.data_ptr(), nbytes, bsize, H, W, D, channels, _lib.stream_of(x),
    )
    return output, mean, sqmean
