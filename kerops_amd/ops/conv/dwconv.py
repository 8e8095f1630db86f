"""DWConv: depthwise 3x3x3 convolution on channels_last_3d fp16 tensors.

Host side of kerops_dwconv_fwd_f16; same name, positional arguments, asserts and
result as kerops/ops/conv/dwconv.py:20-63 of the reference.
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import cl3d, nearest_conv_shape, next_power_of_2, require_cuda
from .variants import FWD_VARIANTS

# gfx950 launch table, keyed by channel count like the reference's `warps` / `dblock`
# (kerops/ops/conv/dwconv.py:10-17): (wavefronts per workgroup, tile extent along D,
# tile extent along W).  A missing key means "no kernel for this channel count".
_WAVES = {8: 4, 16: 8, 32: 8, 64: 8, 128: 8}
_TILE_D = {8: 32, 16: 32, 32: 16, 64: 8, 128: 8}
_TILE_W = {8: 8, 16: 8, 32: 8, 64: 8, 128: 8}
# at 8 channels the patch is 8 x 64 (512 threads) when the volume is more than 32 deep
# 16 = matrix-core kernels (16 channel blocks per MFMA); 2 / 4 = vector kernels (channels per lane)
_LANE_C = {8: 16, 16: 16, 32: 16, 64: 16, 128: 16}


@confexc(KeyError)
def warps(channels, depth=None):
    return 8 if channels == 8 and depth is not None and depth > 32 else _WAVES[channels]


@confexc(KeyError)
def dblock(channels, depth=None):
    return 64 if channels == 8 and depth is not None and depth > 32 else _TILE_D[channels]


@confexc(KeyError)
def wtile(channels):
    return _TILE_W[channels]


@confexc(KeyError)
def lanec(channels):
    return _LANE_C[channels]


@configure(
    ACCTYPE='float32',
    num_warps=lambda x: warps(x.shape[1], x.shape[4]),
    D_block=lambda x: dblock(x.shape[1], x.shape[4]),
    W_block=lambda x: wtile(x.shape[1]),
    H_chunk=0,
    lane_channels=lambda x: lanec(x.shape[1]),
)
def DWConv(
    x,
    weight,
    *,
    ACCTYPE: ConfigurableArg,
    num_warps: ConfigurableArg,
    D_block: ConfigurableArg,
    W_block: ConfigurableArg,
    H_chunk: ConfigurableArg,
    lane_channels: ConfigurableArg,
):
    """y = conv3d(x, weight, padding=1, stride=1, groups=C) with weight laid out [3,3,3,C].

    ACCTYPE / num_warps / D_block keep the reference's names and accept every value the reference accepts
    (kerops/ops/conv/dwconv.py:10-17,33): accumulation is always fp32 ('float16' is accepted and computed in
    fp32); num_warps (any positive count) is accepted and not used, because the library fixes the wavefronts per
    workgroup with the patch shape (4, or 8 for 512-thread patches); D_block (any power of two) is the tile
    extent along D, and a (W_block, D_block) pair the library is not built with runs on the nearest built patch
    shape of the same kernel family.  W_block (tile extent along W), H_chunk (> 0: rows one workgroup marches
    over; 0: the balanced split, in which groups of workgroups share out the rows of all patches evenly; -g:
    that split with groups of g workgroups) and lane_channels (16 = matrix-core kernels, the default; 2 or 4 =
    vector kernels with that many channels per lane) are additional gfx950 knobs.
    """
    channels = x.shape[1]

    assert x.ndim == 5
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert x.dtype == weight.dtype == torch.float16
    assert channels == next_power_of_2(channels)
    assert list(weight.shape) == [3, 3, 3, channels]
    assert D_block == next_power_of_2(D_block)
    {'float32': None, 'float16': None}[ACCTYPE]
    assert int(num_warps) > 0
    require_cuda(x, weight)

    bsize, _, H, W, D = x.shape
    weight = weight.contiguous()
    output = torch.empty_like(x)
    assert cl3d(output)

    w_block, d_block, lane_c = nearest_conv_shape(FWD_VARIANTS, channels, W_block, D_block, lane_channels)
    _lib.call(
        'kerops_dwconv_fwd_f16', x.data_ptr(), weight.data_ptr(), output.data_ptr(), bsize, H, W, D, channels,
        w_block, d_block, int(H_chunk), lane_c, _lib.stream_of(x),
    )
    return output
