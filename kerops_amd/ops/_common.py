"""Helpers shared by the op wrappers."""
import torch


def next_power_of_2(n):
    """Smallest power of two >= n (n >= 1)."""
    return 1 if n <= 1 else 1 << (int(n) - 1).bit_length()


def numel_no_channels(x):
    return x.numel() // x.shape[1]


def require_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                'kerops_amd ops run only on a ROCm device (got a tensor on '
                f'{t.device}); there is no CPU path'
            )


def cl3d(t):
    return t.is_contiguous(memory_format=torch.channels_last_3d)


# wavefront counts the stream kernels are built with
BUILT_WAVES = (4, 8, 16)


def stream_waves(num_warps):
    """Wavefronts per workgroup for a value of the reference's `num_warps` knob.

    The reference accepts any positive count of 32-wide warps (its own defaults are 1, 2, 4 and 8:
    kerops/ops/avgpool.py:13, kerops/ops/stats.py:11, kerops/ops/bnrelu.py:11); the stream kernels are built
    with 4, 8 or 16 wavefronts of 64 lanes.  Every reference-valid value is mapped to the nearest built count
    (ties go to the smaller one); 0 leaves the choice to the library."""
    n = int(num_warps)
    if n == 0:
        return 0
    assert n > 0, 'num_warps must be positive'
    return min(BUILT_WAVES, key=lambda w: (abs(w - n), w))


def nearest_conv_shape(variants, channels, w_block, d_block, lane_channels):
    """(W_block, D_block, lane_channels) of the built launch shape closest to the request.

    The reference accepts any power-of-two D_block (kerops/ops/conv/dwconv.py:33); the library is built with a
    few patch shapes per channel count.  A request that is not built runs on the built shape of the same kernel
    family (lane_channels) whose D extent, then W extent, is nearest in log2; channel counts without a table
    entry are left alone so that the library reports them."""
    built = variants.get(channels)
    req = (int(w_block), int(d_block), int(lane_channels))
    if not built or req in built:
        return req
    family = [v for v in built if v[2] == req[2]] or built

    def log2_dist(a, b):
        return abs(max(int(a), 1).bit_length() - max(int(b), 1).bit_length())

    return min(family, key=lambda v: (log2_dist(v[1], req[1]), log2_dist(v[0], req[0]), v))
