"""Launch shapes the library is built with, per channel count: (W_block, D_block, lane_channels).

lane_channels 16 = matrix-core kernels, 2 / 4 = vector kernels with that many channels per lane; for the weight
gradient 32 = matrix-core kernel with LDS-direct staging and 8-byte operand reads (33 / 34 / 35: the same with
(1,1) / (2,2) / (1,2) planes of x and g ahead of the arithmetic instead of the built-in choice).
These mirror the case tables at the end of csrc/dwconv_fwd.hip and csrc/dwconv_wgrad.hip; the parity
tests run every entry and `kerops_amd.tune` times them.
"""
FWD_VARIANTS = {
    8: [(16, 32, 4), (16, 32, 2), (8, 32, 16), (8, 64, 16)],
    16: [(8, 32, 4), (8, 32, 2), (8, 16, 16), (8, 32, 16)],
    32: [(8, 16, 4), (8, 16, 2), (4, 16, 16), (8, 16, 16)],
    64: [(4, 8, 4), (4, 8, 2), (4, 16, 2), (8, 8, 2), (4, 8, 16), (8, 8, 16), (4, 16, 16)],
    128: [(4, 8, 4), (4, 8, 2), (4, 16, 2), (8, 8, 2), (4, 8, 16), (8, 8, 16), (4, 16, 16)],
}
WGRAD_VARIANTS = {
    8: [(16, 32, 2), (8, 32, 2), (8, 32, 16), (8, 64, 16), (8, 64, 32), (8, 64, 33), (8, 64, 34), (8, 64, 35), (4, 64, 32), (4, 64, 33), (4, 64, 34), (4, 64, 35)],
    16: [(8, 32, 2), (8, 16, 2), (8, 16, 16), (8, 32, 16), (8, 32, 32), (8, 32, 33), (8, 32, 34), (8, 32, 35), (4, 32, 32), (4, 32, 33), (4, 32, 34), (4, 32, 35)],
    32: [(8, 16, 2), (4, 16, 2), (4, 16, 16), (8, 16, 16), (8, 16, 32), (8, 16, 33), (8, 16, 34), (8, 16, 35), (4, 16, 32), (4, 16, 33), (4, 16, 34), (4, 16, 35)],
    64: [(8, 8, 2), (4, 16, 2), (4, 8, 2), (4, 8, 16), (8, 8, 16), (4, 16, 16), (8, 8, 32), (8, 8, 33), (8, 8, 34), (8, 8, 35), (4, 8, 32), (4, 8, 33), (4, 8, 34), (4, 8, 35)],
    128: [(8, 8, 2), (4, 16, 2), (4, 8, 2), (4, 8, 16), (8, 8, 16), (4, 16, 16), (8, 8, 32), (8, 8, 33), (8, 8, 34), (8, 8, 35), (4, 8, 32), (4, 8, 33), (4, 8, 34), (4, 8, 35)],
}


def threads_per_workgroup(channels, w_block, d_block, lane_channels):
    """Workgroup size the library uses for a launch shape (fixed per shape inside the library)."""
    if lane_channels >= 32:
        return 256  # LDS-direct weight gradient: four wavefronts, each with four (8-row patches) or two g rows
    if lane_channels >= 16:
        slab = min(channels, 64)
        return 512 if w_block * d_block * slab // 8 >= 512 else 256
    return 512 if (channels >= 64 and w_block == 8 and d_block == 8) else 256
