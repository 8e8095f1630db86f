// Arguments shared by the weight-gradient and fused-backward kernels of dwconv_wgrad.hip and dwconv_wgrad_dma.hip.
#pragma once

#include "common.hpp"

namespace kerops {

struct WgArgs {
    const half_t* x;
    const half_t* g;
    float* ws;
    const half_t* wt;  // fused backward only: the forward weight [3][3][3][C]
    half_t* dx;        // fused backward only: the input gradient
    int H, W, D, C;
    int n_wt, n_dt, n_hc, n_slab, h_chunk;
    uint32_t nblocks;
    // balanced split (matrix-core weight-gradient kernel): bal_group > 0 switches it on, see pick_balanced
    uint32_t bal_group, bal_q, bal_r;  // workgroups per group; bundles * H plane steps = groups * bal_q + bal_r
    uint32_t n_tiles;                  // tiles in the tensor
    uint32_t n_xcd;                    // accelerator dies of the device: the logical workgroup order follows them
    int stream_interior;               // host side only: selects the kernels built with the streaming hint (NTI)
};

// dwconv_wgrad_dma.hip: launches the LDS-direct matrix-core weight-gradient kernel for (channel groups of 8 per slab,
// patch W, patch D) if it is built with that shape (`depth` = planes ahead: 0 = built-in choice, 11 / 22 / 12 = x and
// g planes ahead); the partials go to a.ws like those of the other kernels.  Returns 1 if no kernel has that shape.
int launch_wgrad_dma(const WgArgs& a, int cg, int tile_w, int tile_d, int depth, hipStream_t stream);


// dwconv_bwd_dma.hip: launches the LDS-direct fused backward kernel for (channel groups of 8 per slab, patch W, patch D)
// if it is built with that shape; dx is written, the weight-gradient partials go to a.ws.  Returns 1 otherwise.
int launch_bwd_dma(const WgArgs& a, int cg, int tile_w, int tile_d, hipStream_t stream);

}  // namespace kerops
