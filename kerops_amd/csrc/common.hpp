// Shared device/host helpers for the gfx950 kernels of kerops_amd.
//
// Data layout everywhere: a torch (N, C, H, W, D) channels_last_3d tensor is the
// dense array [N][H][W][D][C] of fp16; D is the innermost spatial axis and the
// C channels of one voxel are contiguous (2*C bytes).  All kernels move data as
// 16-byte chunks of 8 consecutive channels ("c8 chunks"): consecutive lanes of a
// 64-wide wavefront take consecutive chunks, so every global access of a
// wavefront is one contiguous 1 KiB run.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>
#include <type_traits>

#include "../../include/kerops_hip.h"

namespace kerops {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// An fp32 result that is about to be rounded to fp16, made opaque to the compiler.  Where results are specified as
// fp16(fp32 value) (two roundings, what the reference's kernels and the oracle compute), the product or fused
// multiply-add must exist as an fp32 value first: left alone, the compiler may merge it with the conversion into
// v_fma_mixlo_f16 / v_fma_mixhi_f16, which round the exact result once and differ in the last bit in rare cases.
__device__ __forceinline__ float as_fp32_value(float f)
{
    asm("" : "+v"(f));
    return f;
}
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// ---- shared by the matrix-core depthwise kernels (v_mfma_f32_4x4x4_16B_f16, one block per channel) ----
// LDS patches keep one position in PB = 2*channels bytes; inside a position the channel offset is
// rotated by 32 bytes per position so that the three or four distinct positions read by half a
// wavefront (8 channel pairs each) fall into disjoint banks.  p may be taken relative to any multiple of 4.
template <int PB>
__device__ constexpr int lds_swizzle(int p, int cb)
{
    return p * PB + ((cb + (PB >= 64 ? 32 * (p / (128 / PB)) : 0)) & (PB - 1));
}
// dwords holding two channels at consecutive positions -> the even and the odd channel's fp16x4 operand
__device__ __forceinline__ void split_operands(const uint32_t (&r)[4], half4_t& even, half4_t& odd)
{
    const u32x2_t e = {__builtin_amdgcn_perm(r[1], r[0], 0x05040100u), __builtin_amdgcn_perm(r[3], r[2], 0x05040100u)};
    const u32x2_t o = {__builtin_amdgcn_perm(r[1], r[0], 0x07060302u), __builtin_amdgcn_perm(r[3], r[2], 0x07060302u)};
    even = __builtin_bit_cast(half4_t, e);
    odd = __builtin_bit_cast(half4_t, o);
}
// the same with per-lane byte selectors (0x05040100 / 0x07060302 for live lanes): a lane whose results are never
// used passes 0x0c0c0c0c twice and gets all-zero operands, so that its share of the multipliers does not toggle
__device__ __forceinline__ void split_operands_sel(const uint32_t (&r)[4], uint32_t sel_even, uint32_t sel_odd,
                                                   half4_t& even, half4_t& odd)
{
    const u32x2_t e = {__builtin_amdgcn_perm(r[1], r[0], sel_even), __builtin_amdgcn_perm(r[3], r[2], sel_even)};
    const u32x2_t o = {__builtin_amdgcn_perm(r[1], r[0], sel_odd), __builtin_amdgcn_perm(r[3], r[2], sel_odd)};
    even = __builtin_bit_cast(half4_t, e);
    odd = __builtin_bit_cast(half4_t, o);
}
// same with three positions; the fourth operand element is zero (selector byte 0x0c yields 0x00)
__device__ __forceinline__ void split_operands3(const uint32_t (&r)[3], half4_t& even, half4_t& odd)
{
    const u32x2_t e = {__builtin_amdgcn_perm(r[1], r[0], 0x05040100u), __builtin_amdgcn_perm(0u, r[2], 0x0c0c0100u)};
    const u32x2_t o = {__builtin_amdgcn_perm(r[1], r[0], 0x07060302u), __builtin_amdgcn_perm(0u, r[2], 0x0c0c0302u)};
    even = __builtin_bit_cast(half4_t, e);
    odd = __builtin_bit_cast(half4_t, o);
}

// every lane takes the value of the previous lane of its quad (lane 0 that of lane 3): one DPP move per dword
__device__ __forceinline__ half4_t quad_rotate_up(half4_t v)
{
    u32x2_t w = __builtin_bit_cast(u32x2_t, v);
    // (every lane has a source, so the "old" operand is never kept: passing the source itself lets the move run in place)
    w[0] = (uint32_t)__builtin_amdgcn_update_dpp((int)w[0], (int)w[0], 0x93, 0xf, 0xf, false);  // quad_perm:[3,0,1,2]
    w[1] = (uint32_t)__builtin_amdgcn_update_dpp((int)w[1], (int)w[1], 0x93, 0xf, 0xf, false);
    return __builtin_bit_cast(half4_t, w);
}

constexpr int kWave = 64;

// ---- LDS-direct loads (global_load_lds_dwordx4) with hand-placed waits ------------------------------------
// The compiler neither sees these memory instructions nor counts them: a kernel that uses them issues the same
// number of them in every wavefront and step (an instruction whose mask is empty still counts) and waits with
// wait_loads_in_flight<n>, which returns when all but the newest n vector memory instructions of the wavefront
// have completed (loads and stores retire in issue order).  M0 is used by nothing else in these kernels.
// one LDS-direct load of a wavefront: lane l brings the 16 bytes at sbase + voff to LDS address lds_addr + 16*l;
// lanes outside `mask` do nothing.  sbase, lds_addr and mask are wavefront-uniform (scalar registers).
template <bool STREAM>
__device__ __forceinline__ void lds_direct_load16(const void* sbase, uint32_t voff, uint32_t lds_addr, uint64_t mask)
{
    uint64_t saved;
    if (STREAM)
        asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %2, %1 nt\n\ts_mov_b64 exec, %0"
                     : "=&s"(saved)
                     : "s"(sbase), "v"(voff), "s"(lds_addr), "s"(mask)
                     : "memory");
    else
        asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %2, %1\n\ts_mov_b64 exec, %0"
                     : "=&s"(saved)
                     : "s"(sbase), "v"(voff), "s"(lds_addr), "s"(mask)
                     : "memory");
}
template <int N>
__device__ __forceinline__ void wait_loads_in_flight()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ const char* uniform_ptr(const char* p)
{
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
}

// 16-byte streaming store of the lanes in `mask` to sbase + voff, counted like the loads above
__device__ __forceinline__ void masked_store16_stream(void* sbase, uint32_t voff, u32x4_t data, uint64_t mask)
{
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\tglobal_store_dwordx4 %2, %3, %1 nt\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "s"(sbase), "v"(voff), "v"(data), "s"(mask)
                 : "memory");
}
constexpr int64_t kStreamInteriorMinBytes = 384ll << 20;

// Order in which the 16-byte chunks of a staged plane (a TW x TD patch with its one-voxel halo, CG chunks per
// position) are shared out to the threads: first the chunks that a neighbouring patch reads as well (the halo
// ring around the patch and the patch's own border ring), then the interior, which only this workgroup reads.
// A load instruction whose chunks are all interior carries the streaming hint, so these lines do not push the
// shared ones out of the L2 before the neighbour has read them (forward kernel at 64 channels: x fetched from
// memory 1.148 -> 1.108 times, 2.5 % less time; 3 % at 16 channels).  Streaming loads do not use the 256 MB
// memory-side cache either, so the hint is for tensors that cannot stay there anyway: the launchers switch it on
// above kStreamInteriorMinBytes (with the whole 251 MB (1,8,350,350,128) tensor cached between calls the hint cost
// 34 %, with the 268 MB input of the fused block 7 %).  Runs stay whole lines: full rows of TD + 2 positions, pairs
// of positions at the sides, TD - 2 positions inside.
template <int TW, int TD, int CG>
struct HaloOrder {
    static constexpr int ROWCH = (TD + 2) * CG;                  // chunks of one staged row
    static constexpr int NSH_ROWS = 4 * ROWCH;                   // the two rows above and the two below
    static constexpr int NSH = NSH_ROWS + 4 * (TW - 2) * CG;     // ... and two positions at either side
    static constexpr int N = (TW + 2) * ROWCH;
    // chunk index -> staged row wq in [0, TW + 2), position dq in [0, TD + 2), channel chunk cq
    __device__ static __forceinline__ void decode(int ch, int& wq, int& dq, int& cq)
    {
        if (ch < NSH_ROWS) {
            const int r4 = ch / ROWCH, rem = ch - r4 * ROWCH;
            wq = r4 < 2 ? r4 : TW + r4 - 2;
            dq = rem / CG;
            cq = rem - dq * CG;
        } else if (ch < NSH) {
            const int s2 = ch - NSH_ROWS, wr = s2 / (4 * CG), rem = s2 - wr * 4 * CG, dp = rem / CG;
            wq = 2 + wr;
            dq = dp < 2 ? dp : TD + dp - 2;
            cq = rem - dp * CG;
        } else {
            const int pp = ch - NSH, wr = pp / ((TD - 2) * CG), rem = pp - wr * (TD - 2) * CG;
            wq = 2 + wr;
            dq = 2 + rem / CG;
            cq = rem % CG;
        }
    }
    // whether the load that covers the chunks [first, first + count) touches interior chunks only
    static constexpr bool interior_only(int first) { return first >= NSH; }
};

// ---- error reporting (host) -------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

// ---- device geometry (host) -------------------------------------------------
// Compute units and accelerator dies (XCDs, each with its own L2) of the current device, read once per device
// with hipDeviceGetAttribute (core.hip); without a usable device (a workspace query on a machine without a GPU)
// the MI355X's 256 / 8.  The H-marching kernels size their launch to the workgroups the device holds at once
// and walk every die's share of the tiles contiguously.
struct DeviceGeometry {
    int cus, xcds;
    // workgroups resident at once: 16 wavefronts per compute unit at the register budget of these kernels
    int resident_workgroups(int threads) const { return cus * (threads >= 512 ? 2 : 4); }
};
DeviceGeometry device_geometry();

// ---- cross-file launchers (defined in dwconv_fwd.hip / pointwise.hip) ----------------
int dwconv_fwd_run(const void* x, const void* wt, void* y, const float* scale, const float* shift, int32_t N,
                   int32_t H, int32_t W, int32_t D, int32_t C, int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                   int32_t lane_channels, void* stream);
// fused depthwise -> affine -> ReLU -> pointwise kernel (64 input channels, Cout in {64,128}); workgroup count of
// its grid (= floats of amax_ws it writes)
int dwsep_fused_blocks(int32_t N, int32_t H, int32_t W, int32_t D);
int dwsep_fused_run(const void* x, const void* wt, const float* scale, const float* shift, const void* pw, void* y2,
                    float* amax_ws, int32_t N, int32_t H, int32_t W, int32_t D, int32_t Cout, void* stream);
int pointwise_dispatch(const _Float16* x, const _Float16* Wm, const _Float16* add, _Float16* out, float* amax_ws,
                       int64_t V, int Cin, int Cout, bool relu_in, bool absmax, int blocks, hipStream_t s,
                       const float* scale = nullptr, const float* shift = nullptr);
int pointwise_blocks(int64_t V);
void launch_pw_absmax_final(const float* ws, int n, float* out, hipStream_t s);

// ---- small host helpers -----------------------------------------------------
// for a >= 0, b > 0; no intermediate sum, so extents up to the type's maximum are safe
static inline int64_t ceil_div64(int64_t a, int64_t b) { return a / b + (a % b != 0); }
static inline int ceil_div(int a, int b) { return a / b + (a % b != 0); }
static inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
// N*H*W*D*C elements (all positive) must be addressable with 64-bit byte offsets; checked before any product
// of extents is formed in 64 bits
static inline bool volume_exceeds_i64(int N, int H, int W, int D, int C)
{
    const __int128 lim = (__int128)1 << 60;
    __int128 v = (__int128)N * H * W;  // < 2^93
    if (v >= lim) return true;
    v *= D;
    if (v >= lim) return true;
    return v * C >= lim;
}
// Rows per workgroup of the H-marching convolution kernels.  All workgroups of a launch do the same work, so
// they run in ceil(workgroups / resident slots) rounds; a workgroup that marches over h rows takes h + 2 plane
// steps (two halo planes) plus a fixed cost of about `setup` plane steps (prologue, pipeline fill, epilogue).
// The split that minimises rounds * (h + 2 + setup) wins; ties go to fewer, longer chunks.  Checked against
// H_chunk sweeps of the forward and weight-gradient kernels at 14 shapes from 96^3 x 16 to 350 x 350 x 128 x 128
// channels: the choice is the sweep's optimum or within 2 % of it (a variant that charges half a round for a
// partial last round instead of a whole one was up to 15 % off).
static inline int pick_h_chunk(int H, int64_t per_plane, int slots, int setup)
{
    int best_h = H;
    double best = 1e300;
    const int max_chunks = H < 64 ? H : 64;
    for (int c = 1; c <= max_chunks; ++c) {
        const int h = ceil_div(H, c);
        const int chunks = ceil_div(H, h);
        if (chunks != c) continue;  // the same split as a smaller c
        const double rounds = std::ceil((double)per_plane * chunks / slots);  // (doubles: no overflow at absurd sizes)
        const double cost = rounds * ((double)h + 2 + setup) * (1.0 + 0.004 * c);
        if (cost < best) {
            best = cost;
            best_h = h;
        }
    }
    return best_h;
}
// Balanced split of the H-marching kernels.  The tiles of the tensor, in their linear order (slab fastest, then
// the tiles along D, along W, the batch), are cut into bundles of `group` neighbours; the launch has `ngroups`
// groups of `group` workgroups, and a group owns a contiguous share of the sequence (bundle, row): its workgroups
// march in step over the tiles of a bundle (they share halo voxels through the L2 of their XCD) and cross into
// the next bundle together.  Every group then carries the same number of plane steps whatever the tile count,
// where uniform chunks leave the last round of workgroups partly filled (2-10 % slower at the shapes measured).
// `row_len` = tiles (times slabs) in one row along D.  The group size is chosen by a cost model fitted to
// sweeps at (1, C, 350, 350, 128), C = 8..128: time ~ plane steps of a group, 10 % / (tile rows in a bundle) for
// the halo rows that neighbouring bundles no longer share in L2, 4 % for a group that does not fit one XCD, a
// fixed cost per workgroup and per crossing.
struct BalancedSplit {
    uint32_t group, ngroups;
    int64_t units;  // bundles * H
};
static inline BalancedSplit make_balanced(int H, int64_t tiles, int slots, int group)
{
    BalancedSplit b;
    b.group = (uint32_t)group;
    const int64_t bundles = tiles / group + (tiles % group != 0);
    // more plane steps than the kernels' 32-bit counters hold: any value >= 2^31 makes the callers fall back
    b.units = bundles > (1LL << 31) / H ? (1LL << 40) : bundles * H;
    // a share of fewer than 2 rows is all halo planes: use fewer groups then
    b.ngroups = (uint32_t)std::min<int64_t>(std::max(1, slots / group), std::max<int64_t>(1, b.units / 2));
    return b;
}
static inline double balanced_cost(const BalancedSplit& b, int H, int row_len, int slots, int setup, int xcds)
{
    const double share = (double)((b.units + b.ngroups - 1) / b.ngroups);
    const double crossings = share / H;  // expected bundle boundaries inside a share
    const double rows = (double)b.group / row_len;
    // a group larger than the workgroups one XCD holds is spread over several L2s (measured: 2-3 % slower)
    const double spread = (int)b.group > slots / xcds ? 1.04 : 1.0;
    return (share + 2 + setup + crossings * 5.0) * (1.0 + 0.1 / rows) * (1.0 + 0.004 * H / share) * spread;
}
// slab_mult: the group size must be a multiple of it (kernels that keep per-slab state across bundles)
static inline BalancedSplit pick_balanced(int H, int64_t tiles, int row_len, int slots, int setup, int slab_mult,
                                          int xcds)
{
    BalancedSplit best = make_balanced(H, tiles, slots, slab_mult);
    double best_cost = 1e300;
    auto consider = [&](int64_t g) {
        if (g < 1 || g > slots || g % slab_mult != 0) return;
        if (g >= tiles + row_len && g > slab_mult) return;  // more than a row of idle members
        const BalancedSplit b = make_balanced(H, tiles, slots, (int)g);
        const double c = balanced_cost(b, H, row_len, slots, setup, xcds);
        if (c < best_cost) {
            best_cost = c;
            best = b;
        }
    };
    for (int r = 1; r <= 16; ++r) consider((int64_t)r * row_len);             // whole tile rows
    for (int f = 2; f <= 8; f *= 2)                                           // parts of a long row
        if (row_len % f == 0) consider(row_len / f);
    consider(slab_mult);
    return best;
}
// offsets inside one (W, D, C) plane are 32-bit in the convolution kernels (W, D, C positive)
static inline bool plane_exceeds_i32(int W, int D, int C)
{
    const int64_t wd = (int64_t)W * D;  // < 2^62
    return wd >= (1LL << 31) || wd * C >= (1LL << 31);
}

// Device side of the two splits of the H march: the sequence of (tile, rows [hs, he)) segments of one workgroup.
// Tiles are numbered slab fastest, then along D, along W, then the batch.  Uniform chunks (group = 0): one segment,
// workgroup w = (tile inside the sample, chunk, sample).  Balanced split: the workgroup is member w % group of group
// w / group, which owns the units [u, u_end) of the (bundle of `group` tiles, row) sequence; a share that ends inside
// a bundle continues in the next one, and members beyond the last tile of a partly filled bundle skip it.  All
// values are wavefront-uniform and kept in scalar registers.
struct SegmentWalk {
    uint32_t u, u_end, member, group;
    bool first;
};
// shares of q or q + 1 units: the first r groups take the longer ones
__device__ __forceinline__ SegmentWalk segment_walk_begin(uint32_t wg, uint32_t group, uint32_t q, uint32_t r)
{
    SegmentWalk s{0u, 0u, 0u, group, true};
    if (group > 0) {
        const uint32_t g = wg / group;
        s.member = wg - g * group;
        s.u = __builtin_amdgcn_readfirstlane(g * q + min(g, r));
        s.u_end = __builtin_amdgcn_readfirstlane(s.u + q + (g < r ? 1u : 0u));
    }
    return s;
}
__device__ __forceinline__ bool segment_walk_next(SegmentWalk& s, uint32_t wg, int H, uint32_t n_tiles,
                                                  uint32_t tiles_per_sample, int n_hc, int h_chunk, uint32_t& tile,
                                                  int& hs, int& he)
{
    if (s.group > 0) {
        for (;;) {
            if (s.u >= s.u_end) return false;
            const uint32_t bundle = s.u / (uint32_t)H;
            // (the quotient comes out of a vector division: back to scalar registers)
            hs = __builtin_amdgcn_readfirstlane((int)(s.u - bundle * (uint32_t)H));
            he = (int)min((uint32_t)H, hs + (s.u_end - s.u));
            s.u += he - hs;
            tile = __builtin_amdgcn_readfirstlane(bundle * s.group + s.member);
            if (tile < n_tiles) return true;
        }
    }
    if (!s.first) return false;
    s.first = false;
    const uint32_t rest = wg / tiles_per_sample;
    const int hc = (int)(rest % (uint32_t)n_hc);
    tile = __builtin_amdgcn_readfirstlane((rest / (uint32_t)n_hc) * tiles_per_sample + wg % tiles_per_sample);
    hs = __builtin_amdgcn_readfirstlane(hc * h_chunk);
    he = min(hs + h_chunk, H);
    return true;
}

// The XCDs of the chip (8 on MI355X; the launchers pass the device's count) receive workgroups round-robin
// (workgroup b runs on XCD b % n) and each XCD has a private L2.  remap_xcd turns the hardware workgroup
// index into a logical tile index such that each XCD walks one contiguous range of
// logical tiles: neighbouring tiles (which share halo voxels) then meet in the same
// L2 instead of being fetched once per XCD.
__device__ __forceinline__ uint32_t remap_xcd(uint32_t b, uint32_t nblocks, uint32_t n_xcd)
{
    uint32_t per = (nblocks + n_xcd - 1) / n_xcd;  // logical tiles per XCD (last range may be short)
    uint32_t xcd = b % n_xcd;
    uint32_t idx = b / n_xcd;
    // ranges [xcd*per, (xcd+1)*per); the tail ranges can exceed nblocks, so the
    // grid is launched with per*n_xcd workgroups and the caller drops ids >= nblocks.
    return xcd * per + idx;
}
static inline uint32_t xcd_padded_grid(uint32_t nblocks, uint32_t n_xcd) { return ((nblocks + n_xcd - 1) / n_xcd) * n_xcd; }

// ---- 16-byte chunk access ---------------------------------------------------
__device__ __forceinline__ half8_t load_c8(const half_t* p) { return *reinterpret_cast<const half8_t*>(p); }
__device__ __forceinline__ void store_c8(half_t* p, half8_t v) { *reinterpret_cast<half8_t*>(p) = v; }

// Streaming (non-temporal) variants for data that is touched exactly once.
__device__ __forceinline__ half8_t load_c8_nt(const half_t* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(p));
}
__device__ __forceinline__ void store_c8_nt(half_t* p, half8_t v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<half8_t*>(p));
}

// ---- LDS tile for results that leave the accumulators in 8-byte pieces and LDS in 16-byte chunks ---------------
// A 32x32x16 accumulator holds, per lane (row = lane % 32, half = lane / 32), groups of four consecutive output
// channels: the 8-byte half `half` of the 16-byte chunk `chunk` of the row.  The rows leave LDS as 16-byte chunks,
// lane c taking chunk c % CPR of row c / CPR, for coalesced stores.  Measured on gfx950, LDS writes see 32 banks of
// 4 bytes (16 lanes of an 8-byte write per clock) and reads 64 (16 lanes of a 16-byte read per clock).  Rows are
// dense (2 * COLS bytes), so the 16 lanes of a read phase take 256 consecutive bytes whatever the order inside a
// row; inside a row the chunk slot and the half are flipped by bits of the row number, chosen so that the 16 rows
// of a write phase (same chunk, same half) fall on 16 different bank pairs.
template <int COLS>
struct BounceTile {
    static constexpr int CPR = COLS / 8, RB = 2 * COLS;     // chunks per row, bytes per row
    static constexpr int RPW = RB >= 128 ? 1 : 128 / RB;    // rows per 128 bytes of write banks
    static constexpr int SW = CPR < 8 ? CPR : 8;            // chunk slots that differ in their write banks
    static constexpr int BYTES = 32 * RB;
    static_assert(COLS == 16 || COLS == 32 || COLS == 64 || COLS == 128, "row widths of the built kernels");
    // byte offset of the 8-byte piece (row, chunk, half)
    __device__ static constexpr int piece(int row, int chunk, int half)
    {
        return row * RB + ((chunk ^ ((row / RPW) % SW)) * 16) + ((half ^ (((row / RPW) / SW) & 1)) * 8);
    }
    // byte offset of the 16-byte chunk (row, chunk); its two halves are swapped where halves_swapped(row)
    __device__ static constexpr int chunk16(int row, int chunk) { return row * RB + ((chunk ^ ((row / RPW) % SW)) * 16); }
    __device__ static constexpr bool halves_swapped(int row) { return (((row / RPW) / SW) & 1) != 0; }
    __device__ static half8_t read(const unsigned char* tile, int row, int chunk)
    {
        const half8_t r = *reinterpret_cast<const half8_t*>(tile + chunk16(row, chunk));
        const bool sw = halves_swapped(row);
        return half8_t{sw ? r[4] : r[0], sw ? r[5] : r[1], sw ? r[6] : r[2], sw ? r[7] : r[3],
                       sw ? r[0] : r[4], sw ? r[1] : r[5], sw ? r[2] : r[6], sw ? r[3] : r[7]};
    }
};

// ---- LDS tile of dense [voxel][channel] fp16 rows that is written as 16-byte chunks, read as 16-byte chunks of
// one voxel (matrix operands with the voxel per lane) and read transposed (operands with the channel per lane) -----
// gfx950 reads LDS transposed: ds_read_b64_tr_b16 takes, in every block of 16 lanes, the 16 x 4 matrix M of 16-bit
// values that the lanes address (lane s supplies the address of four consecutive values M[s][0..3]) and returns to
// lane i the values M[4 j + i/4][i%4], j = 0..3.  With lane s pointing at row s/4, columns 4 (s%4) .. 4 (s%4) + 3
// of a row-major tile, lane i receives column i of four consecutive rows: two such reads make the eight reduction
// values (rows 16 s + 8 (lane/32) + 0..7) of a 32x32x16 operand whose lane index is the column.
// Chunk c of row r sits in chunk slot c ^ slot(r).  slot(r) is chosen so that (measured bank structure: 64 banks
// of 4 bytes for reads, 32 for writes) the 16 rows of a 16-byte read phase that takes the same chunk of each fall
// on different banks, the four rows of a transposing read phase (64 bytes of each) likewise, and writes of whole
// rows are conflict-free by construction.
typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 fp16x4_raw_t;
__device__ __forceinline__ half4_t lds_read_tr16(const unsigned char* p)
{
    const auto q = (__attribute__((address_space(3))) fp16x4_raw_t*)(p);
    return __builtin_bit_cast(half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4f16(q));
}
template <int COLS>
struct SwizzledRows {
    static constexpr int CPR = COLS / 8, RB = 2 * COLS;
    static_assert(COLS == 16 || COLS == 32 || COLS == 64 || COLS == 128, "row widths of the built kernels");
    __device__ static constexpr int slot(int r)
    {
        return CPR == 2   ? ((r >> 3) & 1)
               : CPR == 4 ? ((r >> 2) & 3)
               : CPR == 8 ? ((((r >> 1) & 1) << 2) | ((r >> 2) & 3))
                          : (((r & 3) << 2) | ((r >> 2) & 3));
    }
    __device__ static constexpr int chunk16(int row, int chunk) { return row * RB + ((chunk ^ slot(row)) * 16); }
    // Per-lane byte offsets of the two transposing reads of reduction step 0 for the 32-column block `blk32`
    // (columns 32 blk32 + lane % 32; a 16-column tile repeats its columns); step s adds s * 16 * RB.
    __device__ static void tr_offsets(int lane, int blk32, int (&off)[2])
    {
        const int s = lane % 16, b16 = COLS >= 32 ? (lane / 16) % 2 : 0, hl = lane / 32;
        const int col = 32 * blk32 + 16 * b16 + 4 * (s % 4);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int row = 8 * hl + 4 * r + s / 4;
            off[r] = chunk16(row, col / 8) + (col % 8) * 2;
        }
    }
    __device__ static half8_t read_tr(const unsigned char* tile, const int (&off)[2], int step)
    {
        const half4_t a = lds_read_tr16(tile + step * 16 * RB + off[0]);
        const half4_t b = lds_read_tr16(tile + step * 16 * RB + off[1]);
        return half8_t{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    }
};

// ---- wavefront reductions -----------------------------------------------------
// Sum over the lanes of a wavefront whose index differs only in bits >= log2(stride_lo):
// i.e. lanes l and l' are combined when l % stride_lo == l' % stride_lo.
template <int STRIDE_LO>
__device__ __forceinline__ float wave_sum_stride(float v)
{
#pragma unroll
    for (int off = 32; off >= STRIDE_LO; off >>= 1) {
        v += __shfl_xor(v, off, 64);
    }
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        v = fmaxf(v, __shfl_xor(v, off, 64));
    }
    return v;
}

}  // namespace kerops

// ---- per-channel streaming helpers (stream_ops.hip, avgpool.hip) --------------
namespace kerops {

// V consecutive fp16 channels moved as one access; V = min(8, C).
template <int V>
struct HVec {
    typedef _Float16 type __attribute__((ext_vector_type(V)));
};
template <>
struct HVec<1> {
    struct type {
        _Float16 s;
        __device__ __forceinline__ _Float16& operator[](int) { return s; }
        __device__ __forceinline__ const _Float16& operator[](int) const { return s; }
    };
};

// Run the statement list with a constexpr `V` = min(8, C) in scope (C a power of two).
#define KEROPS_DISPATCH_V(C, ...)  \
    do {                           \
        if ((C) >= 8) {            \
            constexpr int V = 8;   \
            __VA_ARGS__;           \
        } else if ((C) == 4) {     \
            constexpr int V = 4;   \
            __VA_ARGS__;           \
        } else if ((C) == 2) {     \
            constexpr int V = 2;   \
            __VA_ARGS__;           \
        } else {                   \
            constexpr int V = 1;   \
            __VA_ARGS__;           \
        }                          \
    } while (0)

template <int V>
__device__ __forceinline__ typename HVec<V>::type ld(const _Float16* p, int64_t chunk)
{
    return *reinterpret_cast<const typename HVec<V>::type*>(p + chunk * V);
}
template <int V>
__device__ __forceinline__ void st(_Float16* p, int64_t chunk, const typename HVec<V>::type& v)
{
    *reinterpret_cast<typename HVec<V>::type*>(p + chunk * V) = v;
}
// Streaming variants for data that is touched exactly once by the kernel: the non-temporal hint
// keeps one-pass streams from displacing each other in L2 (measured on MI355X: a pure read
// stream reaches ~6.5 TB/s with the hint against ~5.9 TB/s without).
template <int V>
__device__ __forceinline__ typename HVec<V>::type ld_stream(const _Float16* p, int64_t chunk)
{
    if constexpr (V == 1) {
        return *reinterpret_cast<const typename HVec<V>::type*>(p + chunk * V);
    } else {
        return __builtin_nontemporal_load(reinterpret_cast<const typename HVec<V>::type*>(p + chunk * V));
    }
}
template <int V>
__device__ __forceinline__ void st_stream(_Float16* p, int64_t chunk, const typename HVec<V>::type& v)
{
    if constexpr (V == 1) {
        *reinterpret_cast<typename HVec<V>::type*>(p + chunk * V) = v;
    } else {
        __builtin_nontemporal_store(v, reinterpret_cast<typename HVec<V>::type*>(p + chunk * V));
    }
}

constexpr int kStreamThreads = 256;
constexpr int kStreamWaves = kStreamThreads / kWave;
constexpr int kMaxReduceChannels = 512;  // per-channel reductions: C/V <= 64 lane groups

// Default workgroup count of the persistent stream kernels.  Measured on MI355X with 256-thread
// workgroups at (1,64,350,350,128): 768 (three per CU, 3 wavefronts per SIMD) is fastest for the
// read-dominated and read+write fp16 streams, 512 for the pooling gather (whole multiples of the 256 CUs; 640 or 896 are measurably worse).
static inline int stream_blocks_default(int64_t work_items, int preferred = 768)
{
    int64_t b = ceil_div64(work_items, kStreamThreads);
    if (b > preferred) b = preferred;
    if (b < 1) b = 1;
    return (int)b;
}

// Sum NACC*V per-thread accumulators over the threads of a workgroup that own the same
// channel group (thread t owns group t % CG, CG <= 64 a power of two) and write the
// workgroup's partial [NACC][CG*V] to `dst`.  `red` is LDS of kStreamWaves*NACC*CG*V floats.
template <int NACC, int V>
__device__ __forceinline__ void block_channel_partials(float (&acc)[NACC][V], int CG, float* red, float* dst)
{
    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
    const int cols = CG * V;
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float v = acc[a][j];
            for (int off = 32; off >= CG; off >>= 1) v += __shfl_xor(v, off, 64);
            acc[a][j] = v;
        }
    if (lane < CG) {
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int j = 0; j < V; ++j) red[(wave * NACC + a) * cols + lane * V + j] = acc[a][j];
    }
    __syncthreads();
    for (int o = t; o < NACC * cols; o += kStreamThreads) {
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kStreamWaves; ++wv) s += red[wv * NACC * cols + o];
        dst[o] = s;
    }
}

// ---- launch shape of the flat stream kernels ------------------------------------------------------------
// A stream kernel walks its 16-byte chunks in steps of U chunks per thread (all U loads of a stream are issued
// before the first value is used).  With T = workgroups * threads, step k of a thread covers
//   interleaved (segment = 1): chunks k*U*T + u*T + b*threads + t          (a workgroup's chunks are T apart)
//   segments    (segment = U): chunks k*U*T + b*U*threads + u*threads + t  (a workgroup reads and writes one
//                                                                           contiguous run of U*threads chunks)
// for u < U; what is left after the last full step (< U*T chunks) is walked one chunk at a time.  Measured on
// MI355X with a plain copy of 2 GB: interleaved 256-thread workgroups reach 5.4-5.8 TB/s depending on the
// workgroup count (power-of-two counts such as 1024 fall to 4.4 TB/s: all accesses in flight then sit a
// power-of-two stride apart), 1024-thread workgroups on 128 KiB segments (U = 8) reach 6.0-6.3 TB/s whatever
// the count.  Both T and threads are multiples of the number of channel groups, so a thread keeps its group.
struct StreamShape {
    int blocks, threads, segment;  // segment: 1 = interleaved (U = 4), 4 or 8 = contiguous segments with that U
    int unroll() const { return segment == 8 ? 8 : 4; }
};
template <int U>
struct ChunkWalk {
    int64_t T, step, su, first, nfull, tail;
    __device__ __forceinline__ ChunkWalk(int64_t nchunks, bool segments)
    {
        const int64_t nthr = blockDim.x;
        T = (int64_t)gridDim.x * nthr;
        step = U * T;
        nfull = nchunks / step;
        su = segments ? nthr : T;
        first = (segments ? (int64_t)blockIdx.x * U * nthr : (int64_t)blockIdx.x * nthr) + threadIdx.x;
        tail = nfull * step + (int64_t)blockIdx.x * nthr + threadIdx.x;
    }
};
constexpr int kStreamMaxThreads = 1024;

// block_channel_partials for any workgroup size up to 1024 threads: the wavefronts hand their sums over in
// rounds of four through the same 4-slot LDS buffer; thread o keeps the running sums of the outputs
// o, o + threads, ... (at most NACC*512 / 256 = 2*NACC of them) and adds the rounds in a fixed order.
template <int NACC, int V>
__device__ __forceinline__ void block_channel_partials_any(float (&acc)[NACC][V], int CG, float* red, float* dst)
{
    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave, nthr = blockDim.x, nwaves = nthr / kWave;
    const int cols = CG * V, nout = NACC * cols;
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float v = acc[a][j];
            for (int off = 32; off >= CG; off >>= 1) v += __shfl_xor(v, off, 64);
            acc[a][j] = v;
        }
    constexpr int kMine = 2 * NACC;
    float run[kMine];
#pragma unroll
    for (int m = 0; m < kMine; ++m) run[m] = 0.0f;
    for (int r = 0; r < nwaves; r += 4) {
        if (wave >= r && wave < r + 4 && lane < CG) {
#pragma unroll
            for (int a = 0; a < NACC; ++a)
#pragma unroll
                for (int j = 0; j < V; ++j) red[((wave - r) * NACC + a) * cols + lane * V + j] = acc[a][j];
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < kMine; ++m) {
            const int o = t + m * nthr;
            if (o < nout) run[m] += (red[o] + red[nout + o]) + (red[2 * nout + o] + red[3 * nout + o]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int m = 0; m < kMine; ++m) {
        const int o = t + m * nthr;
        if (o < nout) dst[o] = run[m];
    }
}

// out[j] = scale * sum_r ws[r*ncols + j] for j < ncols, summed in fp64 in a fixed order;
// columns [0, split) go to out0, the rest to out1.  (Kernel lives in core.hip.)
void launch_reduce_rows(const float* ws, int nrows, int ncols, float* out0, float* out1, int split, double scale,
                        hipStream_t stream);
// the same with the fp32 results rounded to fp16
void launch_reduce_rows_f16(const float* ws, int nrows, int ncols, half_t* out0, half_t* out1, int split, double scale,
                            hipStream_t stream);
// result type of a gradient that a reduction kernel writes: fp32 or fp16
inline bool grad_dtype_ok(int dtype) { return dtype == KEROPS_DTYPE_F32 || dtype == KEROPS_DTYPE_F16; }

}  // namespace kerops
