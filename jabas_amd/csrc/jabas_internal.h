// Shared between the C-ABI front (api.hip) and the per-K kernel translation units
// (fused_kernel.hip compiled once per JABAS_K). Not part of the public interface.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include "jabas_sync.h"

namespace jabas {

// Launch shape: threads per workgroup and tiles per workgroup (a tile = one 16-byte fp32 vector per
// thread; a chunk = the tiles one workgroup processes). Small chunks keep the streamed window of every
// buffer compact (higher HBM rate) and cut the ramp-up / drain of a launch; kernels that carry many
// statistics have low occupancy and a long epilogue, and do better with more work per workgroup.
// Measured per kernel family (A/B builds of the whole library, every shape passes the parity suite):
//   full statistics rows          256 threads x 2 tiles (K <= 4) or 4 tiles (K > 4); 64, 128, 512 and
//                                 1024 threads were all slower (-2 ... -15 %)
//   similarity sums only          256 threads x 2 tiles: with four sums the K > 4 kernels fit 4 waves per SIMD
//                                 with two tiles of loads in flight
//   plain with optimizer, K > 4   256 threads x 2 tiles: +1 % over 512 x 1 and 512 x 2, +3 % over 256 x 4;
//                                 aggregate-only launches stay at 256 x 4
//   plain, Adam kinds, K <= 4     256 threads x 4 tiles, all loads of the chunk in flight at once: +0.5 ... +1.4 %
//                                 over 256 x 2 (8 tiles: -4 %)
//   plain, SGD, fp32, K <= 4      128 threads x 2 tiles: +2 ... +5 % over 256 x 2; 128 x 4 loses 5 % on the short
//                                 ResNet-50 launch when the buffers rotate out of the last-level cache (and reads
//                                 2 % faster than 128 x 2 when they do not: size sweeps over one buffer set mislead)
//   plain, everything else K <= 4 256 threads x 2 tiles
// (these figures are from after the planned launches began to read their tables through the constant address
// space; before that the plain K > 4 kernels were best at 512 x 1 and the K <= 4 ones at 2 tiles).
// The macros let a tuning build try other shapes without touching the sources.
#ifndef JABAS_BLOCK
#define JABAS_BLOCK 256
#endif
#ifndef JABAS_BLOCK_SGD
#define JABAS_BLOCK_SGD 128
#endif
#ifndef JABAS_BLOCK_MANYK
#define JABAS_BLOCK_MANYK 256
#endif
#ifndef JABAS_BLOCK_SIM_MANYK
#define JABAS_BLOCK_SIM_MANYK 256
#endif
#ifndef JABAS_CHUNK_TILES_LO
#define JABAS_CHUNK_TILES_LO 2
#endif
#ifndef JABAS_CHUNK_TILES_HI
#define JABAS_CHUNK_TILES_HI 4
#endif
#ifndef JABAS_CHUNK_TILES_MANYK
#define JABAS_CHUNK_TILES_MANYK 2
#endif
#ifndef JABAS_CHUNK_TILES_SIM_MANYK
#define JABAS_CHUNK_TILES_SIM_MANYK 2
#endif
#ifndef JABAS_CHUNK_TILES_SIM_LO
#define JABAS_CHUNK_TILES_SIM_LO JABAS_CHUNK_TILES_LO
#endif
#ifndef JABAS_CHUNK_TILES_PLAIN_LO
#define JABAS_CHUNK_TILES_PLAIN_LO 4
#endif
constexpr int kBlock = JABAS_BLOCK;         // default threads per workgroup (256 = 4 wave64)
constexpr int kWaves = kBlock / 64;
constexpr bool block_ok(int b) { return b % 64 == 0 && b >= 64 && b <= 1024; }
static_assert(block_ok(JABAS_BLOCK) && block_ok(JABAS_BLOCK_SGD) && block_ok(JABAS_BLOCK_MANYK) &&
              block_ok(JABAS_BLOCK_SIM_MANYK), "whole waves");
constexpr int kMinChunkTiles = JABAS_CHUNK_TILES_LO;
constexpr int kMaxChunkTiles = JABAS_CHUNK_TILES_HI;
// opt_class: 0 none, 1 SGD, 2 Adam/AdamW, 3 Adam/AdamW with amsgrad (launch shapes of class 2);
// stats: 0 none, 1 full rows, 2 similarity sums, 3 full rows + pair products (launch shapes and chunk
// tables of level 1). The shape depends
// on what a plan is encoded for (K, gradient dtype, optimizer class) and on the statistics level of the
// launch; a plan holds one chunk table per shape, so it serves every step.
__host__ __device__ constexpr int launch_block(int K, int grad_dtype, int opt_class, int stats) {
    if (stats == 2 && K > 4) return JABAS_BLOCK_SIM_MANYK;
    if (stats || opt_class == 0) return kBlock;
    if (K > 4) return JABAS_BLOCK_MANYK;
    return (opt_class == 1 && grad_dtype == JABAS_F32) ? JABAS_BLOCK_SGD : kBlock;
}
__host__ __device__ constexpr int launch_chunk_tiles(int K, int /*grad_dtype*/, int opt_class, int stats) {
    if (stats == 2) return K > 4 ? JABAS_CHUNK_TILES_SIM_MANYK : JABAS_CHUNK_TILES_SIM_LO;
    if (K > 4) return (stats || opt_class == 0) ? kMaxChunkTiles : JABAS_CHUNK_TILES_MANYK;
    if (!stats && opt_class >= 2) return JABAS_CHUNK_TILES_PLAIN_LO;
    return kMinChunkTiles;
}
// Statistics level whose launch shape (and chunk table of a plan) a level uses.
__host__ __device__ constexpr int shape_level(int stats) { return stats == JABAS_STATS_GRAM ? JABAS_STATS_FULL : stats; }
// Width of the partial rows of a launch: 4 similarity sums, + K norms, + K(K-1)/2 pair products.
__host__ __device__ constexpr int stats_row_width(int K, int stats) {
    return stats == JABAS_STATS_FULL ? 4 + K : (stats == JABAS_STATS_GRAM ? 4 + K + K * (K - 1) / 2 : (stats ? 4 : 1));
}
constexpr int imin(int a, int b) { return a < b ? a : b; }
// Fewest elements a chunk of a launch with statistics covers (one partial row per chunk): sizes workspaces.
constexpr int kMinStatsChunkElems = 4 * imin(imin(JABAS_BLOCK * JABAS_CHUNK_TILES_LO, JABAS_BLOCK * JABAS_CHUNK_TILES_SIM_LO),
                                             JABAS_BLOCK_SIM_MANYK * JABAS_CHUNK_TILES_SIM_MANYK);
// Fewest elements any chunk covers, over all shapes: sizes blobs that must fit every launch.
constexpr int kMinChunkElems = imin(imin(kMinStatsChunkElems, 4 * JABAS_BLOCK_SGD * JABAS_CHUNK_TILES_LO),
                                    4 * imin(imin(JABAS_BLOCK * JABAS_CHUNK_TILES_PLAIN_LO, JABAS_BLOCK * JABAS_CHUNK_TILES_LO),
                                             imin(JABAS_BLOCK_MANYK * JABAS_CHUNK_TILES_MANYK, JABAS_BLOCK * JABAS_CHUNK_TILES_HI)));
constexpr int kStatsStride = JABAS_STATS_STRIDE;
static_assert(stats_row_width(JABAS_STATS_GRAM_MAX_K, JABAS_STATS_GRAM) <= JABAS_STATS_STRIDE &&
              stats_row_width(JABAS_MAX_K, JABAS_STATS_FULL) <= JABAS_STATS_STRIDE, "every row fits the stride");

// Elements one thread handles per tile: one 16-byte fp32 vector of every fp32 buffer
// (bf16 gradients are then read as 8-byte vectors, which keeps every access of a wave
// contiguous).
__host__ __device__ constexpr int ept_of(int /*grad_dtype*/) { return 4; }
__host__ __device__ constexpr int tile_elems_of(int block) { return block * 4; }

// A span as the kernels see it. Pointers are rebased downwards by `lo` elements so that
// element index 0 of every buffer is 16-byte aligned (256-byte aligned when the buffers allow
// it, lo < 64 then, else lo < 4); [lo, hi) is the live range. Nothing below `lo` is accessed.
struct SpanDev {
    const void* g[JABAS_MAX_K];
    float* out;
    float* p;
    float* s1;
    float* s2;
    float* s3;
    float* fan[JABAS_MAX_K - 1];
    uint64_t lo, hi;
    // Where the Adam moments of grid element e live: float index mom(e) = t + mom_mult * (t & mom_mask),
    // t = e + mom_add, from s1 / s2 / s3. Arrays of their own: all three zero, mom(e) = e. Interleaved in
    // blocks of T elements: s1 = start of the span's first block group, s2 = s1 + T, s3 = s1 + 2 T,
    // mom_add = position of the first live element in its block minus lo (wraps; t >= 0 for every live e),
    // mom_mask = ~(T - 1), mom_mult = arrays interleaved - 1.
    uint64_t mom_add, mom_mask;
    uint32_t mom_mult;
    uint32_t narrow_ok;                      // 32-bit byte offsets reach every access of the span
    uint32_t n_fan;
    uint32_t bound_begin;
    uint32_t bound_count;
    uint32_t pad;
};
// Largest element index a 32-bit byte offset reaches in an fp32 buffer.
constexpr uint64_t kNarrowElems = 1ull << 30;

struct BoundDev {                            // same layout as JabasBound
    uint64_t start;                          // in un-rebased span coordinates
    uint32_t group;
    uint32_t pad;
};

// fp32 constants of one parameter group, derived on the host in double and rounded once,
// the way a Python float becomes an fp32 kernel scalar.
struct GroupDev {
    float wd;            // weight_decay
    float neg_lr;        // SGD: -lr
    float decay;         // AdamW: 1 - lr*wd
    float neg_step_size; // Adam: -(lr / (1 - beta1^t))
    float sqrt_bc2;      // Adam: sqrt(1 - beta2^t)
    float pad[3];
};

struct OptDev {
    float momentum, one_minus_damp;
    float beta1, one_minus_beta1, beta2, one_minus_beta2, eps;
    int32_t has_momentum, first_step, nesterov, adamw;
};

// One workgroup's share of a planned launch: chunk_tiles consecutive tiles of one span.
struct ChunkDesc {
    uint32_t span;                           // index into the span table
    uint32_t tile0;                          // first tile, local to the span
    uint32_t bound0;                         // bound entry (local to the span) covering the chunk's first live element
    uint32_t pad;
};

struct KArgs {
    const SpanDev* spans;                    // device table (planned launch)
    const ChunkDesc* chunks;                 // one per workgroup (planned launch)
    const uint32_t* chunk_prefix;            // n_span + 1 entries: first chunk of each span (planned launch)
    const BoundDev* bounds;                  // device, may be NULL
    double* partials;                        // one row of kStatsStride doubles per workgroup
    const float* grad_scale;                 // device scalar or NULL (clipping)
    uint32_t n_span;
    uint32_t n_chunks;
    uint32_t chunk_tiles;                    // tiles per workgroup (the kernel's own shape; checked on the host)
    uint32_t use_inline;                     // 1: the only span is `span0`, chunk b starts at tile b*chunk_tiles
    uint32_t half_mask;                      // bit k set: VSW k belongs to half B
    uint32_t pad0;
    SpanDev span0;
    float w[JABAS_MAX_K];
    float wh[JABAS_MAX_K];
    OptDev opt;
    GroupDev groups[JABAS_MAX_GROUPS];
    const struct StepScal* dyn;              // device block holding this step's scalars, or NULL (they are the fields above)
};

// The scalars of a step that change from one step to the next (weights, optimizer constants, per-group
// constants), as a block in device memory: a launch that names such a block reads them from there instead
// of from its own arguments, so a launch recorded in a HIP graph can be replayed with the learning rate,
// the Adam step or the weights of the moment. Same layout on host and device; written by
// jabas_step_scalars_encode.
struct StepScal {
    float w[JABAS_MAX_K];
    float wh[JABAS_MAX_K];
    OptDev opt;
    uint32_t half_mask;
    GroupDev groups[JABAS_MAX_GROUPS];
};
static_assert(sizeof(StepScal) == JABAS_STEP_SCALARS_BYTES, "public size of the step-scalar block");

#if defined(__HIPCC__)
// Launch through hipLaunchKernel so that the status is the one of THIS launch: hipGetLastError() would
// also hand back (and clear) whatever an earlier, unrelated HIP call of the calling thread left behind.
template <typename... Params, typename... Given>
inline hipError_t launch_kernel(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                                Given&&... given) {
    static_assert(sizeof...(Params) == sizeof...(Given), "one argument per kernel parameter");
    std::tuple<Params...> values(static_cast<Params>(given)...);
    void* ptrs[sizeof...(Params) > 0 ? sizeof...(Params) : 1];
    std::apply([&](auto&... v) { size_t i = 0; ((ptrs[i++] = static_cast<void*>(&v)), ...); }, values);
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds_bytes, stream);
}

// Sum over the 64 lanes of a wave with DPP moves (no LDS traffic); the total lands in
// lane 63. Pairing order is fixed: lane^1, lane^2, mirror within 8, mirror within 16,
// row 0->1 and 2->3, rows 0..1 -> 2..3.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move(double v) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROW_MASK, 0xf, false);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROW_MASK, 0xf, false);
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double wave_sum_to_lane63(double v) {
    v += dpp_move<0xB1, 0xf>(v);    // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xf>(v);    // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xf>(v);   // row_half_mirror
    v += dpp_move<0x140, 0xf>(v);   // row_mirror
    v += dpp_move<0x142, 0xa>(v);   // row_bcast:15 into rows 1 and 3
    v += dpp_move<0x143, 0xc>(v);   // row_bcast:31 into rows 2 and 3
    return v;
}

#endif

// Per-K launchers, one translation unit each (fused_kernel.hip with -DJABAS_K=k).
// opt_class: 0 none, 1 SGD, 2 Adam/AdamW, 3 the same with amsgrad; dyn: the step's scalars come from a.dyn
// (classes 1 and 2 only).
// Returns hipError_t as int.
#define JABAS_DECLARE_K(k)                                                                   \
    int launch_fused_k##k(int grad_dtype, int opt_class, int stats, int dyn, const KArgs& a, \
                          unsigned grid, hipStream_t stream);
JABAS_DECLARE_K(1) JABAS_DECLARE_K(2) JABAS_DECLARE_K(3) JABAS_DECLARE_K(4)
JABAS_DECLARE_K(5) JABAS_DECLARE_K(6) JABAS_DECLARE_K(7) JABAS_DECLARE_K(8)
JABAS_DECLARE_K(9) JABAS_DECLARE_K(10) JABAS_DECLARE_K(11) JABAS_DECLARE_K(12)
JABAS_DECLARE_K(13) JABAS_DECLARE_K(14) JABAS_DECLARE_K(15) JABAS_DECLARE_K(16)
#undef JABAS_DECLARE_K

}  // namespace jabas
