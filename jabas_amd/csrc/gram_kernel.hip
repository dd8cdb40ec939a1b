// K x K Gram matrix of the K worker gradients of one span: gram[a][b] = sum_e g_a[e]*g_b[e].
// Fixed order of operations: bit-identical run to run.
//   few workers    grid-stride over 4-element vectors, exact fp64 products of the fp32 (or widened bf16) values,
//                  K(K+1)/2 fp64 accumulators per thread on the vector ALU, wave64 shuffle tree -> LDS -> one
//                  packed partial row per workgroup (K <= 5 for fp32 gradients, K <= 7 for bf16);
//   more, to 16    fp32 gradients: fp64 matrix cores, v_mfma_f64_4x4x4 over 4 x 4 blocks of worker pairs, fed
//                  from registers (gram_mfma_kernel below), still exact products and fp64 sums;
//                  bf16 gradients: bf16 matrix cores, exact fp32 products, fp32 running sums over short runs,
//                  then fp64 (gram_bf16_mfma_kernel).
// Then a single-workgroup finalize that sums the workgroup rows in a fixed order.
#include "jabas_internal.h"

#ifndef JABAS_GRAM_VALU_MAX_K
#define JABAS_GRAM_VALU_MAX_K 5
#endif

namespace jabas {
namespace {

#ifndef JABAS_GRAM_VALU_MAX_K_BF16
#define JABAS_GRAM_VALU_MAX_K_BF16 7
#endif
// Up to here the vector-ALU kernel, beyond it the matrix cores. Measured on 86.6 M elements: fp32 K = 5: 5.95
// against 4.96 TB/s, K = 6: 5.54 against 5.94, K = 8: 5.45 against 6.01; bf16 gradients K = 6: 5.83 against 5.81,
// K = 8: 5.45 against 6.0.
constexpr int gram_valu_max_k(int grad_dtype) { return grad_dtype == JABAS_BF16 ? JABAS_GRAM_VALU_MAX_K_BF16 : JABAS_GRAM_VALU_MAX_K; }

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }

template <int DT> struct GramLoad;
template <> struct GramLoad<JABAS_F32> {
    static constexpr int EPT = 4;
    using Raw = f32x4;
    static __device__ __forceinline__ Raw raw(const void* base, uint64_t e) {
        return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + e));
    }
    static __device__ __forceinline__ float elem(const Raw& r, int i) { return r[i]; }
    static __device__ __forceinline__ Raw from(const float (&x)[4]) { return Raw{x[0], x[1], x[2], x[3]}; }
    static __device__ __forceinline__ void vec(const void* base, uint64_t e, float (&x)[4]) {
        const f32x4 r = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + e));
        x[0] = r.x; x[1] = r.y; x[2] = r.z; x[3] = r.w;
    }
    static __device__ __forceinline__ float one(const void* base, uint64_t e) { return static_cast<const float*>(base)[e]; }
};
template <> struct GramLoad<JABAS_BF16> {
    static constexpr int EPT = 4;
    using Raw = u32x2;
    static __device__ __forceinline__ Raw raw(const void* base, uint64_t e) {
        return __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(base) + e));
    }
    static __device__ __forceinline__ float elem(const Raw& r, int i) {
        const uint32_t w = i < 2 ? r.x : r.y;
        return bits_to_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    static __device__ __forceinline__ Raw from(const float (&x)[4]) {       // values that came from bf16: exact
        return Raw{(__builtin_bit_cast(uint32_t, x[0]) >> 16) | (__builtin_bit_cast(uint32_t, x[1]) & 0xffff0000u),
                   (__builtin_bit_cast(uint32_t, x[2]) >> 16) | (__builtin_bit_cast(uint32_t, x[3]) & 0xffff0000u)};
    }
    static __device__ __forceinline__ void vec(const void* base, uint64_t e, float (&x)[4]) {
        const u32x2 r = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(base) + e));
        x[0] = bits_to_float(r.x << 16); x[1] = bits_to_float(r.x & 0xffff0000u);
        x[2] = bits_to_float(r.y << 16); x[3] = bits_to_float(r.y & 0xffff0000u);
    }
    static __device__ __forceinline__ float one(const void* base, uint64_t e) {
        return bits_to_float(static_cast<uint32_t>(static_cast<const uint16_t*>(base)[e]) << 16);
    }
};

template <int K, int DT>
__global__ void __launch_bounds__(kBlock) gram_kernel(const SpanDev sp, double* partials) {
    using L = GramLoad<DT>;
    constexpr int EPT = L::EPT;
    constexpr int NP = K * (K + 1) / 2;
    double acc[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) acc[i] = 0.0;

    const uint64_t nvec = (sp.hi + EPT - 1) / EPT;
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t v = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; v < nvec; v += stride) {
        const uint64_t e = v * EPT;
        float g[K][EPT];
        if (e >= sp.lo && e + EPT <= sp.hi) {
#pragma unroll
            for (int k = 0; k < K; ++k) L::vec(sp.g[k], e, g[k]);
        } else {
#pragma unroll
            for (int i = 0; i < EPT; ++i) {
                const bool live = (e + i >= sp.lo) && (e + i < sp.hi);
#pragma unroll
                for (int k = 0; k < K; ++k) g[k][i] = live ? L::one(sp.g[k], e + i) : 0.0f;
            }
        }
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            double d[K];
#pragma unroll
            for (int k = 0; k < K; ++k) d[k] = static_cast<double>(g[k][i]);
            int idx = 0;
#pragma unroll
            for (int a = 0; a < K; ++a)
#pragma unroll
                for (int b = 0; b <= a; ++b, ++idx) acc[idx] = __builtin_fma(d[a], d[b], acc[idx]);
        }
    }

    __shared__ double red[kWaves][NP];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        double v = acc[i];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
        if (lane == 0) red[wave][i] = v;
    }
    __syncthreads();
    if (threadIdx.x < NP) {
        double s = red[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) s += red[w][threadIdx.x];
        partials[static_cast<uint64_t>(blockIdx.x) * JABAS_GRAM_STRIDE + threadIdx.x] = s;
    }
}

// Sums the workgroup rows and writes the symmetric matrix. 256 threads: thread (value, part) adds rows
// part, part + 16, ... of one packed entry in increasing order, the 16 parts of an entry sit in one
// 16-lane row and are combined by a fixed DPP pattern, so the result does not depend on timing. (One
// wave walking all rows of its entry one after the other took 0.23 ms for 1024 rows: more than the
// Gram kernel itself.)
constexpr int kGramFinalizeBlock = 256;
__global__ void __launch_bounds__(kGramFinalizeBlock) gram_finalize_kernel(int K, const double* partials, unsigned grid,
                                                                         double* gram_out) {
    const int np = K * (K + 1) / 2;
    const int t = threadIdx.x;
    if (t < JABAS_GRAM_STRIDE) gram_out[t] = 0.0;
    __syncthreads();
    const int part = t & 15;
    for (int v0 = 0; v0 < np; v0 += kGramFinalizeBlock / 16) {
        const int v = v0 + (t >> 4);
        double s = 0.0;
        if (v < np) {
#pragma unroll 8
            for (unsigned b = part; b < grid; b += 16) s += partials[static_cast<uint64_t>(b) * JABAS_GRAM_STRIDE + v];
        }
        s += dpp_move<0xB1, 0xf>(s);     // quad_perm [1,0,3,2]
        s += dpp_move<0x4E, 0xf>(s);     // quad_perm [2,3,0,1]
        s += dpp_move<0x141, 0xf>(s);    // row_half_mirror
        s += dpp_move<0x140, 0xf>(s);    // row_mirror
        if (v < np && part == 0) {
            int a = 0;
            while ((a + 1) * (a + 2) / 2 <= v) ++a;  // packed index v = a*(a+1)/2 + b, b <= a
            const int b = v - a * (a + 1) / 2;
            gram_out[a * JABAS_GRAM_MAX_K + b] = s;
            gram_out[b * JABAS_GRAM_MAX_K + a] = s;
        }
    }
}


// ---- K >= 5: fp64 matrix cores, 4 x 4 blocks ----------------------------------------------------------
// The Gram matrix is a contraction over the elements, X X^T with X the K x N matrix of the workers'
// gradients. The workers are cut into G = ceil(K / 4) groups of four; v_mfma_f64_4x4x4 (four independent
// 4 x 4 x 4 products per instruction) forms, for one pair of groups (ga <= gb), the 4 x 4 block of products
// over four elements in each of its four products. Lane l is
// worker l % 4 of every group and vector l / 4 of a 64-element block: it loads ONE 16-byte vector per group
// (a wave reads 256 contiguous bytes of each worker) and feeds round r of every pair from registers,
// A = element r of its vector of group ga, B = element r of its vector of group gb: no LDS, no shuffles,
// G(G+1)/2 running sums per lane instead of K(K+1)/2 register pairs per thread (which is what limits the
// vector-ALU form to K <= 8). Products of widened fp32 values are exact in fp64 and the order is fixed.
// Per 64 elements: 4 G(G+1)/2 MFMAs and 4 G conversions per wave, against 36 fp64 multiply-adds and 8
// conversions PER ELEMENT AND THREAD at K = 8 on the vector ALU.
#ifndef JABAS_GRAM_RUN_F32
#define JABAS_GRAM_RUN_F32 2
#endif
#ifndef JABAS_GRAM_RUN_BF16
#define JABAS_GRAM_RUN_BF16 4
#endif
// 64-element blocks a wave loads before it multiplies (bf16 vectors are half as long: twice as many in flight)
template <int DT> struct GramRun { static constexpr int value = DT == JABAS_BF16 ? JABAS_GRAM_RUN_BF16 : JABAS_GRAM_RUN_F32; };

template <int DT, int G>
__global__ void __launch_bounds__(kBlock) gram_mfma_kernel(const SpanDev sp, int K, double* partials) {
    using L = GramLoad<DT>;
    constexpr int P = G * (G + 1) / 2;
    constexpr int kGramRunBlocks = GramRun<DT>::value;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wi = lane & 3;                           // worker inside its group
    const uint32_t lane_off = static_cast<uint32_t>(lane >> 2) * 4u;
    const void* base[G];
    bool live[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        live[g] = g * 4 + wi < K;
        base[g] = sp.g[live[g] ? g * 4 + wi : 0];
    }
    double acc[P];
#pragma unroll
    for (int p = 0; p < P; ++p) acc[p] = 0.0;
    const uint64_t n_blocks = (sp.hi + 63) / 64;
    const uint64_t n_runs = (n_blocks + kGramRunBlocks - 1) / kGramRunBlocks;
    const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * kWaves;
    for (uint64_t run = static_cast<uint64_t>(blockIdx.x) * kWaves + wave; run < n_runs; run += n_waves) {
        typename L::Raw x[kGramRunBlocks][G];
#pragma unroll
        for (int u = 0; u < kGramRunBlocks; ++u) {
            const uint64_t e = (run * kGramRunBlocks + u) * 64 + lane_off;
            const bool whole = e >= sp.lo && e + 4 <= sp.hi;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (whole) {
                    // a lane beyond the last worker reads worker 0's vector (the same line another lane of the
                    // wave reads anyway) and drops it when it multiplies: the wave stays on one path and no
                    // load waits for another
                    x[u][g] = L::raw(base[g], e);
                } else {                             // a vector across the span's first or last element
                    float y[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        y[i] = (live[g] && e + i >= sp.lo && e + i < sp.hi) ? L::one(base[g], e + i) : 0.0f;
                    x[u][g] = L::from(y);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kGramRunBlocks; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                double d[G];
#pragma unroll
                for (int g = 0; g < G; ++g) d[g] = live[g] ? static_cast<double>(L::elem(x[u][g], r)) : 0.0;
                int p = 0;
#pragma unroll
                for (int ga = 0; ga < G; ++ga)
#pragma unroll
                    for (int gb = ga; gb < G; ++gb, ++p)
                        acc[p] = __builtin_amdgcn_mfma_f64_4x4x4f64(d[ga], d[gb], acc[p], 0, 0, 0);
            }
    }
    // The instruction's contraction index is lane / 16 and its four independent products are indexed by
    // (lane / 4) % 4; entry (i, j) of product b sits in lane j + 4 b + 16 i. Which of a lane's elements meets
    // which is therefore fixed by the lanes alone (A and B come from the same lane), and the four products
    // are partial sums over different elements of the same 4 x 4 block. Row of the workgroup: entry
    // [p][4 i + j] is the sum over the four products and the four waves (in that order) for pair p.
    __shared__ double red[kWaves][P][64];
#pragma unroll
    for (int p = 0; p < P; ++p) red[wave][p][lane] = acc[p];
    __syncthreads();
    for (int t = threadIdx.x; t < P * 16; t += kBlock) {
        const int p = t >> 4, i = (t >> 2) & 3, j = t & 3;
        const int l0 = j + 16 * i;
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) s += ((red[w][p][l0] + red[w][p][l0 + 4]) + red[w][p][l0 + 8]) + red[w][p][l0 + 12];
        partials[static_cast<uint64_t>(blockIdx.x) * JABAS_GRAM_STRIDE + t] = s;
    }
}

// Sums the workgroup rows (1024 threads: thread (entry, part) adds rows part, part + 4, ... in order, then
// the four parts in order) and unfolds the blocks: entry [p][4 i + j] of pair p = (ga, gb) is the product sum
// of workers 4 ga + i and 4 gb + j.
constexpr int kGramMfmaFinalizeBlock = 1024;
__global__ void __launch_bounds__(kGramMfmaFinalizeBlock) gram_mfma_finalize_kernel(int K, const double* partials, unsigned grid,
                                                                                    double* gram_out) {
    __shared__ double part_sum[4][256];
    __shared__ double tile[256];
    const int t = threadIdx.x, e = t & 255, part = t >> 8;
    const int G = (K + 3) / 4, P = G * (G + 1) / 2;
    double s = 0.0;
    if (e < P * 16) {
#pragma unroll 8
        for (unsigned b = part; b < grid; b += 4) s += partials[static_cast<uint64_t>(b) * JABAS_GRAM_STRIDE + e];
    }
    part_sum[part][e] = s;
    __syncthreads();
    if (t < 256) tile[t] = ((part_sum[0][t] + part_sum[1][t]) + part_sum[2][t]) + part_sum[3][t];
    __syncthreads();
    if (t < JABAS_GRAM_STRIDE) {
        const int a = t / JABAS_GRAM_MAX_K, b = t % JABAS_GRAM_MAX_K;
        double out = 0.0;
        if (a < K && b < K) {
            const int lo = a < b ? a : b, hi = a < b ? b : a;      // one triangle, mirrored: symmetric bit for bit
            const int ga = lo >> 2, gb = hi >> 2;
            const int p = ga * G - ga * (ga - 1) / 2 + (gb - ga);  // index of pair (ga, gb), ga <= gb
            out = tile[p * 16 + 4 * (lo & 3) + (hi & 3)];
        }
        gram_out[t] = out;
    }
}

// One workgroup on one compute unit pulls 1024 rows of up to 160 doubles (1.3 MB) in 12-29 us, a tenth of the
// bf16 K = 8 Gram launch itself. When the workspace has room for kGramFoldRows more rows, kGramFoldRows
// workgroups first fold rows j, j + kGramFoldRows, ... (in that order) into row j of that room and the finalize
// sums those. Which of the two forms runs depends on the sizes the caller passes only: same call, same bits.
constexpr unsigned kGramFoldRows = 32;
__global__ void __launch_bounds__(JABAS_GRAM_STRIDE) gram_mfma_fold_kernel(int K, const double* partials, unsigned grid, double* folded) {
    const int G = (K + 3) / 4, E = G * (G + 1) / 2 * 16;
    const int e = threadIdx.x;
    double s = 0.0;
    if (e < E) {
#pragma unroll 8
        for (unsigned b = blockIdx.x; b < grid; b += kGramFoldRows) s += partials[static_cast<uint64_t>(b) * JABAS_GRAM_STRIDE + e];
    }
    folded[static_cast<uint64_t>(blockIdx.x) * JABAS_GRAM_STRIDE + e] = s;
}

// ---- bf16 gradients: bf16 matrix cores ------------------------------------------------------------------
// v_mfma_f32_4x4x4_16b_bf16 multiplies, in each of its 16 independent products, a 4 x 4 operand by a 4 x 4
// operand whose contraction index runs over the four bf16 values ONE lane supplies in a register pair. With the lane
// layout above (lane l = worker l % 4 of its group, vector l / 4 of the block) the raw loaded registers ARE
// the operands: no widening, no conversion, one instruction per pair of groups and four elements of every
// lane. A lane loads 16 bytes (two operands) per group; a wave reads 256 contiguous bytes of each worker.
// Products of bf16 values are exact in fp32; the instruction adds four of them to an fp32 running sum, which
// is moved into fp64 sums (LDS, per wave) after at most kGramBf16FlushRuns runs, i.e. after at most
// 4 * 2 * RUN * kGramBf16FlushRuns elements: fp32 rounding stays near 1e-6 of |g_a| |g_b|, the order is fixed.
// Lanes beyond the last worker multiply worker 0's values into entries the finalize never reads.
template <int CTRL> __device__ __forceinline__ float gram_dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(8))) u32x4_a8;     // element 0 of a bf16 buffer is 8-byte aligned, not more

// 128-element blocks a wave loads before it multiplies, by number of groups
#ifndef JABAS_GRAM_RUN_BF16_G1
#define JABAS_GRAM_RUN_BF16_G1 2
#endif
#ifndef JABAS_GRAM_RUN_BF16_G2
#define JABAS_GRAM_RUN_BF16_G2 2
#endif
#ifndef JABAS_GRAM_RUN_BF16_G3
#define JABAS_GRAM_RUN_BF16_G3 2
#endif
#ifndef JABAS_GRAM_RUN_BF16_G4
#define JABAS_GRAM_RUN_BF16_G4 4
#endif
constexpr int gram_bf16_run(int G) {
    return G == 1 ? JABAS_GRAM_RUN_BF16_G1 : G == 2 ? JABAS_GRAM_RUN_BF16_G2 : G == 3 ? JABAS_GRAM_RUN_BF16_G3 : JABAS_GRAM_RUN_BF16_G4;
}
constexpr int kGramBf16FlushRuns = 128;

template <int G>
__global__ void __launch_bounds__(kBlock) gram_bf16_mfma_kernel(const SpanDev sp, int K, double* partials) {
    constexpr int P = G * (G + 1) / 2;
    constexpr int U = gram_bf16_run(G);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wi = lane & 3;
    const uint32_t lane_off = static_cast<uint32_t>(lane >> 2) * 8u;
    const uint16_t* base[G];
    bool live[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        live[g] = g * 4 + wi < K;
        base[g] = static_cast<const uint16_t*>(sp.g[live[g] ? g * 4 + wi : 0]);
    }
    // fp64 sums of the wave: [pair * 4 + i][16-lane row * 4 + j]
    __shared__ double sums[kWaves][P * 4][16];
    double* const wave_sums = &sums[0][0][0] + static_cast<size_t>(wave) * (P * 64);     // this wave's P * 64 sums, flat
    for (int i = lane; i < P * 64; i += 64) wave_sums[i] = 0.0;
    // the zeros are written by other lanes than the ones that add to them later: order the two within the wave
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x4 acc[P];
#pragma unroll
    for (int p = 0; p < P; ++p) acc[p] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // entry (i, j) of a product sits in register i of lane j + 4 * product: a rotation by 4 and by 8 inside the
    // 16-lane row adds the row's four products; lanes 0..3 of every row then own one fp64 sum each per register
    const bool owner = ((lane >> 2) & 3) == 0;
    const int col = (lane >> 4) * 4 + wi;
    auto flush = [&]() {
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = acc[p][i];
                v += gram_dpp_f32<0x124>(v);        // row_ror:4
                v += gram_dpp_f32<0x128>(v);        // row_ror:8
                if (owner) sums[wave][p * 4 + i][col] += static_cast<double>(v);
                acc[p][i] = 0.0f;
            }
    };
    const uint64_t n_blocks = (sp.hi + 127) / 128;
    const uint64_t n_runs = (n_blocks + U - 1) / U;
    const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * kWaves;
    int pending = 0;
    for (uint64_t run = static_cast<uint64_t>(blockIdx.x) * kWaves + wave; run < n_runs; run += n_waves) {
        u32x4 x[U][G];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t e = (run * U + u) * 128 + lane_off;
            const bool whole = e >= sp.lo && e + 8 <= sp.hi;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (whole) {
                    x[u][g] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_a8*>(base[g] + e));
                } else {                             // a vector across the span's first or last element
                    uint32_t h[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) h[i] = (e + i >= sp.lo && e + i < sp.hi) ? base[g][e + i] : 0u;
                    x[u][g] = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                s16x4 d[G];
#pragma unroll
                for (int g = 0; g < G; ++g)
                    d[g] = __builtin_bit_cast(s16x4, half ? u32x2{x[u][g].z, x[u][g].w} : u32x2{x[u][g].x, x[u][g].y});
                int p = 0;
#pragma unroll
                for (int ga = 0; ga < G; ++ga)
#pragma unroll
                    for (int gb = ga; gb < G; ++gb, ++p)
                        acc[p] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(d[ga], d[gb], acc[p], 0, 0, 0);
            }
        if (++pending == kGramBf16FlushRuns) { flush(); pending = 0; }
    }
    flush();
    __syncthreads();
    // row of the workgroup, the format of gram_mfma_kernel: entry [p][4 i + j], rows then waves in order
    for (int t = threadIdx.x; t < P * 16; t += kBlock) {
        const int p = t >> 4, i = (t >> 2) & 3, j = t & 3;
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
            s += ((sums[w][p * 4 + i][j] + sums[w][p * 4 + i][4 + j]) + sums[w][p * 4 + i][8 + j]) + sums[w][p * 4 + i][12 + j];
        partials[static_cast<uint64_t>(blockIdx.x) * JABAS_GRAM_STRIDE + t] = s;
    }
}

int launch_gram_bf16_mfma(int K, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    switch ((K + 3) / 4) {
        case 1: return static_cast<int>(launch_kernel(gram_bf16_mfma_kernel<1>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        case 2: return static_cast<int>(launch_kernel(gram_bf16_mfma_kernel<2>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        case 3: return static_cast<int>(launch_kernel(gram_bf16_mfma_kernel<3>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        case 4: return static_cast<int>(launch_kernel(gram_bf16_mfma_kernel<4>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        default: return -1;
    }
}

template <int K>
int launch_gram_k(int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    if (grad_dtype == JABAS_BF16)
        return static_cast<int>(launch_kernel(gram_kernel<K, JABAS_BF16>, dim3(grid), dim3(kBlock), 0, stream, sp, partials));
    return static_cast<int>(launch_kernel(gram_kernel<K, JABAS_F32>, dim3(grid), dim3(kBlock), 0, stream, sp, partials));
}

template <int DT>
int launch_gram_mfma(int K, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    switch ((K + 3) / 4) {
        case 1: return static_cast<int>(launch_kernel(gram_mfma_kernel<DT, 1>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        case 2: return static_cast<int>(launch_kernel(gram_mfma_kernel<DT, 2>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        case 3: return static_cast<int>(launch_kernel(gram_mfma_kernel<DT, 3>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        case 4: return static_cast<int>(launch_kernel(gram_mfma_kernel<DT, 4>, dim3(grid), dim3(kBlock), 0, stream, sp, K, partials));
        default: return -1;
    }
}

}  // namespace

int launch_gram(int K, int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    if (K > gram_valu_max_k(grad_dtype))
        return grad_dtype == JABAS_BF16 ? launch_gram_bf16_mfma(K, sp, partials, grid, stream)
                                        : launch_gram_mfma<JABAS_F32>(K, sp, partials, grid, stream);
    switch (K) {
        case 1: return launch_gram_k<1>(grad_dtype, sp, partials, grid, stream);
        case 2: return launch_gram_k<2>(grad_dtype, sp, partials, grid, stream);
        case 3: return launch_gram_k<3>(grad_dtype, sp, partials, grid, stream);
        case 4: return launch_gram_k<4>(grad_dtype, sp, partials, grid, stream);
        case 5: return launch_gram_k<5>(grad_dtype, sp, partials, grid, stream);
        case 6: return launch_gram_k<6>(grad_dtype, sp, partials, grid, stream);
        case 7: return launch_gram_k<7>(grad_dtype, sp, partials, grid, stream);
        case 8: return launch_gram_k<8>(grad_dtype, sp, partials, grid, stream);
        default: return -1;
    }
}

unsigned gram_fold_rows() { return kGramFoldRows; }

// spare_rows: rows of JABAS_GRAM_STRIDE doubles the workspace holds beyond the `grid` partial rows
int launch_gram_finalize(int K, int grad_dtype, double* partials, unsigned grid, unsigned spare_rows, double* gram_out,
                         hipStream_t stream) {
    if (K > gram_valu_max_k(grad_dtype)) {
        if (grid > 4 * kGramFoldRows && spare_rows >= kGramFoldRows) {
            double* folded = partials + static_cast<uint64_t>(grid) * JABAS_GRAM_STRIDE;
            if (launch_kernel(gram_mfma_fold_kernel, dim3(kGramFoldRows), dim3(JABAS_GRAM_STRIDE), 0, stream, K,
                              static_cast<const double*>(partials), grid, folded) != 0)
                return -1;
            return static_cast<int>(launch_kernel(gram_mfma_finalize_kernel, dim3(1), dim3(kGramMfmaFinalizeBlock), 0, stream, K,
                                                  static_cast<const double*>(folded), kGramFoldRows, gram_out));
        }
        return static_cast<int>(launch_kernel(gram_mfma_finalize_kernel, dim3(1), dim3(kGramMfmaFinalizeBlock), 0, stream, K,
                                              static_cast<const double*>(partials), grid, gram_out));
    }
    return static_cast<int>(launch_kernel(gram_finalize_kernel, dim3(1), dim3(kGramFinalizeBlock), 0, stream, K,
                                          static_cast<const double*>(partials), grid, gram_out));
}

}  // namespace jabas
