// K x K Gram matrix of the K worker gradients of one span: gram[a][b] = sum_e g_a[e]*g_b[e].
// fp32 (or widened bf16) inputs, exact fp64 products, fp64 sums, fixed order: bit-identical run to run.
//   K <= 8   grid-stride over 4-element vectors, K(K+1)/2 fp64 accumulators per thread on the vector
//            ALU, wave64 shuffle tree -> LDS -> one packed partial row per workgroup;
//   K >= 9   the Gram matrix is a contraction over the elements, X X^T with X the K x N matrix of the
//            workers' gradients: v_mfma_f64_16x16x4 with the SAME register as A and B operand (lane l
//            holds X[l % 16][l / 16] of a 16 x 4 slice, which is both A[i][k] and B[k][j] = A[j][k]).
//            The 256 running sums of the 16 x 16 tile take 8 registers per lane instead of K(K+1)/2
//            register pairs per thread, which is what limited the vector-ALU form to K <= 8. For K <= 8
//            the 16 rows hold two (K <= 4: four ...) element groups of the K workers, and the diagonal
//            blocks of the tile are added up at the end.
// Then a single-workgroup finalize that sums the workgroup rows in a fixed order.
#include "jabas_internal.h"

#ifndef JABAS_GRAM_VALU_MAX_K
#define JABAS_GRAM_VALU_MAX_K 8
#endif

namespace jabas {
namespace {

constexpr int kGramValuMaxK = JABAS_GRAM_VALU_MAX_K;   // up to here the vector-ALU kernel, beyond it the matrix cores

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }

template <int DT> struct GramLoad;
template <> struct GramLoad<JABAS_F32> {
    static constexpr int EPT = 4;
    static __device__ __forceinline__ void vec(const void* base, uint64_t e, float (&x)[4]) {
        const f32x4 r = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + e));
        x[0] = r.x; x[1] = r.y; x[2] = r.z; x[3] = r.w;
    }
    static __device__ __forceinline__ float one(const void* base, uint64_t e) { return static_cast<const float*>(base)[e]; }
};
template <> struct GramLoad<JABAS_BF16> {
    static constexpr int EPT = 4;
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


// ---- K >= 9: fp64 matrix cores -------------------------------------------------------------------------
typedef double f64x4 __attribute__((ext_vector_type(4)));
#ifndef JABAS_GRAM_RUN
#define JABAS_GRAM_RUN 4
#endif
constexpr int kGramRunBlocks = JABAS_GRAM_RUN;   // element blocks a wave loads before it multiplies

// Rows of the 16 x 16 tile: row r = group * Kp + worker, Kp = K rounded up to a power of two, 16 / Kp
// element groups. A block is 16 * (16 / Kp) consecutive elements: lane (r, ks) reads the four elements at
// group * 16 + ks * 4 of its worker, so every worker's part of a block is one contiguous stretch of 64 to
// 256 bytes and a run of blocks a contiguous kilobyte or more. Four MFMAs per load: the j-th takes element
// j of every lane's vector (which element sits in which k slot does not matter as long as A and B agree,
// and they are the same register).
template <int DT>
__global__ void __launch_bounds__(kBlock) gram_mfma_kernel(const SpanDev sp, int K, int log_kp, double* partials) {
    using L = GramLoad<DT>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, ks = lane >> 4;
    const int kp = 1 << log_kp;
    const int worker = r & (kp - 1), group = r >> log_kp;
    const int groups = 16 >> log_kp;
    const uint64_t block_elems = 16ull * groups;
    const uint64_t n_blocks = (sp.hi + block_elems - 1) / block_elems;
    const bool row_live = worker < K;
    const void* base = sp.g[row_live ? worker : 0];
    const uint32_t lane_off = static_cast<uint32_t>(group) * 16u + static_cast<uint32_t>(ks) * 4u;
    f64x4 acc = {0.0, 0.0, 0.0, 0.0}, acc1 = {0.0, 0.0, 0.0, 0.0};     // two chains: a multiply need not wait for the one before
    const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * kWaves;
    const uint64_t n_runs = (n_blocks + kGramRunBlocks - 1) / kGramRunBlocks;
    for (uint64_t run = static_cast<uint64_t>(blockIdx.x) * kWaves + wave; run < n_runs; run += n_waves) {
        float x[kGramRunBlocks][4];
#pragma unroll
        for (int u = 0; u < kGramRunBlocks; ++u) {
            const uint64_t e = (run * kGramRunBlocks + u) * block_elems + lane_off;
            if (row_live && e >= sp.lo && e + 4 <= sp.hi) {
                L::vec(base, e, x[u]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    x[u][i] = (row_live && e + i >= sp.lo && e + i < sp.hi) ? L::one(base, e + i) : 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < kGramRunBlocks; ++u)
#pragma unroll
            for (int i = 0; i < 4; i += 2) {
                const double d0 = static_cast<double>(x[u][i]), d1 = static_cast<double>(x[u][i + 1]);
                acc = __builtin_amdgcn_mfma_f64_16x16x4f64(d0, d0, acc, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f64_16x16x4f64(d1, d1, acc1, 0, 0, 0);
            }
    }
    acc += acc1;
    // the four waves' tiles, added in wave order: entry t = v * 64 + lane of the tile is register v of lane
    __shared__ double red[kWaves][256];
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][v * 64 + lane] = acc[v];
    __syncthreads();
    const int t = threadIdx.x;
    double s = red[0][t];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) s += red[w][t];
    partials[static_cast<uint64_t>(blockIdx.x) * JABAS_GRAM_STRIDE + t] = s;
}

// Sums the workgroup tiles (1024 threads: thread (entry, part) adds rows part, part + 4, ... in order, the
// four parts in order), then folds the diagonal blocks: gram[a][b] = sum over groups of
// tile[group * Kp + a][group * Kp + b]. Register v of lane l holds tile[4 * v + l / 16][l % 16].
constexpr int kGramMfmaFinalizeBlock = 1024;
__global__ void __launch_bounds__(kGramMfmaFinalizeBlock) gram_mfma_finalize_kernel(int K, int log_kp, const double* partials,
                                                                                    unsigned grid, double* gram_out) {
    __shared__ double part_sum[4][256];
    __shared__ double tile[256];
    const int t = threadIdx.x, e = t & 255, part = t >> 8;
    double s = 0.0;
#pragma unroll 8
    for (unsigned b = part; b < grid; b += 4) s += partials[static_cast<uint64_t>(b) * JABAS_GRAM_STRIDE + e];
    part_sum[part][e] = s;
    __syncthreads();
    if (t < 256) tile[t] = ((part_sum[0][t] + part_sum[1][t]) + part_sum[2][t]) + part_sum[3][t];
    __syncthreads();
    if (t < JABAS_GRAM_STRIDE) {
        const int a = t / JABAS_GRAM_MAX_K, b = t % JABAS_GRAM_MAX_K;
        double out = 0.0;
        if (a < K && b < K) {
            const int lo = a < b ? a : b, hi = a < b ? b : a;      // one triangle, mirrored: symmetric bit for bit
            const int kp = 1 << log_kp;
            for (int g = 0; g < (16 >> log_kp); ++g) {
                const int i = g * kp + lo, j = g * kp + hi;
                out += tile[(i >> 2) * 64 + (i & 3) * 16 + j];
            }
        }
        gram_out[t] = out;
    }
}

template <int K>
int launch_gram_k(int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    if (grad_dtype == JABAS_BF16)
        return static_cast<int>(launch_kernel(gram_kernel<K, JABAS_BF16>, dim3(grid), dim3(kBlock), 0, stream, sp, partials));
    return static_cast<int>(launch_kernel(gram_kernel<K, JABAS_F32>, dim3(grid), dim3(kBlock), 0, stream, sp, partials));
}

}  // namespace

int launch_gram(int K, int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    if (K > kGramValuMaxK) {
        int log_kp = 0;
        while ((1 << log_kp) < K) ++log_kp;
        if (grad_dtype == JABAS_BF16)
            return static_cast<int>(launch_kernel(gram_mfma_kernel<JABAS_BF16>, dim3(grid), dim3(kBlock), 0, stream, sp, K, log_kp, partials));
        return static_cast<int>(launch_kernel(gram_mfma_kernel<JABAS_F32>, dim3(grid), dim3(kBlock), 0, stream, sp, K, log_kp, partials));
    }
    switch (K) {
        case 1: return launch_gram_k<1>(grad_dtype, sp, partials, grid, stream);
        case 2: return launch_gram_k<2>(grad_dtype, sp, partials, grid, stream);
        case 3: return launch_gram_k<3>(grad_dtype, sp, partials, grid, stream);
        case 4: return launch_gram_k<4>(grad_dtype, sp, partials, grid, stream);
#if JABAS_GRAM_VALU_MAX_K > 4
        case 5: return launch_gram_k<5>(grad_dtype, sp, partials, grid, stream);
        case 6: return launch_gram_k<6>(grad_dtype, sp, partials, grid, stream);
        case 7: return launch_gram_k<7>(grad_dtype, sp, partials, grid, stream);
        case 8: return launch_gram_k<8>(grad_dtype, sp, partials, grid, stream);
#endif
        default: return -1;
    }
}

int launch_gram_finalize(int K, const double* partials, unsigned grid, double* gram_out, hipStream_t stream) {
    if (K > kGramValuMaxK) {
        int log_kp = 0;
        while ((1 << log_kp) < K) ++log_kp;
        return static_cast<int>(launch_kernel(gram_mfma_finalize_kernel, dim3(1), dim3(kGramMfmaFinalizeBlock), 0, stream, K, log_kp,
                                              partials, grid, gram_out));
    }
    return static_cast<int>(launch_kernel(gram_finalize_kernel, dim3(1), dim3(kGramFinalizeBlock), 0, stream, K, partials, grid, gram_out));
}

}  // namespace jabas
