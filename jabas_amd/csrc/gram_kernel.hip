// K x K Gram matrix of the K worker gradients of one span: gram[a][b] = sum_e g_a[e]*g_b[e].
// fp32 (or widened bf16) inputs, exact fp64 products, fp64 sums. Grid-stride over 4-element
// vectors, K(K+1)/2 accumulators per thread, wave64 shuffle tree -> LDS -> one packed
// partial row per workgroup, then a single-workgroup finalize that sums the rows in a fixed
// order and mirrors the lower triangle.
#include "jabas_internal.h"

namespace jabas {
namespace {

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

template <int K>
int launch_gram_k(int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
    if (grad_dtype == JABAS_BF16)
        return static_cast<int>(launch_kernel(gram_kernel<K, JABAS_BF16>, dim3(grid), dim3(kBlock), 0, stream, sp, partials));
    return static_cast<int>(launch_kernel(gram_kernel<K, JABAS_F32>, dim3(grid), dim3(kBlock), 0, stream, sp, partials));
}

}  // namespace

int launch_gram(int K, int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream) {
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

int launch_gram_finalize(int K, const double* partials, unsigned grid, double* gram_out, hipStream_t stream) {
    return static_cast<int>(launch_kernel(gram_finalize_kernel, dim3(1), dim3(kGramFinalizeBlock), 0, stream, K, partials, grid, gram_out));
}

}  // namespace jabas
