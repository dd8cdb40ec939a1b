// stream_mix_probe: what this machine's HBM delivers for the stream mixes of the fused sync kernel
// when the arithmetic is trivial. It answers "how far is fused_kernel from what the memory system
// gives a kernel of the same shape": same launch shape (one 256-thread workgroup per chunk of 2 or
// 4 tiles, dispatched in order), same access widths (16-byte, 8-byte for bf16 gradients), same
// nontemporal hints, K gradient read streams, S read-modify-write state streams, one write stream.
// Also: pure read, pure write, copy. Not part of libjabas_sync.so; a measurement aid.
//
//   ./stream_mix_probe [stagger_bytes]   prints one line per mix: ms, GB/s, fraction of 8 TB/s
//   ./stream_mix_probe [stagger_bytes [lds_bytes]]
//   stagger_bytes (default 0, multiple of 16): stream i starts i * stagger_bytes into its allocation,
//   to see what the relative placement of the streams in memory is worth
//   lds_bytes (default 0): unused dynamic LDS per workgroup, which caps the workgroups resident on a
//   CU (160 KB of LDS each), to see what occupancy is worth: 40960 -> 3 workgroups = 3 waves per SIMD
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));

#define CK(x)                                                                            \
    do {                                                                                 \
        hipError_t e_ = (x);                                                             \
        if (e_ != hipSuccess) {                                                          \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);   \
            std::exit(1);                                                                \
        }                                                                                \
    } while (0)

constexpr int kMaxK = 8, kMaxState = 3;
constexpr double kPeakGBs = 8000.0;

struct Streams {
    const void* grad[kMaxK];    // read-only
    float* state[kMaxState];    // read-modify-write
    float* out;                 // write-only
};

__device__ __forceinline__ float widen(unsigned hi16) { return __builtin_bit_cast(float, hi16); }

// One workgroup = TILES tiles of 1024 elements, processed U tiles at a time (all loads first).
template <int K, bool BF16, int S, bool OUT, int TILES, int U>
__global__ void __launch_bounds__(256) mix_kernel(Streams P) {
    const size_t tile0 = static_cast<size_t>(blockIdx.x) * TILES;
#pragma unroll
    for (int r = 0; r < TILES; r += U) {
        f4 g[U][K > 0 ? K : 1], st[U][S > 0 ? S : 1];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t e = ((tile0 + r + u) * 256 + threadIdx.x) * 4;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if (BF16) {
                    const u2 x = __builtin_nontemporal_load(reinterpret_cast<const u2*>(static_cast<const unsigned short*>(P.grad[k]) + e));
                    g[u][k] = f4{widen(x.x << 16), widen(x.x & 0xffff0000u), widen(x.y << 16), widen(x.y & 0xffff0000u)};
                } else {
                    g[u][k] = __builtin_nontemporal_load(reinterpret_cast<const f4*>(static_cast<const float*>(P.grad[k]) + e));
                }
            }
#pragma unroll
            for (int s = 0; s < S; ++s) st[u][s] = __builtin_nontemporal_load(reinterpret_cast<const f4*>(P.state[s] + e));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t e = ((tile0 + r + u) * 256 + threadIdx.x) * 4;
            f4 a = {1.f, 2.f, 3.f, 4.f};
#pragma unroll
            for (int k = 0; k < K; ++k) a = a + g[u][k] * 0.25f;
#pragma unroll
            for (int s = 0; s < S; ++s) __builtin_nontemporal_store(st[u][s] * 0.9f + a, reinterpret_cast<f4*>(P.state[s] + e));
            if (OUT) __builtin_nontemporal_store(a, reinterpret_cast<f4*>(P.out + e));
            if (!OUT && S == 0 && a.x == 123.456f) P.out[0] = a.y;      // keeps the loads of a pure-read run alive
        }
    }
}

template <typename F>
static float time_ms(F launch, int iters = 20) {
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    for (int i = 0; i < 3; ++i) launch();
    CK(hipEventRecord(a));
    for (int i = 0; i < iters; ++i) launch();
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    CK(hipGetLastError());
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, a, b));
    CK(hipEventDestroy(a));
    CK(hipEventDestroy(b));
    return ms / iters;
}

static unsigned g_lds_bytes = 0;

template <int K, bool BF16, int S, bool OUT, int TILES, int U>
static void run(const char* label, const Streams& P, size_t n) {
    const unsigned grid = static_cast<unsigned>(n / (1024u * TILES));      // n is a multiple of 4096
    const float ms = time_ms([&] { hipLaunchKernelGGL((mix_kernel<K, BF16, S, OUT, TILES, U>), dim3(grid), dim3(256), g_lds_bytes, 0, P); });
    const double bytes = static_cast<double>(n) * (K * (BF16 ? 2 : 4) + 8 * S + (OUT ? 4 : 0));
    const double gbs = bytes / ms / 1e6;
    std::printf("%-58s %8.3f ms %7.0f GB/s  %5.1f %% of 8 TB/s\n", label, ms, gbs, 100.0 * gbs / kPeakGBs);
    std::fflush(stdout);
}

int main(int argc, char** argv) {
    const size_t stagger = argc > 1 ? std::strtoull(argv[1], nullptr, 10) / 16 * 16 : 0;
    g_lds_bytes = argc > 2 ? static_cast<unsigned>(std::strtoul(argv[2], nullptr, 10)) : 0;
    const size_t n = static_cast<size_t>(1) << 27;      // elements per stream: 512 MiB fp32, 256 MiB bf16
    Streams P{};
    for (int k = 0; k < kMaxK; ++k) {
        char* p = nullptr;
        CK(hipMalloc(reinterpret_cast<void**>(&p), n * 4 + 16 * stagger));
        CK(hipMemset(p, 0, n * 4 + 16 * stagger));
        P.grad[k] = p + k * stagger;
    }
    for (int s = 0; s < kMaxState; ++s) {
        char* p = nullptr;
        CK(hipMalloc(reinterpret_cast<void**>(&p), n * 4 + 16 * stagger));
        CK(hipMemset(p, 0, n * 4 + 16 * stagger));
        P.state[s] = reinterpret_cast<float*>(p + (kMaxK + s) * stagger);
    }
    {
        char* p = nullptr;
        CK(hipMalloc(reinterpret_cast<void**>(&p), n * 4 + 16 * stagger));
        CK(hipMemset(p, 0, n * 4 + 16 * stagger));
        P.out = reinterpret_cast<float*>(p + (kMaxK + kMaxState) * stagger);
    }
    CK(hipDeviceSynchronize());

    std::printf("stream_mix_probe: %zu elements per stream, stagger %zu B, %u B of idle LDS per workgroup, one 256-thread workgroup per chunk, nontemporal accesses\n", n, stagger, g_lds_bytes);
    run<1, false, 0, false, 2, 2>("pure read, 1 stream", P, n);
    run<4, false, 0, false, 2, 2>("pure read, 4 streams", P, n);
    run<8, false, 0, false, 2, 2>("pure read, 8 streams", P, n);
    run<0, false, 0, true, 2, 2>("pure write, 1 stream", P, n);
    run<1, false, 0, true, 2, 2>("copy (1 read, 1 write)", P, n);
    run<0, false, 1, false, 2, 2>("in-place update (1 read-modify-write)", P, n);
    run<4, false, 0, true, 2, 2>("aggregate only, K=4 fp32 (20 B/elem)", P, n);
    run<2, false, 2, true, 2, 2>("resnet50 mix: K=2 fp32 + SGD (28 B/elem)", P, n);
    run<3, false, 2, true, 2, 2>("faster_rcnn mix: K=3 fp32 + SGD (32 B/elem)", P, n);
    run<4, false, 3, true, 2, 2>("vit_b16 / gnmt mix: K=4 fp32 + Adam (44 B/elem)", P, n);
    run<8, true, 3, true, 4, 2>("vit_l16 mix: K=8 bf16 + Adam (44 B/elem), 4-tile chunks", P, n);
    run<8, true, 3, true, 2, 2>("vit_l16 mix: K=8 bf16 + Adam (44 B/elem), 2-tile chunks", P, n);
    {
        const float ms = time_ms([&] { CK(hipMemcpyAsync(P.out, P.grad[0], n * 4, hipMemcpyDeviceToDevice, 0)); });
        const double gbs = static_cast<double>(n) * 8 / ms / 1e6;
        std::printf("%-58s %8.3f ms %7.0f GB/s  %5.1f %% of 8 TB/s\n", "hipMemcpyAsync device to device (read + write)", ms, gbs, 100.0 * gbs / kPeakGBs);
    }
    return 0;
}
