// Fused VSW-aggregate + gradient statistics + optimizer kernel for gfx950 (MI355X).
// Compiled once per JABAS_K (number of virtual stream workers) so that the K gradient
// streams are fully unrolled into independent 128-bit loads.
//
// Execution shape
//   - one workgroup per chunk of consecutive tiles of one span; a tile is one 16-byte vector of
//     every fp32 buffer (one 8-byte vector of a bf16 gradient buffer) per thread. Threads per
//     workgroup and tiles per chunk depend on the kernel family (launch_block / launch_chunk_tiles):
//     256 threads x 2 or 4 tiles with statistics, 128 x 2, 256 x 2 or 256 x 4 without. Small,
//     short-lived workgroups dispatched in order keep the part of every buffer that is being
//     streamed at any moment compact, which on MI355X sustains a markedly higher HBM rate than a
//     persistent grid that spreads over the whole buffers;
//   - every global access is a vector access with the nontemporal hint (each byte is touched
//     exactly once per step);
//   - tiles that lie wholly inside the live range of a span and inside one parameter
//     group take the vector path (all loads of U tiles issued before any arithmetic);
//     the few tiles that straddle a span end or a group change take a scalar path;
//   - statistics: per-thread fp64 accumulators -> LDS -> 16-way sums in fixed order -> DPP row
//     reduction -> one partial row of 4 + K doubles per workgroup in the workspace, summed in
//     fixed order by the finalize kernel. The order is fixed, so results are bit-identical run to run.
//
// Arithmetic is compiled with -ffp-contract=off: every fp32 product and sum of the
// aggregate and of the optimizer formulas is rounded on its own, so results can be
// compared bit for bit with a CPU restatement that applies the same operations in the
// same order. The formulas follow torch 1.8.1 optim/_functional.py (sgd, adam, adamw),
// the version the reference pins (README.md:59-64 of the JABAS repository).
#include "jabas_internal.h"

#ifndef JABAS_K
#error "compile with -DJABAS_K=<1..16>"
#endif
// Most tiles whose loads are in flight together: a whole 4-tile chunk without statistics,
// 2 tiles with (the fp64 accumulators need the registers).
#ifndef JABAS_UNROLL_PLAIN
#define JABAS_UNROLL_PLAIN 4
#endif
#ifndef JABAS_UNROLL_STATS
#define JABAS_UNROLL_STATS 2
#endif

namespace jabas {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }

// Address of element e of a buffer whose base is uniform over the workgroup. NARROW: the byte offset
// fits 32 bits (spans of up to kNarrowElems elements), so the address is "scalar base + zero-extended
// 32-bit lane offset": the form a global access takes with the base in scalar registers and ONE vector
// register of offset shared by every stream of the same element size, instead of a 64-bit vector
// address (two registers and two additions) per stream and tile.
template <bool NARROW, int ES> __device__ __forceinline__ const char* elem_addr(const void* base, uint64_t e) {
    if constexpr (NARROW) {
        const uint32_t off = static_cast<uint32_t>(e) * static_cast<uint32_t>(ES);
        return static_cast<const char*>(base) + static_cast<uint64_t>(off);
    } else {
        return static_cast<const char*>(base) + e * ES;
    }
}

template <int DT> struct Grad;

template <> struct Grad<JABAS_F32> {
    static constexpr int EPT = 4;
    using Raw = f32x4;
    template <bool NARROW> static __device__ __forceinline__ Raw load(const void* base, uint64_t e) {
        return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(elem_addr<NARROW, 4>(base, e)));
    }
    static __device__ __forceinline__ void widen(const Raw& r, float (&x)[4]) {
        x[0] = r.x; x[1] = r.y; x[2] = r.z; x[3] = r.w;
    }
    static __device__ __forceinline__ float load1(const void* base, uint64_t e) {
        return static_cast<const float*>(base)[e];
    }
};

template <> struct Grad<JABAS_BF16> {
    static constexpr int EPT = 4;
    using Raw = u32x2;
    template <bool NARROW> static __device__ __forceinline__ Raw load(const void* base, uint64_t e) {
        return __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(elem_addr<NARROW, 2>(base, e)));
    }
    // bf16 -> fp32 is exact: the 16 bits become the high half of the fp32 pattern.
    static __device__ __forceinline__ void widen(const Raw& r, float (&x)[4]) {
        x[0] = bits_to_float(r.x << 16); x[1] = bits_to_float(r.x & 0xffff0000u);
        x[2] = bits_to_float(r.y << 16); x[3] = bits_to_float(r.y & 0xffff0000u);
    }
    static __device__ __forceinline__ float load1(const void* base, uint64_t e) {
        return bits_to_float(static_cast<uint32_t>(static_cast<const uint16_t*>(base)[e]) << 16);
    }
};

constexpr int OPT_NONE = 0, OPT_SGD = 1, OPT_ADAM = 2, OPT_AMS = 3;    // OPT_AMS: Adam / AdamW with amsgrad
__host__ __device__ constexpr bool is_adam(int opt) { return opt == OPT_ADAM || opt == OPT_AMS; }
// Kernels with statistics form the addresses of the vector path as scalar base + 32-bit lane offset (measured
// on the ViT-L/16 set, K = 8 bf16: +0.5 % with full rows, +2 % with similarity sums; K = 4 fp32 Adam: 8-9 fewer
// VGPRs, full rows 131 -> 123 and 4 waves per SIMD instead of 3, ViT-B/16 +1.2 % with similarity sums, +0.4 % with
// full rows, GNMT +-0.3 %); their spans that 32-bit byte offsets do not reach (over 4 GiB of fp32 per buffer)
// go through the careful path tile by tile: correct but slower. The plain kernels keep 64-bit vector addresses
// (no gain there: their registers are not what limits them).
__host__ __device__ constexpr bool narrow_addressing(int /*K*/, int SL) { return SL != 0; }

// Statistics level of a launch: 0 none, 1 the full row (4 + K sums), 2 the four sums of the halves and of
// the aggregate only (what the cosine similarity and global-norm clipping read), 3 the full row and the
// products of every pair of workers (the Gram matrix; up to JABAS_STATS_GRAM_MAX_K workers).
template <int K, int SL> struct NStats { static constexpr int value = stats_row_width(K, SL); };
constexpr bool per_vsw_norms(int SL) { return SL == JABAS_STATS_FULL || SL == JABAS_STATS_GRAM; }

// Per-thread running sums of the statistics. fp32 gradients: fp64 (a product of two fp32 values is exact
// in fp64). bf16 gradients: fp32 within the thread's chunk (at most 16 elements), widened to fp64 when the
// workgroup reduces: a product of two bf16 values is exact in fp32 and the few fp32 additions keep the
// sums within 1e-6 relative, four orders inside the 1e-2 bar of reduced-precision gradients, at a third
// of the arithmetic and half the registers (fp64 multiply-adds and conversions run at half rate).
template <int DT> struct StatAcc { using type = double; };
template <> struct StatAcc<JABAS_BF16> { using type = float; };
__device__ __forceinline__ double stat_fma(float a, float b, double acc) {
    return __builtin_fma(static_cast<double>(a), static_cast<double>(b), acc);
}
__device__ __forceinline__ float stat_fma(float a, float b, float acc) { return __builtin_fmaf(a, b, acc); }

// The step's scalars as the arithmetic below names them (a.w[k], a.wh[k], a.half_mask, a.opt, a.groups[i],
// plus a.bounds and a.grad_scale), backed by a StepScal block in device memory instead of the kernel
// arguments. The block is read through the constant address space: uniform loads that the compiler may
// place anywhere, the same instructions a kernel-argument read compiles to, and the block is not written
// while a launch that names it runs. Every function below takes either KArgs or this view.
struct DynView {
    typedef const __attribute__((address_space(4))) StepScal* Block;
    struct Weights {
        const __attribute__((address_space(4))) float* p;
        __device__ __forceinline__ float operator[](int k) const { return p[k]; }
    };
    struct Groups {
        Block b;
        __device__ __forceinline__ GroupDev operator[](uint32_t i) const {
            GroupDev g;
            g.wd = b->groups[i].wd; g.neg_lr = b->groups[i].neg_lr; g.decay = b->groups[i].decay;
            g.neg_step_size = b->groups[i].neg_step_size; g.sqrt_bc2 = b->groups[i].sqrt_bc2;
            return g;
        }
    };
    Weights w, wh;
    Groups groups;
    OptDev opt;
    uint32_t half_mask;
    const BoundDev* bounds;
    const float* grad_scale;
    __device__ __forceinline__ explicit DynView(const KArgs& a) {
        Block b = (Block)a.dyn;
        w.p = b->w; wh.p = b->wh; groups.b = b;
        opt.momentum = b->opt.momentum; opt.one_minus_damp = b->opt.one_minus_damp;
        opt.beta1 = b->opt.beta1; opt.one_minus_beta1 = b->opt.one_minus_beta1;
        opt.beta2 = b->opt.beta2; opt.one_minus_beta2 = b->opt.one_minus_beta2; opt.eps = b->opt.eps;
        opt.has_momentum = b->opt.has_momentum; opt.first_step = b->opt.first_step;
        opt.nesterov = b->opt.nesterov; opt.adamw = b->opt.adamw;
        half_mask = b->half_mask;
        bounds = a.bounds;
        grad_scale = a.grad_scale;
    }
};

// Float index of grid element e's Adam moments from the span's moment bases: e itself when the moments are
// arrays of their own, its place in the interleaved arena otherwise (SpanDev). Two integer operations.
// The bound table of a launch is, like the plan's other tables, not written while the launch runs: read through
// the constant address space (uniform loads the compiler is free to move or repeat).
typedef const __attribute__((address_space(4))) BoundDev* ConstBounds;
__device__ __forceinline__ ConstBounds const_bounds(const BoundDev* p) { return (ConstBounds)p; }

template <class SP> __device__ __forceinline__ uint64_t moment_index(const SP& sp, uint64_t e) {
    const uint64_t t = e + sp.mom_add;
    return t + sp.mom_mult * (t & sp.mom_mask);
}

// One element of the optimizer step. g is the aggregated gradient.
template <int OPT>
__device__ __forceinline__ void opt_elem(float g, float& p, float& s1, float& s2, float& s3,
                                         const GroupDev& G, const OptDev& O) {
    if constexpr (OPT == OPT_SGD) {
        float d = g;
        if (G.wd != 0.0f) d = d + G.wd * p;
        if (O.has_momentum) {
            if (O.first_step) s1 = d;
            else s1 = s1 * O.momentum + d * O.one_minus_damp;
            d = O.nesterov ? d + O.momentum * s1 : s1;
        }
        p = p + G.neg_lr * d;
    } else if constexpr (is_adam(OPT)) {
        if (O.adamw) p = p * G.decay;
        else if (G.wd != 0.0f) g = g + G.wd * p;
        s1 = s1 * O.beta1 + g * O.one_minus_beta1;
        s2 = s2 * O.beta2 + (O.one_minus_beta2 * g) * g;
        float second = s2;
        if constexpr (OPT == OPT_AMS) {       // torch.maximum(max_exp_avg_sq, exp_avg_sq): a NaN on either side stays
            s3 = (s3 != s3) ? s3 : ((s2 != s2) ? s2 : (s3 > s2 ? s3 : s2));
            second = s3;
        }
        const float denom = __builtin_sqrtf(second) / G.sqrt_bc2 + O.eps;
        p = p + (G.neg_step_size * s1) / denom;
    }
}

// Aggregate, statistics and optimizer for N consecutive elements held in registers.
template <int K, int N, int DT, int OPT, int SL, bool HD, class A>
__device__ __forceinline__ void compute(const float (&g)[K][N], float (&p)[N], float (&s1)[N],
                                        float (&s2)[N], float (&s3)[N], float (&agg)[N], const A& a,
                                        const GroupDev& G, float clip, typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float s = g[0][i] * a.w[0];
#pragma unroll
        for (int k = 1; k < K; ++k) s = s + g[k][i] * a.w[k];
        if (clip < 1.0f) s = s * clip;         // global-norm clipping: only ever scales down
        agg[i] = s;
        if constexpr (SL) {
            float ga = 0.0f, gb = 0.0f;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const float t = g[k][i] * a.wh[k];
                if constexpr (HD) {            // default halves: even worker -> A, odd -> B
                    if (k & 1) gb = gb + t; else ga = ga + t;
                } else {
                    const bool in_b = (a.half_mask >> k) & 1u;
                    gb = in_b ? gb + t : gb;
                    ga = in_b ? ga : ga + t;
                }
                if constexpr (per_vsw_norms(SL))
                    acc[JABAS_STAT_NORM_VSW0 + k] = stat_fma(g[k][i], g[k][i], acc[JABAS_STAT_NORM_VSW0 + k]);
                if constexpr (SL == JABAS_STATS_GRAM) {
#pragma unroll
                    for (int b = k + 1; b < K; ++b)
                        acc[JABAS_STAT_PAIR(K, k, b)] = stat_fma(g[k][i], g[b][i], acc[JABAS_STAT_PAIR(K, k, b)]);
                }
            }
            // fp64 sums: fp32 x fp32 products are exact in fp64, so fma == mul followed by add there.
            acc[JABAS_STAT_DOT_AB] = stat_fma(ga, gb, acc[JABAS_STAT_DOT_AB]);
            acc[JABAS_STAT_NORM_A] = stat_fma(ga, ga, acc[JABAS_STAT_NORM_A]);
            acc[JABAS_STAT_NORM_B] = stat_fma(gb, gb, acc[JABAS_STAT_NORM_B]);
            acc[JABAS_STAT_NORM_AGG] = stat_fma(s, s, acc[JABAS_STAT_NORM_AGG]);
        }
        if constexpr (OPT != OPT_NONE) opt_elem<OPT>(s, p[i], s1[i], s2[i], s3[i], G, a.opt);
        // keep the elements' dependency chains apart: interleaving them costs the statistics
        // kernels a third of their occupancy in registers and buys nothing in a memory-bound loop
        if constexpr (SL) __builtin_amdgcn_sched_barrier(0);
    }
}

template <int NV, bool NARROW> __device__ __forceinline__ void load_vec(f32x4 (&r)[NV], const float* base, uint64_t e) {
#pragma unroll
    for (int v = 0; v < NV; ++v)
        r[v] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(elem_addr<NARROW, 4>(base, e + 4 * v)));
}
template <int NV, bool NARROW> __device__ __forceinline__ void store_vec(const float (&x)[4 * NV], float* base, uint64_t e) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        f32x4 r = {x[4 * v], x[4 * v + 1], x[4 * v + 2], x[4 * v + 3]};
        __builtin_nontemporal_store(r, reinterpret_cast<f32x4*>(const_cast<char*>(elem_addr<NARROW, 4>(base, e + 4 * v))));
    }
}
template <int NV> __device__ __forceinline__ void unpack_vec(const f32x4 (&r)[NV], float (&x)[4 * NV]) {
#pragma unroll
    for (int v = 0; v < NV; ++v) { x[4 * v] = r[v].x; x[4 * v + 1] = r[v].y; x[4 * v + 2] = r[v].z; x[4 * v + 3] = r[v].w; }
}

// Registers of U consecutive full tiles: the raw 16-byte vectors as loaded.
template <int K, int DT, int U, int OPT = OPT_ADAM> struct TileRegs {
    typename Grad<DT>::Raw g[U][K];
    f32x4 p[U][Grad<DT>::EPT / 4], s1[U][Grad<DT>::EPT / 4], s2[U][Grad<DT>::EPT / 4];
    f32x4 s3[OPT == OPT_AMS ? U : 1][Grad<DT>::EPT / 4];
};

// Issues every load of U consecutive full tiles. e is the (rebased) index of this
// thread's first element in the first tile.
template <int K, int DT, int OPT, int U, int BS, bool NARROW, class SP>
__device__ __forceinline__ void issue_loads(TileRegs<K, DT, U, OPT>& r, const SP& sp, uint64_t e, bool load_s1) {
    using GR = Grad<DT>;
    constexpr int EPT = GR::EPT, NV = EPT / 4;
    constexpr uint64_t TE = static_cast<uint64_t>(BS) * EPT;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t eu = e + u * TE;
#pragma unroll
        for (int k = 0; k < K; ++k) r.g[u][k] = GR::template load<NARROW>(sp.g[k], eu);
        if constexpr (OPT != OPT_NONE) {
            load_vec<NV, NARROW>(r.p[u], sp.p, eu);
            const uint64_t mu = is_adam(OPT) ? moment_index(sp, eu) : eu;
            if (load_s1) load_vec<NV, NARROW>(r.s1[u], sp.s1, mu);
            if constexpr (is_adam(OPT)) load_vec<NV, NARROW>(r.s2[u], sp.s2, mu);
            if constexpr (OPT == OPT_AMS) load_vec<NV, NARROW>(r.s3[u], sp.s3, mu);
        }
    }
}

// Arithmetic and stores of U tiles whose loads were issued by issue_loads.
template <int K, int DT, int OPT, int SL, bool HD, int U, bool NARROW, class A, class SP>
__device__ __forceinline__ void consume(const TileRegs<K, DT, U, OPT>& r, const SP& sp, uint64_t e, const A& a,
                                        const GroupDev& G, float clip, bool use_s1, bool load_s1,
                                        typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
    using GR = Grad<DT>;
    constexpr int EPT = GR::EPT, NV = EPT / 4;
    constexpr uint64_t TE = static_cast<uint64_t>(launch_block(K, DT, OPT, SL)) * EPT;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t eu = e + u * TE;
        float g[K][EPT], p[EPT], s1[EPT], s2[EPT], s3[EPT], agg[EPT];
#pragma unroll
        for (int k = 0; k < K; ++k) GR::widen(r.g[u][k], g[k]);
        if constexpr (OPT != OPT_NONE) {
            unpack_vec<NV>(r.p[u], p);
            if (load_s1) unpack_vec<NV>(r.s1[u], s1);
            else {
#pragma unroll
                for (int i = 0; i < EPT; ++i) s1[i] = 0.0f;
            }
            if constexpr (is_adam(OPT)) unpack_vec<NV>(r.s2[u], s2);
            if constexpr (OPT == OPT_AMS) unpack_vec<NV>(r.s3[u], s3);
        }
        compute<K, EPT, DT, OPT, SL, HD>(g, p, s1, s2, s3, agg, a, G, clip, acc);
        if (sp.out) store_vec<NV, NARROW>(agg, sp.out, eu);
        if constexpr (OPT != OPT_NONE) {
            store_vec<NV, NARROW>(p, sp.p, eu);
            const uint64_t mu = is_adam(OPT) ? moment_index(sp, eu) : eu;
            if (use_s1) store_vec<NV, NARROW>(s1, sp.s1, mu);
            if constexpr (is_adam(OPT)) store_vec<NV, NARROW>(s2, sp.s2, mu);
            if constexpr (OPT == OPT_AMS) store_vec<NV, NARROW>(s3, sp.s3, mu);
            for (uint32_t f = 0; f < sp.n_fan; ++f) store_vec<NV, NARROW>(p, sp.fan[f], eu);
        }
    }
}

// Vector path over nfull consecutive full tiles of one parameter group: groups of U tiles,
// then U/2, ... down to single tiles.
template <int K, int DT, int OPT, int SL, bool HD, int U, class A, class SP>
__device__ __forceinline__ void fast_run(const SP& sp, uint64_t e, uint32_t nfull, const A& a,
                                         const GroupDev& G, float clip, typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
    constexpr int BS = launch_block(K, DT, OPT, SL);
    constexpr uint64_t TE = static_cast<uint64_t>(BS) * Grad<DT>::EPT;
    const bool use_s1 = is_adam(OPT) || (OPT == OPT_SGD && a.opt.has_momentum);
    const bool load_s1 = is_adam(OPT) || (OPT == OPT_SGD && a.opt.has_momentum && !a.opt.first_step);
    uint32_t i = 0;
    for (; i + U <= nfull; i += U, e += U * TE) {
        TileRegs<K, DT, U, OPT> r;
        issue_loads<K, DT, OPT, U, BS, narrow_addressing(K, SL)>(r, sp, e, load_s1);
        consume<K, DT, OPT, SL, HD, U, narrow_addressing(K, SL)>(r, sp, e, a, G, clip, use_s1, load_s1, acc);
    }
    if constexpr (U > 1) fast_run<K, DT, OPT, SL, HD, U / 2>(sp, e, nfull - i, a, G, clip, acc);
}

// One tile that touches a span edge or a group change. tile_e0 is the (rebased) index of the first
// element of the tile, j the bound entry covering the first live element of the tile. Each thread
// looks at its own four elements: all live and in one parameter group -> the vector path with that
// group's constants (held per thread); otherwise -> element by element. Only the few threads whose
// vector straddles the span's first or last element or a bound take the slow way, so such a tile costs
// little more than a full one (ResNet-50's batch-norm tensors and ViT's biases put a group change
// into roughly every hundredth tile; one span per tensor puts an edge into every tensor).
template <int K, int DT, int OPT, int SL, class A, class SP>
__device__ __forceinline__ void careful_tile(const SP& sp, uint64_t tile_e0, const A& a, uint32_t j,
                                             float clip, typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
    using GR = Grad<DT>;
    constexpr int EPT = GR::EPT;
    constexpr int BS = launch_block(K, DT, OPT, SL);
    const bool use_s1 = is_adam(OPT) || (OPT == OPT_SGD && a.opt.has_momentum);
    const bool load_s1 = is_adam(OPT) || (OPT == OPT_SGD && a.opt.has_momentum && !a.opt.first_step);
    ConstBounds bd = sp.bound_count ? const_bounds(a.bounds + sp.bound_begin) : nullptr;
    const uint64_t e_first = tile_e0 + static_cast<uint64_t>(threadIdx.x) * EPT;
    const bool all_live = e_first >= sp.lo && e_first + EPT <= sp.hi;
    bool one_group = true;
    uint32_t gid_first = 0;
    if (bd && all_live) {
        const uint64_t rel = e_first - sp.lo;
        uint32_t jj = j;
        while (jj + 1 < sp.bound_count && bd[jj + 1].start <= rel) ++jj;
        gid_first = bd[jj].group & (JABAS_MAX_GROUPS - 1);
        one_group = jj + 1 >= sp.bound_count || bd[jj + 1].start >= rel + EPT;
    }
    if (all_live && one_group) {
        const GroupDev G = a.groups[gid_first];
        TileRegs<K, DT, 1, OPT> r;
        issue_loads<K, DT, OPT, 1, BS, false>(r, sp, e_first, load_s1);
        consume<K, DT, OPT, SL, false, 1, false>(r, sp, e_first, a, G, clip, use_s1, load_s1, acc);   // halves from the mask: always right
        return;
    }
    for (int i = 0; i < EPT; ++i) {
        const uint64_t e = e_first + i;
        if (e < sp.lo || e >= sp.hi) continue;
        uint32_t gid = 0;
        if (bd) {
            const uint64_t rel = e - sp.lo;
            uint32_t jj = j;
            while (jj + 1 < sp.bound_count && bd[jj + 1].start <= rel) ++jj;
            gid = bd[jj].group & (JABAS_MAX_GROUPS - 1);   // a bound table on the device cannot be checked by the host
        }
        const GroupDev G = a.groups[gid];
        float g[K][1], p[1] = {0.0f}, s1[1] = {0.0f}, s2[1] = {0.0f}, s3[1] = {0.0f}, agg[1];
#pragma unroll
        for (int k = 0; k < K; ++k) g[k][0] = GR::load1(sp.g[k], e);
        [[maybe_unused]] const uint64_t me = is_adam(OPT) ? moment_index(sp, e) : e;
        if constexpr (OPT != OPT_NONE) {
            p[0] = sp.p[e];
            if (load_s1) s1[0] = sp.s1[me];
            if constexpr (is_adam(OPT)) s2[0] = sp.s2[me];
            if constexpr (OPT == OPT_AMS) s3[0] = sp.s3[me];
        }
        compute<K, 1, DT, OPT, SL, false>(g, p, s1, s2, s3, agg, a, G, clip, acc);
        if (sp.out) sp.out[e] = agg[0];
        if constexpr (OPT != OPT_NONE) {
            sp.p[e] = p[0];
            if (use_s1) sp.s1[me] = s1[0];
            if constexpr (is_adam(OPT)) sp.s2[me] = s2[0];
            if constexpr (OPT == OPT_AMS) sp.s3[me] = s3[0];
            for (uint32_t r = 0; r < sp.n_fan; ++r) sp.fan[r][e] = p[0];
        }
    }
}

// Tiles [lt0, lt1) of one span (tile indices local to the span).
template <int K, int DT, int OPT, int SL, bool HD, class A, class SP>
__device__ __forceinline__ void span_range(const SP& sp, uint32_t lt0, uint32_t lt1, uint32_t j0,
                                           const A& a, typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
    const float clip = a.grad_scale ? *a.grad_scale : 1.0f;      // uniform: one scalar load per workgroup
    using GR = Grad<DT>;
    constexpr int EPT = GR::EPT;
    constexpr uint64_t TE = static_cast<uint64_t>(launch_block(K, DT, OPT, SL)) * EPT;
    constexpr int UW = SL ? JABAS_UNROLL_STATS : JABAS_UNROLL_PLAIN;
    constexpr int CT = launch_chunk_tiles(K, DT, OPT, SL);
    constexpr int U0 = UW < CT ? UW : CT;     // never more than a chunk holds
    // 9..16 gradient streams: one tile's loads fill the registers; so do eight fp32 ones beside the 28 fp64 pair
    // sums of the Gram level (two tiles in flight: 256 registers and one wave per SIMD, 13 % slower)
    constexpr int U = (K > 8 || (SL == JABAS_STATS_GRAM && DT == JABAS_F32 && K > 7)) ? 1 : U0;
    static_assert((U & (U - 1)) == 0, "the unroll cascade halves U down to 1");
    const uint32_t nb = sp.bound_count;
    ConstBounds bd = nb ? const_bounds(a.bounds + sp.bound_begin) : nullptr;
    uint32_t lt = lt0, j = j0;
    while (lt < lt1) {
        const uint64_t e0 = static_cast<uint64_t>(lt) * TE;
        const uint64_t cur = e0 > sp.lo ? e0 : sp.lo;
        const uint64_t rel = cur - sp.lo;
        uint64_t stretch_end = sp.hi;
        uint32_t gid = 0;
        if (nb) {
            while (j + 1 < nb && bd[j + 1].start <= rel) ++j;
            gid = bd[j].group & (JABAS_MAX_GROUPS - 1);
            if (j + 1 < nb) stretch_end = sp.lo + bd[j + 1].start;
        }
        uint32_t nfull = 0;
        // spans beyond 32-bit byte offsets take the careful path tile by tile (64-bit addresses there)
        if (e0 >= sp.lo && stretch_end >= e0 + TE && (!narrow_addressing(K, SL) || sp.narrow_ok)) {
            const uint64_t fit = (stretch_end - e0) / TE;
            const uint32_t left = lt1 - lt;
            nfull = fit < left ? static_cast<uint32_t>(fit) : left;
        }
        if (nfull) {
            const GroupDev G = a.groups[gid];
            fast_run<K, DT, OPT, SL, HD, U>(sp, e0 + static_cast<uint64_t>(threadIdx.x) * EPT, nfull, a, G, clip, acc);
            lt += nfull;
        } else {
            careful_tile<K, DT, OPT, SL>(sp, e0, a, j, clip, acc);
            lt += 1;
        }
    }
}

// Statistics kernels carry two copies of the arithmetic: one with the default halves
// (even worker -> A, odd -> B) resolved at compile time, one driven by the half mask.
template <int K, int DT, int OPT, int SL, class A, class SP>
__device__ __forceinline__ void run_chunk(const SP& sp, uint32_t lt0, uint32_t lt1, uint32_t j0, const A& a,
                                          typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
    if constexpr (SL) {
        constexpr uint32_t kDefaultMask = 0xAAAAu & ((1u << K) - 1u);
        if (a.half_mask == kDefaultMask) span_range<K, DT, OPT, SL, true>(sp, lt0, lt1, j0, a, acc);
        else span_range<K, DT, OPT, SL, false>(sp, lt0, lt1, j0, a, acc);
    } else {
        span_range<K, DT, OPT, 0, true>(sp, lt0, lt1, j0, a, acc);
    }
}

// Workgroup sum of NS per-thread accumulators -> one partial row, fp64 accumulators (fp32 gradients).
// Through LDS rather than wave shuffles: NS stores + 16 loads per thread instead of ~18 DPP-and-add
// instructions per value, which matters because a workgroup only covers a few thousand elements.
//   stage 1  thread (v, part) adds entries part, part+16, ..., part+240 of value v (in order);
//   stage 2  the 16 parts of a value sit in one 16-lane row: DPP row reduction.
// BS / 16 values go through the table at a time (16 with 256 threads), so rows wider than that take several
// passes over a table of 32 KB instead of one of up to 80 (pair products of eight workers: 40 values).
// The order is fixed, so the row is bit-identical from run to run.
template <int NS, int BS>
__device__ __forceinline__ void flush_stats(double (&acc)[NS], double* row) {
    constexpr int kParts = 16;                       // lanes of one DPP row
    constexpr int kPerPass = BS / kParts;            // values reduced per pass
    constexpr int kBuf = NS < kPerPass ? NS : kPerPass;
    __shared__ double buf[kBuf][BS];
    const int tid = threadIdx.x;
#pragma unroll
    for (int v0 = 0; v0 < NS; v0 += kPerPass) {
        if (v0) __syncthreads();                     // the table is read out before it is filled again
#pragma unroll
        for (int i = 0; i < kPerPass; ++i)
            if (v0 + i < NS) buf[i][tid] = acc[v0 + i];
        __syncthreads();
        if (tid < (NS - v0) * kParts) {              // at most kPerPass * 16 = BS threads
            const int v = tid >> 4, part = tid & 15;
            double s = buf[v][part];
#pragma unroll
            for (int i = 1; i < BS / kParts; ++i) s += buf[v][i * kParts + part];
            s += dpp_move<0xB1, 0xf>(s);     // quad_perm [1,0,3,2]
            s += dpp_move<0x4E, 0xf>(s);     // quad_perm [2,3,0,1]
            s += dpp_move<0x141, 0xf>(s);    // row_half_mirror
            s += dpp_move<0x140, 0xf>(s);    // row_mirror
            if (part == 0) row[v0 + v] = s;
        }
    }
}

template <int CTRL> __device__ __forceinline__ float dpp_move_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// The same for fp32 accumulators (bf16 gradients). The sums of a 16-lane row are formed first, in fp32 by
// DPP (one instruction per step and value, no LDS traffic, no wait); only one entry per row and value goes
// through LDS, and what follows the barrier is short: thread (v, part) adds entries part, part+16, ... of
// value v in fp64 and the 16 parts meet by DPP. Every lane of the workgroup is active here.
template <int NS, int BS>
__device__ __forceinline__ void flush_stats(float (&acc)[NS], double* row) {
    constexpr int kParts = 16;
    constexpr int kRows = BS / 16;                   // 16-lane rows of the workgroup
    constexpr int kPerPass = BS / kParts;
    __shared__ float buf[NS][kRows];
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        float v = acc[i];
        v += dpp_move_f32<0xB1>(v);          // quad_perm [1,0,3,2]
        v += dpp_move_f32<0x4E>(v);          // quad_perm [2,3,0,1]
        v += dpp_move_f32<0x141>(v);         // row_half_mirror
        v += dpp_move_f32<0x140>(v);         // row_mirror
        if ((tid & 15) == 0) buf[i][tid >> 4] = v;
    }
    __syncthreads();
#pragma unroll
    for (int v0 = 0; v0 < NS; v0 += kPerPass) {
        if (tid < (NS - v0) * kParts) {
            const int v = v0 + (tid >> 4), part = tid & 15;
            double s = 0.0;
#pragma unroll
            for (int i = 0; i < (kRows + kParts - 1) / kParts; ++i)
                if (i * kParts + part < kRows) s += static_cast<double>(buf[v][i * kParts + part]);
            s += dpp_move<0xB1, 0xf>(s);
            s += dpp_move<0x4E, 0xf>(s);
            s += dpp_move<0x141, 0xf>(s);
            s += dpp_move<0x140, 0xf>(s);
            if (part == 0) row[v] = s;
        }
    }
}

// The chunk of workgroup b: a names the launch (spans, chunk table), s the step's scalars (a itself, or the
// view of the device block).
template <int K, int DT, int OPT, int SL, class A>
__device__ __forceinline__ void workgroup_chunk(const KArgs& a, const A& s, uint32_t b,
                                                typename StatAcc<DT>::type (&acc)[NStats<K, SL>::value]) {
    constexpr int BS = launch_block(K, DT, OPT, SL);
    constexpr uint32_t CT = launch_chunk_tiles(K, DT, OPT, SL);     // the host cuts the chunk table for the same shape
    constexpr uint64_t TE = static_cast<uint64_t>(BS) * Grad<DT>::EPT;
    if (a.use_inline) {
        const SpanDev& sp = a.span0;
        const uint32_t tiles = static_cast<uint32_t>((sp.hi + TE - 1) / TE);
        const uint32_t lt0 = b * CT;
        const uint32_t lt1 = lt0 + CT < tiles ? lt0 + CT : tiles;
        uint32_t j0 = 0;
        if (sp.bound_count) {                  // largest j with bounds[j].start <= first live element
            ConstBounds bd = const_bounds(a.bounds + sp.bound_begin);
            const uint64_t e0 = static_cast<uint64_t>(lt0) * TE;
            const uint64_t rel = (e0 > sp.lo ? e0 : sp.lo) - sp.lo;
            uint32_t lo = 0, hi = sp.bound_count;
            while (hi - lo > 1) {
                const uint32_t mid = (lo + hi) >> 1;
                if (bd[mid].start <= rel) lo = mid; else hi = mid;
            }
            j0 = lo;
        }
        run_chunk<K, DT, OPT, SL>(sp, lt0, lt1, j0, s, acc);
    } else {
        // The plan's tables are not written while a launch that names them runs: read through the constant
        // address space, their fields are loaded like kernel arguments (uniform loads the compiler may move,
        // repeat or keep as it likes) instead of being fetched again after every store that might alias them.
        typedef const __attribute__((address_space(4))) ChunkDesc* ConstChunk;
        typedef __attribute__((address_space(4))) SpanDev ConstSpan;
        ConstChunk cp = (ConstChunk)(a.chunks + b);
        const uint32_t c_span = cp->span, c_tile0 = cp->tile0, c_bound0 = cp->bound0;
        const ConstSpan& sp = *(const ConstSpan*)(a.spans + c_span);
        const uint32_t tiles = static_cast<uint32_t>((sp.hi + TE - 1) / TE);
        const uint32_t lt1 = c_tile0 + CT < tiles ? c_tile0 + CT : tiles;
        run_chunk<K, DT, OPT, SL>(sp, c_tile0, lt1, c_bound0, s, acc);
    }
}

// DYN: the step's scalars are read from the device block a.dyn names (a launch that a HIP graph replays
// with another learning rate or Adam step) instead of from the kernel arguments.
template <int K, int DT, int OPT, int SL, bool DYN>
__global__ void __launch_bounds__(launch_block(K, DT, OPT, SL)) fused_kernel(const KArgs a) {
    constexpr int NS = NStats<K, SL>::value;
    constexpr int BS = launch_block(K, DT, OPT, SL);
    const uint32_t b = blockIdx.x;
    typename StatAcc<DT>::type acc[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) acc[i] = 0;
    if constexpr (DYN) {
        const DynView s(a);
        workgroup_chunk<K, DT, OPT, SL>(a, s, b, acc);
    } else {
        workgroup_chunk<K, DT, OPT, SL>(a, a, b, acc);
    }
    if constexpr (SL) flush_stats<NS, BS>(acc, a.partials + static_cast<uint64_t>(b) * NS);   // compact rows of 4 + K
}

template <int K, int DT, int OPT, int SL>
int launch_one(const KArgs& a, unsigned grid, hipStream_t stream, bool dyn) {
    // Residency cap through idle dynamic LDS (160 KB per CU). Fewer resident workgroups keep the
    // streamed window of every buffer more compact, which the memory system rewards on write-heavy
    // mixes as long as the kernel does not need the waves to hide its own arithmetic. Measured (A/B in
    // one process, and over whole bench runs with rotating buffers): Adam/AdamW at K <= 4 with fp32
    // gradients gains 0-4 % without statistics at 5 workgroups per CU instead of the 6 its registers
    // allow, and 0.2-2.4 % with statistics at 3 workgroups per CU instead of 4 (more with replica
    // weights to refresh); SGD kernels, bf16 gradients and K > 4 lose or stay flat.
#ifndef JABAS_IDLE_LDS_BYTES
#define JABAS_IDLE_LDS_BYTES 32768u
#endif
#ifndef JABAS_STATS_LDS_BYTES
#define JABAS_STATS_LDS_BYTES 53248u      // per workgroup, flush_stats' own table included: three workgroups per CU
#endif
    constexpr bool capped = OPT == OPT_ADAM && K <= 4 && DT == JABAS_F32;
    constexpr unsigned flush_bytes = imin(NStats<K, SL>::value, launch_block(K, DT, OPT, SL) / 16) * launch_block(K, DT, OPT, SL) * 8u;   // flush_stats' fp64 table
    static_assert(!capped || !SL || flush_bytes < JABAS_STATS_LDS_BYTES, "the cap is what is left beside the table");
    constexpr unsigned idle = !capped ? 0u : SL ? JABAS_STATS_LDS_BYTES - flush_bytes : JABAS_IDLE_LDS_BYTES;
    const dim3 block(launch_block(K, DT, OPT, SL));
    if constexpr (SL == JABAS_STATS_GRAM && K > JABAS_STATS_GRAM_MAX_K) {
        return static_cast<int>(hipErrorInvalidValue);              // refused by the front before it gets here
    } else {
        if constexpr (OPT == OPT_SGD || OPT == OPT_ADAM) {
            if (dyn) return static_cast<int>(launch_kernel(fused_kernel<K, DT, OPT, SL, true>, dim3(grid), block, idle, stream, a));
        } else {
            if (dyn) return static_cast<int>(hipErrorInvalidValue);     // refused by the front before it gets here
        }
        return static_cast<int>(launch_kernel(fused_kernel<K, DT, OPT, SL, false>, dim3(grid), block, idle, stream, a));
    }
}

}  // namespace

#define JABAS_CAT_(a, b) a##b
#define JABAS_CAT(a, b) JABAS_CAT_(a, b)

#define JABAS_DISPATCH(FN, ...)                                                              \
    const int key = (opt_class * 2 + (grad_dtype == JABAS_BF16 ? 1 : 0)) * 4 + stats;           \
    switch (key) {                                                                           \
        case 0: return FN<JABAS_K, JABAS_F32, OPT_NONE, 0>(__VA_ARGS__);                     \
        case 1: return FN<JABAS_K, JABAS_F32, OPT_NONE, 1>(__VA_ARGS__);                     \
        case 2: return FN<JABAS_K, JABAS_F32, OPT_NONE, 2>(__VA_ARGS__);                     \
        case 3: return FN<JABAS_K, JABAS_F32, OPT_NONE, 3>(__VA_ARGS__);                     \
        case 4: return FN<JABAS_K, JABAS_BF16, OPT_NONE, 0>(__VA_ARGS__);                    \
        case 5: return FN<JABAS_K, JABAS_BF16, OPT_NONE, 1>(__VA_ARGS__);                    \
        case 6: return FN<JABAS_K, JABAS_BF16, OPT_NONE, 2>(__VA_ARGS__);                    \
        case 7: return FN<JABAS_K, JABAS_BF16, OPT_NONE, 3>(__VA_ARGS__);                    \
        case 8: return FN<JABAS_K, JABAS_F32, OPT_SGD, 0>(__VA_ARGS__);                      \
        case 9: return FN<JABAS_K, JABAS_F32, OPT_SGD, 1>(__VA_ARGS__);                      \
        case 10: return FN<JABAS_K, JABAS_F32, OPT_SGD, 2>(__VA_ARGS__);                     \
        case 11: return FN<JABAS_K, JABAS_F32, OPT_SGD, 3>(__VA_ARGS__);                     \
        case 12: return FN<JABAS_K, JABAS_BF16, OPT_SGD, 0>(__VA_ARGS__);                    \
        case 13: return FN<JABAS_K, JABAS_BF16, OPT_SGD, 1>(__VA_ARGS__);                    \
        case 14: return FN<JABAS_K, JABAS_BF16, OPT_SGD, 2>(__VA_ARGS__);                    \
        case 15: return FN<JABAS_K, JABAS_BF16, OPT_SGD, 3>(__VA_ARGS__);                    \
        case 16: return FN<JABAS_K, JABAS_F32, OPT_ADAM, 0>(__VA_ARGS__);                    \
        case 17: return FN<JABAS_K, JABAS_F32, OPT_ADAM, 1>(__VA_ARGS__);                    \
        case 18: return FN<JABAS_K, JABAS_F32, OPT_ADAM, 2>(__VA_ARGS__);                    \
        case 19: return FN<JABAS_K, JABAS_F32, OPT_ADAM, 3>(__VA_ARGS__);                    \
        case 20: return FN<JABAS_K, JABAS_BF16, OPT_ADAM, 0>(__VA_ARGS__);                   \
        case 21: return FN<JABAS_K, JABAS_BF16, OPT_ADAM, 1>(__VA_ARGS__);                   \
        case 22: return FN<JABAS_K, JABAS_BF16, OPT_ADAM, 2>(__VA_ARGS__);                   \
        case 23: return FN<JABAS_K, JABAS_BF16, OPT_ADAM, 3>(__VA_ARGS__);                   \
        case 24: return FN<JABAS_K, JABAS_F32, OPT_AMS, 0>(__VA_ARGS__);                     \
        case 25: return FN<JABAS_K, JABAS_F32, OPT_AMS, 1>(__VA_ARGS__);                     \
        case 26: return FN<JABAS_K, JABAS_F32, OPT_AMS, 2>(__VA_ARGS__);                     \
        case 27: return FN<JABAS_K, JABAS_F32, OPT_AMS, 3>(__VA_ARGS__);                     \
        case 28: return FN<JABAS_K, JABAS_BF16, OPT_AMS, 0>(__VA_ARGS__);                    \
        case 29: return FN<JABAS_K, JABAS_BF16, OPT_AMS, 1>(__VA_ARGS__);                    \
        case 30: return FN<JABAS_K, JABAS_BF16, OPT_AMS, 2>(__VA_ARGS__);                    \
        case 31: return FN<JABAS_K, JABAS_BF16, OPT_AMS, 3>(__VA_ARGS__);                    \
        default: return -1;                                                                  \
    }

int JABAS_CAT(launch_fused_k, JABAS_K)(int grad_dtype, int opt_class, int stats, int dyn, const KArgs& a,
                                       unsigned grid, hipStream_t stream) {
    JABAS_DISPATCH(launch_one, a, grid, stream, dyn != 0)
}

}  // namespace jabas
