// C ABI of libjabas_sync.so: argument validation, plan encoding, derivation of the fp32
// kernel constants, grid sizing, and the finalize kernel of the two-level statistics
// reduction. The streaming kernels themselves live in fused_kernel.hip / gram_kernel.hip.
#include <math.h>
#include <string.h>

#include <atomic>

#include "jabas_internal.h"

#define JABAS_API extern "C" __attribute__((visibility("default")))

namespace jabas {

int launch_gram(int K, int grad_dtype, const SpanDev& sp, double* partials, unsigned grid, hipStream_t stream);
int launch_gram_finalize(int K, int grad_dtype, double* partials, unsigned grid, unsigned spare_rows, double* gram_out,
                         hipStream_t stream);

namespace {

#ifndef JABAS_GRAM_GRID
#define JABAS_GRAM_GRID 1024
#endif
constexpr uint64_t kGramGrid = JABAS_GRAM_GRID;     // persistent workgroups of the Gram kernel
constexpr uint32_t kPlanMagic = 0x4a425359u;  // "JBSY"
constexpr uint32_t kPlanVersion = 8;

// A plan holds one chunk table per launch shape, indexed by the statistics level of the launch (0 none,
// 1 full rows, 2 similarity sums). Levels whose shapes are the same share one table.
struct PlanShape {
    uint32_t block;           // threads per workgroup the chunk table was cut for
    uint32_t chunk_tiles;     // tiles per workgroup
    uint32_t n_chunks;        // workgroups of one launch
    uint32_t max_span_chunks; // chunks of the largest span (sizes the striped finalize)
    uint64_t off_prefix, off_chunks;
};
struct PlanHeader {
    uint32_t magic, version;
    uint32_t n_span, n_bounds;
    int32_t K, grad_dtype, opt_kind;
    uint32_t max_group;       // largest group index any bound names
    uint32_t all_have_s1;     // every non-empty span carries a state1 pointer
    uint32_t pad;
    PlanShape shape[3];
    uint64_t off_spans, off_bounds, total_bytes;
};
static_assert(sizeof(PlanShape) == 32 && sizeof(PlanHeader) == 160, "plan header layout");
constexpr size_t kHeaderBytes = 160;
static_assert(kHeaderBytes >= sizeof(PlanHeader) && kHeaderBytes % 16 == 0, "plan header slot");

inline size_t align16(size_t x) { return (x + 15) & ~static_cast<size_t>(15); }

inline int opt_class_of(int kind) {
    switch (kind) {
        case JABAS_OPT_NONE: return 0;
        case JABAS_OPT_SGD: return 1;
        case JABAS_OPT_ADAM:
        case JABAS_OPT_ADAMW: return 2;
        case JABAS_OPT_ADAM_AMSGRAD:
        case JABAS_OPT_ADAMW_AMSGRAD: return 3;
        default: return -1;
    }
}

inline bool ranges_overlap(const void* a, size_t na, const void* b, size_t nb) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + nb && b0 < a0 + na;
}

// The live range of a span starts `skew` elements into the kernels' element grid. When every buffer
// of the span sits at the same element offset within kWideElems elements (256 bytes of fp32), the
// grid starts at that 256-byte line: every full tile then reads and writes whole cache lines, which
// is worth 8-17 % of the rate on spans that start at arbitrary elements. Otherwise the grid starts
// at the 16-byte line of the first element, the least the vector accesses need.
constexpr uint32_t kWideElems = 64;
inline uint64_t tiles_of(uint64_t hi, int block) {
    const uint64_t te = tile_elems_of(block);
    return (hi + te - 1) / te;
}
inline uint64_t chunks_of_tiles(uint64_t tiles, uint64_t ct) { return (tiles + ct - 1) / ct; }

// Validates one span and produces the rebased device view. Host-only logic.
int encode_span(const JabasSpan& in, int K, int grad_dtype, int opt_kind, int block, SpanDev* out, uint32_t* tiles) {
    const int gs = grad_dtype == JABAS_BF16 ? 2 : 4;
    const int ept = ept_of(grad_dtype);
    if (in.numel > (static_cast<uint64_t>(1) << 40)) return JABAS_ERR_SIZE;
    if (in.n_fanout > JABAS_MAX_K - 1) return JABAS_ERR_SIZE;
    if (in.numel == 0) {                       // empty span: nothing to read, pointers may be NULL
        memset(out, 0, sizeof(*out));
        *tiles = 0;
        return JABAS_OK;
    }
    for (int k = 0; k < K; ++k)
        if (!in.grads[k]) return JABAS_ERR_NULL;
    const int oc = opt_class_of(opt_kind);
    if (oc < 0) return JABAS_ERR_OPT;
    if (oc != 0 && !in.param) return JABAS_ERR_NULL;
    if (oc >= 2 && (!in.state1 || !in.state2)) return JABAS_ERR_NULL;
    if (oc == 3 && !in.state3) return JABAS_ERR_NULL;
    if (oc == 0 && in.n_fanout) return JABAS_ERR_OPT;
    for (uint32_t r = 0; r < in.n_fanout; ++r)
        if (!in.fanout[r]) return JABAS_ERR_NULL;
    // interleaved moments: the span's place in an arena of alternating blocks of T elements per moment
    const uint32_t il_log2 = in.state_block_log2;
    const uint64_t il_T = il_log2 ? static_cast<uint64_t>(1) << (il_log2 & 31) : 0;
    const uint64_t il_ways = oc == 3 ? 3 : 2;
    if (il_log2) {
        if (oc < 2) return JABAS_ERR_OPT;
        if (il_log2 < 8 || il_log2 > 24 || in.state_block_pos >= il_T) return JABAS_ERR_SIZE;
        const uintptr_t s1a = reinterpret_cast<uintptr_t>(in.state1);
        if (reinterpret_cast<uintptr_t>(in.state2) != s1a + il_T * 4) return JABAS_ERR_ALIGN;
        if (oc == 3 && reinterpret_cast<uintptr_t>(in.state3) != s1a + il_T * 8) return JABAS_ERR_ALIGN;
        if (s1a < static_cast<uintptr_t>(in.state_block_pos) * 4 || (s1a - static_cast<uintptr_t>(in.state_block_pos) * 4) % 16)
            return JABAS_ERR_ALIGN;
    }
    // bytes from state1 to the end of the last element's last moment (one written range when interleaved)
    uint64_t il_bytes = 0;
    if (il_log2) {
        const uint64_t tl = in.state_block_pos + in.numel - 1;
        il_bytes = 4 * (tl + (il_ways - 1) * (tl & ~(il_T - 1)) + (il_ways - 1) * il_T + 1 - in.state_block_pos);
    }

    const uintptr_t g0 = reinterpret_cast<uintptr_t>(in.grads[0]);
    if (g0 % gs) return JABAS_ERR_ALIGN;
    const uint32_t wide_skew = static_cast<uint32_t>((g0 / gs) % kWideElems);
    bool wide = true;
    auto same_wide = [&](const void* p, int es) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        if (p && (a % es || (a / es) % kWideElems != wide_skew)) wide = false;
    };
    for (int k = 0; k < K; ++k) same_wide(in.grads[k], gs);
    same_wide(in.agg_out, 4);
    if (oc != 0) {
        same_wide(in.param, 4);
        same_wide(in.state1, 4);
        if (!il_log2) {                        // interleaved: state2 and state3 sit whole blocks behind state1
            same_wide(in.state2, 4);
            if (oc == 3) same_wide(in.state3, 4);
        }
        for (uint32_t r = 0; r < in.n_fanout; ++r) same_wide(in.fanout[r], 4);
    }
    // elements before the line the grid starts at
    const uint32_t skew = wide ? wide_skew : static_cast<uint32_t>((g0 / gs) % ept);
    auto rebase_g = [&](const void* p, const void** dst) -> bool {
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        if (a % gs || (a / gs) % ept != skew % ept) return false;
        *dst = reinterpret_cast<const void*>(a - static_cast<uintptr_t>(skew) * gs);
        return true;
    };
    auto rebase_f = [&](float* p, float** dst) -> bool {
        if (!p) { *dst = nullptr; return true; }
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        if (a % 4 || (a / 4) % 4 != skew % 4) return false;
        *dst = reinterpret_cast<float*>(a - static_cast<uintptr_t>(skew) * 4);
        return true;
    };
    memset(out, 0, sizeof(*out));
    for (int k = 0; k < K; ++k)
        if (!rebase_g(in.grads[k], &out->g[k])) return JABAS_ERR_ALIGN;
    if (!rebase_f(in.agg_out, &out->out)) return JABAS_ERR_ALIGN;
    if (oc != 0) {
        if (!rebase_f(in.param, &out->p) || !rebase_f(in.state1, &out->s1)) return JABAS_ERR_ALIGN;
        if (il_log2) {
            // the moment bases are the start of the span's first block group; a grid element finds its moments
            // through its position in the arena (SpanDev::mom_*). state1 passed the congruence check above and
            // the block group starts on a 16-byte line, so a thread's four elements never straddle a block.
            float* group = in.state1 - in.state_block_pos;
            out->s1 = group;
            out->s2 = group + il_T;
            out->s3 = oc == 3 ? group + 2 * il_T : nullptr;
            out->mom_add = static_cast<uint64_t>(in.state_block_pos) - skew;
            out->mom_mask = ~(il_T - 1);
            out->mom_mult = static_cast<uint32_t>(il_ways - 1);
        } else {
            if (!rebase_f(in.state2, &out->s2)) return JABAS_ERR_ALIGN;
            if (oc == 3 && !rebase_f(in.state3, &out->s3)) return JABAS_ERR_ALIGN;
        }
        for (uint32_t r = 0; r < in.n_fanout; ++r)
            if (!rebase_f(in.fanout[r], &out->fan[r])) return JABAS_ERR_ALIGN;
        out->n_fan = in.n_fanout;
    }
    if (in.agg_out) {
        const size_t ob = in.numel * 4;
        for (int k = 0; k < K; ++k) {
            if (!ranges_overlap(in.agg_out, ob, in.grads[k], in.numel * gs)) continue;
            if (grad_dtype != JABAS_F32 || static_cast<const void*>(in.agg_out) != in.grads[k]) return JABAS_ERR_ALIAS;
        }
    }
    // Every buffer the launch writes must be disjoint from every other buffer of the span (the
    // in-place aggregate above is the one exception): each element is read and written by a
    // different thread at a different time, so any overlap would be a silent race.
    const void* written[5 + JABAS_MAX_K - 1];
    size_t wbytes[5 + JABAS_MAX_K - 1];
    const size_t fb = in.numel * 4;
    int nw = 0;
    auto add_written = [&](const void* p, size_t bytes) { written[nw] = p; wbytes[nw++] = bytes; };
    if (in.agg_out) add_written(in.agg_out, fb);
    if (oc != 0) {
        add_written(in.param, fb);
        if (il_log2) {
            add_written(in.state1, il_bytes);
        } else {
            if (in.state1) add_written(in.state1, fb);
            if (oc >= 2) add_written(in.state2, fb);
            if (oc == 3) add_written(in.state3, fb);
        }
        for (uint32_t r = 0; r < in.n_fanout; ++r) add_written(in.fanout[r], fb);
    }
    for (int i = 0; i < nw; ++i) {
        for (int j = i + 1; j < nw; ++j)
            if (ranges_overlap(written[i], wbytes[i], written[j], wbytes[j])) return JABAS_ERR_ALIAS;
        if (written[i] == static_cast<const void*>(in.agg_out)) continue;      // checked against the gradients above
        for (int k = 0; k < K; ++k)
            if (ranges_overlap(written[i], wbytes[i], in.grads[k], in.numel * gs)) return JABAS_ERR_ALIAS;
    }
    out->lo = skew;
    out->hi = skew + in.numel;
    out->narrow_ok = out->hi <= kNarrowElems &&
                     (!il_log2 || il_ways * (in.state_block_pos + in.numel + il_T) <= kNarrowElems);
    out->bound_begin = in.bound_begin;
    out->bound_count = in.bound_count;
    const uint64_t nt = tiles_of(out->hi, block);
    if (nt > 0x7fffffffull) return JABAS_ERR_SIZE;
    *tiles = static_cast<uint32_t>(nt);
    return JABAS_OK;
}

int check_bounds_host(const JabasSpan& sp, const JabasBound* bounds, uint32_t n_bounds, uint32_t* max_group) {
    if (sp.bound_count == 0) return JABAS_OK;
    if (!bounds) return JABAS_ERR_NULL;
    if (static_cast<uint64_t>(sp.bound_begin) + sp.bound_count > n_bounds) return JABAS_ERR_GROUP;
    const JabasBound* b = bounds + sp.bound_begin;
    if (b[0].start != 0) return JABAS_ERR_GROUP;
    for (uint32_t i = 0; i < sp.bound_count; ++i) {
        if (b[i].group >= JABAS_MAX_GROUPS) return JABAS_ERR_GROUP;
        if (i && b[i].start <= b[i - 1].start) return JABAS_ERR_GROUP;
        if (sp.numel && b[i].start >= sp.numel && i) return JABAS_ERR_GROUP;
        if (b[i].group > *max_group) *max_group = b[i].group;
    }
    return JABAS_OK;
}

// StepArgs (doubles, as the Python optimizer holds them) -> the fp32 scalars the kernels read.
int fill_step_scal(const JabasStepArgs* s, StepScal* a) {
    if (!s) return JABAS_ERR_NULL;
    if (s->K < 1 || s->K > JABAS_MAX_K) return JABAS_ERR_K;
    if (s->grad_dtype != JABAS_F32 && s->grad_dtype != JABAS_BF16) return JABAS_ERR_DTYPE;
    const int oc = opt_class_of(s->opt_kind);
    if (oc < 0) return JABAS_ERR_OPT;
    if (s->stats < JABAS_STATS_NONE || s->stats > JABAS_STATS_GRAM) return JABAS_ERR_OPT;
    if (s->stats == JABAS_STATS_GRAM && s->K > JABAS_STATS_GRAM_MAX_K) return JABAS_ERR_K;
    memset(a, 0, sizeof(*a));
    uint32_t mask = 0;
    for (int k = 0; k < s->K; ++k) {
        a->w[k] = s->weight[k];
        a->wh[k] = s->half_weight[k];
        if (s->half_id[k] > 1) return JABAS_ERR_K;
        if (s->half_id[k]) mask |= 1u << k;
    }
    a->half_mask = mask;
    if (oc == 0) return JABAS_OK;
    if (s->n_groups < 1 || s->n_groups > JABAS_MAX_GROUPS) return JABAS_ERR_GROUP;
    OptDev& o = a->opt;
    o.momentum = static_cast<float>(s->momentum);
    o.one_minus_damp = static_cast<float>(1.0 - s->dampening);
    o.beta1 = static_cast<float>(s->beta1);
    o.one_minus_beta1 = static_cast<float>(1.0 - s->beta1);
    o.beta2 = static_cast<float>(s->beta2);
    o.one_minus_beta2 = static_cast<float>(1.0 - s->beta2);
    o.eps = static_cast<float>(s->eps);
    o.has_momentum = (oc == 1 && s->momentum != 0.0) ? 1 : 0;
    o.first_step = s->first_step ? 1 : 0;
    o.nesterov = s->nesterov ? 1 : 0;
    o.adamw = (s->opt_kind == JABAS_OPT_ADAMW || s->opt_kind == JABAS_OPT_ADAMW_AMSGRAD) ? 1 : 0;
    if (oc == 1 && o.nesterov && (s->momentum <= 0.0 || s->dampening != 0.0)) return JABAS_ERR_OPT;
    for (int i = 0; i < s->n_groups; ++i) {
        const JabasGroup& g = s->groups[i];
        GroupDev& d = a->groups[i];
        d.wd = static_cast<float>(g.weight_decay);
        d.neg_lr = static_cast<float>(-g.lr);
        d.decay = static_cast<float>(1.0 - g.lr * g.weight_decay);
        d.neg_step_size = 0.0f;
        d.sqrt_bc2 = 1.0f;
        if (oc >= 2) {
            if (g.step < 1) return JABAS_ERR_OPT;
            const double bc1 = 1.0 - pow(s->beta1, static_cast<double>(g.step));
            const double bc2 = 1.0 - pow(s->beta2, static_cast<double>(g.step));
            d.neg_step_size = static_cast<float>(-(g.lr / bc1));
            d.sqrt_bc2 = static_cast<float>(sqrt(bc2));
        }
    }
    return JABAS_OK;
}

// The launch arguments' share of a step: the scalars by value, and the device block when the caller names one
// (the by-value copy is then what the call was checked against, the kernel reads the block).
int fill_kargs(const JabasStepArgs* s, KArgs* a) {
    StepScal sc;
    const int rc = fill_step_scal(s, &sc);
    if (rc != JABAS_OK) return rc;
    memset(a, 0, sizeof(*a));
    memcpy(a->w, sc.w, sizeof(sc.w));
    memcpy(a->wh, sc.wh, sizeof(sc.wh));
    a->half_mask = sc.half_mask;
    a->opt = sc.opt;
    memcpy(a->groups, sc.groups, sizeof(sc.groups));
    a->grad_scale = s->grad_scale;
    if (s->scalars_dev) {
        const int oc = opt_class_of(s->opt_kind);
        if (oc == 0) return JABAS_ERR_OPT;           // nothing of an aggregate-only launch moves between steps
        if (oc == 3) return JABAS_ERR_OPT;           // the amsgrad kernels take their scalars by value only
        if (reinterpret_cast<uintptr_t>(s->scalars_dev) % 16) return JABAS_ERR_ALIGN;
        a->dyn = static_cast<const StepScal*>(s->scalars_dev);
    }
    return JABAS_OK;
}

typedef int (*LaunchFn)(int, int, int, int, const KArgs&, unsigned, hipStream_t);
const LaunchFn kLaunch[JABAS_MAX_K] = {launch_fused_k1,  launch_fused_k2,  launch_fused_k3,  launch_fused_k4,
                                       launch_fused_k5,  launch_fused_k6,  launch_fused_k7,  launch_fused_k8,
                                       launch_fused_k9,  launch_fused_k10, launch_fused_k11, launch_fused_k12,
                                       launch_fused_k13, launch_fused_k14, launch_fused_k15, launch_fused_k16};

// Second level of the statistics reduction: sums partial rows in a fixed order.
//   stripes == 0  rows [s*in_stripes, (s+1)*in_stripes) of `in` -> row s of `out`
//   stripes >= 1  stripe j = blockIdx.x of the chunk rows of span s = blockIdx.y -> row s*stripes + j
// Thread t adds rows t, t+256, ... in increasing order; the 256 per-thread sums then go
// through the fixed wave tree and a wave-order sum, so the result does not depend on the
// machine or on timing. A span with many chunks is cut into stripes (one workgroup each,
// then one more launch over the stripe rows) because a single workgroup reads its rows at
// the bandwidth of one CU.
constexpr int kFinalizeBlock = 256;
constexpr uint32_t kStripeRows = 512;        // chunk rows one workgroup sums in the striped launch
constexpr uint32_t kMaxStripes = 32;
constexpr uint32_t kSingleLaunchRows = 2560; // up to here one workgroup per span finishes in about 6 us
constexpr uint32_t kMaxStatsSpans = 65535;   // spans index the y dimension of the finalize grid
template <int NS>
__global__ void __launch_bounds__(kFinalizeBlock) finalize_stats_kernel(const uint32_t* chunk_prefix, uint32_t n_chunks,
                                                                        uint32_t use_inline, uint32_t stripes,
                                                                        uint32_t in_stripes, uint32_t out_stride,
                                                                        const double* in, double* out) {
    // input rows are compact (NS doubles each, the width of the level); output rows have out_stride slots, the unused ones 0
    __shared__ double red[kFinalizeBlock / 64][NS];
    const uint32_t s = blockIdx.y, j = blockIdx.x, t = threadIdx.x;
    uint32_t c0, c1, o;
    if (stripes == 0) {
        c0 = s * in_stripes;
        c1 = c0 + in_stripes;
        o = s;
    } else {
        uint32_t b0 = 0, b1 = n_chunks;
        if (!use_inline) { b0 = chunk_prefix[s]; b1 = chunk_prefix[s + 1]; }
        const uint32_t per = (b1 - b0 + stripes - 1) / stripes;
        c0 = b0 + j * per < b1 ? b0 + j * per : b1;
        c1 = c0 + per < b1 ? c0 + per : b1;
        o = s * stripes + j;
    }
    double acc[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) acc[i] = 0.0;
#pragma unroll 2
    for (uint32_t c = c0 + t; c < c1; c += kFinalizeBlock) {
        const double* row = in + static_cast<uint64_t>(c) * NS;
#pragma unroll
        for (int i = 0; i < NS; ++i) acc[i] += row[i];
    }
    const int lane = t & 63, wave = t >> 6;
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const double v = wave_sum_to_lane63(acc[i]);
        if (lane == 63) red[wave][i] = v;
    }
    __syncthreads();
    if (t < out_stride) {
        double sum = 0.0;
        if (t < NS) {
            sum = red[0][t];
#pragma unroll
            for (int w = 1; w < kFinalizeBlock / 64; ++w) sum += red[w][t];
        }
        out[static_cast<uint64_t>(o) * out_stride + t] = sum;
    }
}

template <int NS>
hipError_t launch_finalize(dim3 grid, hipStream_t stream, const KArgs& a, uint32_t stripes, uint32_t in_stripes,
                           uint32_t out_stride, const double* in, double* out) {
    return launch_kernel(finalize_stats_kernel<NS>, grid, dim3(kFinalizeBlock), 0, stream, a.chunk_prefix, a.n_chunks,
                         a.use_inline, stripes, in_stripes, out_stride, in, out);
}
// One instantiation per row width: 4 (similarity sums), 4 + K, K = 1..16, and 4 + K + K(K-1)/2 for K <= 8
// (7, 10, 14, 19: among the widths of the full rows; 25, 32, 40).
hipError_t finalize(int ns, dim3 grid, hipStream_t stream, const KArgs& a, uint32_t stripes, uint32_t in_stripes,
                    uint32_t out_stride, const double* in, double* out) {
    switch (ns) {
#define JABAS_FIN(n) case n: return launch_finalize<n>(grid, stream, a, stripes, in_stripes, out_stride, in, out);
        JABAS_FIN(4) JABAS_FIN(5) JABAS_FIN(6) JABAS_FIN(7) JABAS_FIN(8) JABAS_FIN(9) JABAS_FIN(10) JABAS_FIN(11) JABAS_FIN(12)
        JABAS_FIN(13) JABAS_FIN(14) JABAS_FIN(15) JABAS_FIN(16) JABAS_FIN(17) JABAS_FIN(18) JABAS_FIN(19) JABAS_FIN(20) JABAS_FIN(25)
        JABAS_FIN(32) JABAS_FIN(40)
#undef JABAS_FIN
        default: return hipErrorInvalidValue;
    }
}

inline uint32_t stripes_for(uint32_t max_span_chunks) {
    if (max_span_chunks <= kSingleLaunchRows) return 1;      // a second launch costs more than it saves
    const uint32_t st = (max_span_chunks + kStripeRows - 1) / kStripeRows;
    return st > kMaxStripes ? kMaxStripes : st;
}
// workspace rows: one per chunk, then one per (span, stripe)
constexpr size_t workspace_rows(uint64_t n_chunks, uint64_t n_span) { return n_chunks + n_span * kMaxStripes + 1; }

// One wave: fixed-order sum of slot NORM_AGG over the rows, then the coefficient.
__global__ void __launch_bounds__(64) clip_coef_kernel(const double* rows, uint32_t n_rows, double max_norm, double eps,
                                                       float* coef_out) {
    double acc = 0.0;
    for (uint32_t r = threadIdx.x; r < n_rows; r += 64) acc += rows[static_cast<uint64_t>(r) * kStatsStride + JABAS_STAT_NORM_AGG];
    const double total = wave_sum_to_lane63(acc);
    if (threadIdx.x == 63) *coef_out = static_cast<float>(max_norm / (sqrt(total) + eps));
}

int run_fused(KArgs& a, const JabasStepArgs* s, uint32_t max_span_chunks, double* stats_out, void* workspace,
              size_t workspace_bytes, hipStream_t stream) {
    const int oc = opt_class_of(s->opt_kind);
    const int stats = s->stats;                  // level, checked by fill_kargs
    if (stats) {
        if (!stats_out) return JABAS_ERR_NULL;
        if (a.n_span > kMaxStatsSpans) return JABAS_ERR_SIZE;     // before anything is launched: no half-done step
        if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 8) return JABAS_ERR_WORKSPACE;
        // one compact partial row per chunk and per (span, stripe), as wide as the level's rows are
        if (workspace_bytes < workspace_rows(a.n_chunks, a.n_span) * stats_row_width(s->K, stats) * sizeof(double))
            return JABAS_ERR_WORKSPACE;
        if (reinterpret_cast<uintptr_t>(stats_out) % 8) return JABAS_ERR_ALIGN;
    }
    a.partials = static_cast<double*>(workspace);
    if (a.n_chunks) {
        const int err = kLaunch[s->K - 1](s->grad_dtype, oc, stats, a.dyn != nullptr, a, a.n_chunks, stream);
        if (err != 0) return JABAS_ERR_LAUNCH;
    }
    if (stats) {
        const uint32_t st = stripes_for(max_span_chunks);
        const int ns = stats_row_width(s->K, stats);                // width of the partial rows
        hipError_t err;
        if (st == 1) {
            err = finalize(ns, dim3(1, a.n_span), stream, a, 1u, 0u, kStatsStride, a.partials, stats_out);
        } else {
            double* level2 = a.partials + static_cast<uint64_t>(a.n_chunks) * ns;
            err = finalize(ns, dim3(st, a.n_span), stream, a, st, 0u, static_cast<uint32_t>(ns), a.partials, level2);
            if (err == hipSuccess)
                err = finalize(ns, dim3(1, a.n_span), stream, a, 0u, st, kStatsStride, level2, stats_out);
        }
        if (err != hipSuccess) return JABAS_ERR_LAUNCH;
    }
    return JABAS_OK;
}

}  // namespace
}  // namespace jabas

using namespace jabas;

JABAS_API const char* jabas_sync_version(void) { return "jabas_sync 0.6 (gfx950)"; }

JABAS_API const char* jabas_status_string(int status) {
    switch (status) {
        case JABAS_OK: return "ok";
        case JABAS_ERR_NULL: return "a required pointer is NULL";
        case JABAS_ERR_K: return "K outside 1..16 or half_id not 0/1";
        case JABAS_ERR_ALIGN: return "buffers of a span are not mutually congruent modulo 16 bytes";
        case JABAS_ERR_DTYPE: return "unsupported gradient dtype";
        case JABAS_ERR_OPT: return "unknown optimizer kind or inconsistent optimizer arguments";
        case JABAS_ERR_GROUP: return "parameter group index/count out of range or bounds not sorted";
        case JABAS_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case JABAS_ERR_PLAN: return "plan blob malformed, too small or not matching the step arguments";
        case JABAS_ERR_SIZE: return "element, span or fan-out count out of range (jabas_sync_bucket_static: more than JABAS_STATIC_MAX_NUMEL elements)";
        case JABAS_ERR_LAUNCH: return "HIP runtime refused the kernel launch";
        case JABAS_ERR_ALIAS: return "a written buffer overlaps another buffer of the span (only agg_out == grads[k], fp32, may alias)";
        case JABAS_ERR_STATE: return "rendezvous: bucket handed over twice by one VSW in a step, or described again in the middle of a step";
        default: return "unknown status";
    }
}

JABAS_API int jabas_step_scalars_encode(const JabasStepArgs* args, void* host_block, size_t block_bytes) {
    static_assert(sizeof(StepScal) % 16 == 0, "the block is copied and read in 16-byte pieces");
    if (!args || !host_block) return JABAS_ERR_NULL;
    if (block_bytes < sizeof(StepScal)) return JABAS_ERR_SIZE;
    StepScal sc;
    const int rc = fill_step_scal(args, &sc);
    if (rc != JABAS_OK) return rc;
    if (opt_class_of(args->opt_kind) == 0 || opt_class_of(args->opt_kind) == 3) return JABAS_ERR_OPT;
    memcpy(host_block, &sc, sizeof(sc));
    return JABAS_OK;
}

namespace {
// One wave writes a step-scalar block that arrives by value in the kernel arguments: the refresh of the block
// stays on the compute queue, in stream order with the launches that read it (a host-to-device copy would run
// on a copy engine and cost a hand-over between engines before every step).
struct ScalWords { uint32_t v[sizeof(StepScal) / 4]; };
__global__ void __launch_bounds__(64) store_scalars_kernel(const ScalWords src, uint32_t* dst) {
    for (uint32_t i = threadIdx.x; i < sizeof(StepScal) / 4; i += 64) dst[i] = src.v[i];
}
}  // namespace

JABAS_API int jabas_step_scalars_upload(const JabasStepArgs* args, void* scalars_dev, jabas_stream_t stream) {
    if (!args || !scalars_dev) return JABAS_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(scalars_dev) % 16) return JABAS_ERR_ALIGN;
    ScalWords words;
    static_assert(sizeof(words) == sizeof(StepScal), "same bytes");
    const int rc = jabas_step_scalars_encode(args, &words, sizeof(words));
    if (rc != JABAS_OK) return rc;
    const hipError_t err = launch_kernel(store_scalars_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                                         words, static_cast<uint32_t*>(scalars_dev));
    return err == hipSuccess ? JABAS_OK : JABAS_ERR_LAUNCH;
}

JABAS_API size_t jabas_sync_workspace_bytes(uint64_t numel, int32_t grad_dtype) {
    // chunks of a single span whose first element may sit anywhere in the line the grid starts at,
    // under the launch shape with the smallest chunks
    (void)grad_dtype;
    const uint64_t chunks = (numel + kWideElems - 1 + kMinChunkElems - 1) / kMinChunkElems;
    return workspace_rows(chunks, 1) * kStatsStride * sizeof(double);
}

namespace {
// Upper bound of the chunks of a plan over these spans, for any K, optimizer and buffer alignment.
uint64_t plan_chunks_bound(const JabasSpan* spans, uint32_t n_span) {
    uint64_t n = 0;
    for (uint32_t i = 0; i < n_span; ++i)
        if (spans[i].numel) n += (spans[i].numel + kWideElems - 1 + kMinChunkElems - 1) / kMinChunkElems;
    return n;
}
size_t table_bytes(uint32_t n_span, uint64_t n_chunks) {
    return align16((static_cast<size_t>(n_span) + 1) * sizeof(uint32_t)) + align16(static_cast<size_t>(n_chunks) * sizeof(ChunkDesc));
}
size_t plan_fixed_bytes(uint32_t n_span, uint32_t n_bounds) {
    return kHeaderBytes + align16(static_cast<size_t>(n_span) * sizeof(SpanDev)) +
           align16(static_cast<size_t>(n_bounds) * sizeof(BoundDev));
}
}  // namespace

JABAS_API size_t jabas_plan_bytes(const JabasSpan* spans, uint32_t n_span, uint32_t n_bounds, int32_t grad_dtype) {
    if (!spans || (grad_dtype != JABAS_F32 && grad_dtype != JABAS_BF16)) return 0;
    // K and the optimizer are not known here: one chunk table per statistics level, of the launch shape with the smallest chunks
    return plan_fixed_bytes(n_span, n_bounds) +
           3 * table_bytes(n_span, plan_chunks_bound(spans, n_span));
}

JABAS_API int jabas_plan_encode(const JabasSpan* spans, uint32_t n_span, const JabasBound* bounds,
                                uint32_t n_bounds, int32_t K, int32_t grad_dtype, int32_t opt_kind,
                                void* host_blob, size_t blob_bytes) {
    static_assert(sizeof(BoundDev) == sizeof(JabasBound), "bound layout");
    if (!spans || !host_blob) return JABAS_ERR_NULL;
    if (n_bounds && !bounds) return JABAS_ERR_NULL;
    if (n_span < 1 || n_span > (1u << 24)) return JABAS_ERR_SIZE;
    if (K < 1 || K > JABAS_MAX_K) return JABAS_ERR_K;
    if (grad_dtype != JABAS_F32 && grad_dtype != JABAS_BF16) return JABAS_ERR_DTYPE;
    if (opt_class_of(opt_kind) < 0) return JABAS_ERR_OPT;
    for (uint32_t i = 0; i < n_span; ++i)
        if (spans[i].numel && !spans[i].grads[0]) return JABAS_ERR_NULL;
    const int oc = opt_class_of(opt_kind);
    PlanHeader h;
    memset(&h, 0, sizeof(h));
    const size_t fixed = plan_fixed_bytes(n_span, n_bounds);
    if (blob_bytes < fixed) return JABAS_ERR_PLAN;
    if (reinterpret_cast<uintptr_t>(host_blob) % 8) return JABAS_ERR_ALIGN;
    h.off_spans = kHeaderBytes;
    h.off_bounds = h.off_spans + align16(static_cast<size_t>(n_span) * sizeof(SpanDev));
    h.magic = kPlanMagic;
    h.version = kPlanVersion;
    h.n_span = n_span;
    h.n_bounds = n_bounds;
    h.K = K;
    h.grad_dtype = grad_dtype;
    h.opt_kind = opt_kind;
    h.all_have_s1 = 1;
    for (int v = 0; v < 3; ++v) {
        h.shape[v].block = static_cast<uint32_t>(launch_block(K, grad_dtype, oc, v));
        h.shape[v].chunk_tiles = static_cast<uint32_t>(launch_chunk_tiles(K, grad_dtype, oc, v));
    }

    // spans first: where a span's element grid starts (and so how many chunks it has) depends on
    // the alignment of all its buffers
    char* base = static_cast<char*>(host_blob);
    memset(base, 0, fixed);
    SpanDev* sd = reinterpret_cast<SpanDev*>(base + h.off_spans);
    for (uint32_t i = 0; i < n_span; ++i) {
        uint32_t tiles = 0;
        int rc = encode_span(spans[i], K, grad_dtype, opt_kind, static_cast<int>(h.shape[0].block), &sd[i], &tiles);
        if (rc != JABAS_OK) return rc;
        rc = check_bounds_host(spans[i], bounds, n_bounds, &h.max_group);
        if (rc != JABAS_OK) return rc;
        if (spans[i].numel && !spans[i].state1) h.all_have_s1 = 0;
    }
    size_t cursor = fixed;
    int table_of[3];                             // level -> the level whose table it uses (itself when it owns one)
    for (int v = 0; v < 3; ++v) {
        PlanShape& ps = h.shape[v];
        table_of[v] = v;
        for (int u = 0; u < v; ++u)
            if (h.shape[u].block == ps.block && h.shape[u].chunk_tiles == ps.chunk_tiles) { table_of[v] = table_of[u]; break; }
        if (table_of[v] != v) continue;          // same shape: one table serves both kinds of launch
        uint64_t n_chunks = 0;
        for (uint32_t i = 0; i < n_span; ++i) {
            const uint64_t tiles = tiles_of(sd[i].hi, static_cast<int>(ps.block));
            if (tiles > 0x7fffffffull) return JABAS_ERR_SIZE;
            n_chunks += chunks_of_tiles(tiles, ps.chunk_tiles);
        }
        if (n_chunks > 0x7fffffffull) return JABAS_ERR_SIZE;
        ps.n_chunks = static_cast<uint32_t>(n_chunks);
        ps.off_prefix = cursor;
        ps.off_chunks = cursor + align16((static_cast<size_t>(n_span) + 1) * sizeof(uint32_t));
        cursor += table_bytes(n_span, n_chunks);
    }
    const size_t need = cursor;
    if (blob_bytes < need) return JABAS_ERR_PLAN;
    memset(base + fixed, 0, need - fixed);
    h.total_bytes = need;
    for (int v = 0; v < 3; ++v) {
        if (table_of[v] != v) continue;
        PlanShape& ps = h.shape[v];
        uint32_t* prefix = reinterpret_cast<uint32_t*>(base + ps.off_prefix);
        ChunkDesc* cd = reinterpret_cast<ChunkDesc*>(base + ps.off_chunks);
        const uint64_t te = tile_elems_of(static_cast<int>(ps.block));
        const uint32_t ct = ps.chunk_tiles;
        uint32_t c = 0;
        for (uint32_t i = 0; i < n_span; ++i) {
            const uint32_t tiles = static_cast<uint32_t>(tiles_of(sd[i].hi, static_cast<int>(ps.block)));
            prefix[i] = c;
            const uint32_t span_chunks = static_cast<uint32_t>(chunks_of_tiles(tiles, ct));
            if (span_chunks > ps.max_span_chunks) ps.max_span_chunks = span_chunks;
            uint32_t j = 0;
            for (uint32_t t0 = 0; t0 < tiles; t0 += ct, ++c) {
                cd[c].span = i;
                cd[c].tile0 = t0;
                if (spans[i].bound_count) {       // bound entry covering the chunk's first live element
                    const uint64_t e0 = static_cast<uint64_t>(t0) * te;
                    const uint64_t rel = (e0 > sd[i].lo ? e0 : sd[i].lo) - sd[i].lo;
                    const JabasBound* b = bounds + spans[i].bound_begin;
                    while (j + 1 < spans[i].bound_count && b[j + 1].start <= rel) ++j;
                }
                cd[c].bound0 = j;
            }
        }
        prefix[n_span] = c;
        if (c != ps.n_chunks) return JABAS_ERR_PLAN;
    }
    for (int v = 0; v < 3; ++v)
        if (table_of[v] != v) h.shape[v] = h.shape[table_of[v]];
    if (n_bounds) memcpy(base + h.off_bounds, bounds, static_cast<size_t>(n_bounds) * sizeof(JabasBound));
    memcpy(base, &h, sizeof(h));
    return JABAS_OK;
}

namespace {
bool read_plan_header(const void* host_blob, PlanHeader* h) {
    memcpy(h, host_blob, sizeof(*h));
    return h->magic == kPlanMagic && h->version == kPlanVersion;
}
}  // namespace

JABAS_API int64_t jabas_plan_chunks(const void* host_blob, int32_t stats) {
    if (!host_blob) return JABAS_ERR_NULL;
    PlanHeader h;
    if (!read_plan_header(host_blob, &h)) return JABAS_ERR_PLAN;
    if (stats < JABAS_STATS_NONE || stats > JABAS_STATS_GRAM) return JABAS_ERR_OPT;
    return h.shape[shape_level(stats)].n_chunks;
}

JABAS_API size_t jabas_plan_workspace_bytes(const void* host_blob) {
    if (!host_blob) return 0;
    PlanHeader h;
    if (!read_plan_header(host_blob, &h)) return 0;
    const uint32_t rows = h.shape[1].n_chunks > h.shape[2].n_chunks ? h.shape[1].n_chunks : h.shape[2].n_chunks;
    return workspace_rows(rows, h.n_span) * kStatsStride * sizeof(double);
}

JABAS_API int jabas_sync_fused(const void* plan_host, const void* plan_dev, const JabasStepArgs* args,
                               double* stats_out, void* workspace, size_t workspace_bytes,
                               jabas_stream_t stream) {
    if (!plan_host || !plan_dev || !args) return JABAS_ERR_NULL;
    PlanHeader h;
    memcpy(&h, plan_host, sizeof(h));
    if (h.magic != kPlanMagic || h.version != kPlanVersion) return JABAS_ERR_PLAN;
    if (reinterpret_cast<uintptr_t>(plan_dev) % 16) return JABAS_ERR_ALIGN;
    KArgs a;
    int rc = fill_kargs(args, &a);
    if (rc != JABAS_OK) return rc;
    if (args->K != h.K || args->grad_dtype != h.grad_dtype) return JABAS_ERR_PLAN;
    const int oc = opt_class_of(args->opt_kind);
    // the chunk tables are cut for the launch shapes of (K, dtype, optimizer class), and the state pointers
    // were validated for that class only
    if (opt_class_of(h.opt_kind) != oc) return JABAS_ERR_PLAN;
    const int stats = args->stats;
    const PlanShape& ps = h.shape[shape_level(stats)];
    if (ps.block != static_cast<uint32_t>(launch_block(h.K, h.grad_dtype, oc, stats)) ||
        ps.chunk_tiles != static_cast<uint32_t>(launch_chunk_tiles(h.K, h.grad_dtype, oc, stats)))
        return JABAS_ERR_PLAN;
    if (oc != 0) {
        if (h.max_group >= static_cast<uint32_t>(args->n_groups)) return JABAS_ERR_GROUP;
        if (oc == 1 && args->momentum != 0.0 && !h.all_have_s1) return JABAS_ERR_NULL;
    }
    const char* dev = static_cast<const char*>(plan_dev);
    a.spans = reinterpret_cast<const SpanDev*>(dev + h.off_spans);
    a.chunk_prefix = reinterpret_cast<const uint32_t*>(dev + ps.off_prefix);
    a.chunks = reinterpret_cast<const ChunkDesc*>(dev + ps.off_chunks);
    a.bounds = h.n_bounds ? reinterpret_cast<const BoundDev*>(dev + h.off_bounds) : nullptr;
    a.n_span = h.n_span;
    a.n_chunks = ps.n_chunks;
    a.chunk_tiles = ps.chunk_tiles;
    a.use_inline = 0;
    return run_fused(a, args, ps.max_span_chunks, stats_out, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

JABAS_API int jabas_sync_bucket(const JabasSpan* span, const JabasBound* bounds_dev, const JabasStepArgs* args,
                                double* stats_out, void* workspace, size_t workspace_bytes,
                                jabas_stream_t stream) {
    if (!span || !args) return JABAS_ERR_NULL;
    KArgs a;
    int rc = fill_kargs(args, &a);
    if (rc != JABAS_OK) return rc;
    uint32_t tiles = 0;
    const int oc = opt_class_of(args->opt_kind);
    const int stats = args->stats;
    rc = encode_span(*span, args->K, args->grad_dtype, args->opt_kind,
                     launch_block(args->K, args->grad_dtype, oc, stats), &a.span0, &tiles);
    if (rc != JABAS_OK) return rc;
    if (oc == 1 && args->momentum != 0.0 && !span->state1) return JABAS_ERR_NULL;
    if (span->bound_count && !bounds_dev) return JABAS_ERR_NULL;
    // bounds_dev is indexed from its own start: the span's entries begin at element 0 of it
    a.span0.bound_begin = 0;
    a.bounds = reinterpret_cast<const BoundDev*>(bounds_dev);
    a.spans = nullptr;
    a.chunks = nullptr;
    a.chunk_prefix = nullptr;
    a.n_span = 1;
    a.chunk_tiles = launch_chunk_tiles(args->K, args->grad_dtype, oc, stats);
    a.n_chunks = static_cast<uint32_t>(chunks_of_tiles(tiles, a.chunk_tiles));
    a.use_inline = 1;
    return run_fused(a, args, a.n_chunks, stats_out, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

// --- the entry point that allocates nothing -------------------------------------------------
// The partial rows of the statistics reduction live in a file-scope device array instead of a
// caller-provided workspace. Every GPU the library runs on holds its own copy of the array at its
// own address until the process ends; the address is looked up once per device, on the first call
// made with that device current.
namespace {
constexpr uint64_t kStaticMaxNumel = JABAS_STATIC_MAX_NUMEL;
constexpr uint64_t kStaticMinChunkElems = kMinStatsChunkElems;    // one partial row per chunk of a statistics launch
constexpr int kStaticRowDoubles = 4 + JABAS_MAX_K;            // the widest rows it serves: full rows of 16 VSWs
constexpr size_t kStaticScratchBytes =
    workspace_rows((kStaticMaxNumel + kWideElems - 1 + kStaticMinChunkElems - 1) / kStaticMinChunkElems, 1) *
    kStaticRowDoubles * sizeof(double);
static_assert(kStaticScratchBytes <= (6u << 20), "static scratch stays modest");
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
namespace {
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of this GPU's copy of `scratch`. In host code the array's name is only a handle for
// the runtime, never an address a kernel could use.
int static_scratch(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return JABAS_ERR_LAUNCH;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return JABAS_ERR_LAUNCH;
        g_scratch_ptr[dev].store(p, std::memory_order_release);     // racing first calls look up the same address
    }
    *out = p;
    return JABAS_OK;
}
}  // namespace

JABAS_API int jabas_sync_bucket_static(const JabasSpan* span, const JabasBound* bounds_dev, const JabasStepArgs* args,
                                       double* stats_out, jabas_stream_t stream) {
    if (!span || !args) return JABAS_ERR_NULL;
    if (span->numel > kStaticMaxNumel) return JABAS_ERR_SIZE;
    void* ws = nullptr;
    if (args->stats) {
        if (args->K >= 1 && args->K <= JABAS_MAX_K && args->stats <= JABAS_STATS_GRAM &&
            stats_row_width(args->K, args->stats) > kStaticRowDoubles)
            return JABAS_ERR_SIZE;                    // pair products of more than five VSWs: rows wider than the array holds
        const int rc = static_scratch(&ws);
        if (rc != JABAS_OK) return rc;
    }
    // Every partial row the finalize launches read is written by this call's own launches first, so
    // nothing has to be cleared between calls.
    return jabas_sync_bucket(span, bounds_dev, args, stats_out, ws, ws ? kStaticScratchBytes : 0, stream);
}

JABAS_API int jabas_aggregate(const void* const* grads, int32_t K, int32_t grad_dtype, const float* weight,
                              float* out, uint64_t numel, jabas_stream_t stream) {
    if (!grads || !weight || !out) return JABAS_ERR_NULL;
    if (K < 1 || K > JABAS_MAX_K) return JABAS_ERR_K;
    JabasSpan sp;
    memset(&sp, 0, sizeof(sp));
    JabasStepArgs s;
    memset(&s, 0, sizeof(s));
    for (int k = 0; k < K; ++k) { sp.grads[k] = grads[k]; s.weight[k] = weight[k]; }
    sp.agg_out = out;
    sp.numel = numel;
    s.K = K;
    s.grad_dtype = grad_dtype;
    s.opt_kind = JABAS_OPT_NONE;
    return jabas_sync_bucket(&sp, nullptr, &s, nullptr, nullptr, 0, stream);
}

JABAS_API int jabas_stats(const void* const* grads, int32_t K, int32_t grad_dtype, const float* weight,
                          const uint8_t* half_id, const float* half_weight, uint64_t numel, double* stats_out,
                          void* workspace, size_t workspace_bytes, jabas_stream_t stream) {
    if (!grads || !weight || !half_id || !half_weight || !stats_out) return JABAS_ERR_NULL;
    if (K < 1 || K > JABAS_MAX_K) return JABAS_ERR_K;
    JabasSpan sp;
    memset(&sp, 0, sizeof(sp));
    JabasStepArgs s;
    memset(&s, 0, sizeof(s));
    for (int k = 0; k < K; ++k) {
        sp.grads[k] = grads[k];
        s.weight[k] = weight[k];
        s.half_id[k] = half_id[k];
        s.half_weight[k] = half_weight[k];
    }
    sp.numel = numel;
    s.K = K;
    s.grad_dtype = grad_dtype;
    s.stats = 1;
    s.opt_kind = JABAS_OPT_NONE;
    return jabas_sync_bucket(&sp, nullptr, &s, stats_out, workspace, workspace_bytes, stream);
}

JABAS_API int jabas_gram(const void* const* grads, int32_t K, int32_t grad_dtype, uint64_t numel,
                         double* gram_out, void* workspace, size_t workspace_bytes, jabas_stream_t stream) {
    if (!grads || !gram_out) return JABAS_ERR_NULL;
    if (K < 1 || K > JABAS_GRAM_MAX_K) return JABAS_ERR_K;
    if (grad_dtype != JABAS_F32 && grad_dtype != JABAS_BF16) return JABAS_ERR_DTYPE;
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 8) return JABAS_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(gram_out) % 8) return JABAS_ERR_ALIGN;
    JabasSpan sp;
    memset(&sp, 0, sizeof(sp));
    for (int k = 0; k < K; ++k) sp.grads[k] = grads[k];
    sp.numel = numel;
    SpanDev sd;
    uint32_t tiles = 0;
    const int rc = encode_span(sp, K, grad_dtype, JABAS_OPT_NONE, kBlock, &sd, &tiles);
    if (rc != JABAS_OK) return rc;
    uint64_t g = kGramGrid;
    if (g > tiles) g = tiles;
    if (g < 1) g = 1;
    if (workspace_bytes < g * JABAS_GRAM_STRIDE * sizeof(double)) return JABAS_ERR_WORKSPACE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (launch_gram(K, grad_dtype, sd, static_cast<double*>(workspace), static_cast<unsigned>(g), st) != 0)
        return JABAS_ERR_LAUNCH;
    const size_t spare = workspace_bytes / (JABAS_GRAM_STRIDE * sizeof(double)) - g;
    if (launch_gram_finalize(K, grad_dtype, static_cast<double*>(workspace), static_cast<unsigned>(g),
                             static_cast<unsigned>(spare > 0xffffffffu ? 0xffffffffu : spare), gram_out, st) != 0)
        return JABAS_ERR_LAUNCH;
    return JABAS_OK;
}

JABAS_API int jabas_clip_coef(const double* stats_rows, uint32_t n_rows, double max_norm, double eps, float* coef_out,
                              jabas_stream_t stream) {
    if (!stats_rows || !coef_out) return JABAS_ERR_NULL;
    if (n_rows < 1) return JABAS_ERR_SIZE;
    if (!(max_norm > 0.0) || eps < 0.0) return JABAS_ERR_OPT;
    if (reinterpret_cast<uintptr_t>(stats_rows) % 8 || reinterpret_cast<uintptr_t>(coef_out) % 4) return JABAS_ERR_ALIGN;
    const hipError_t err = launch_kernel(clip_coef_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                                         stats_rows, n_rows, max_norm, eps, coef_out);
    return err == hipSuccess ? JABAS_OK : JABAS_ERR_LAUNCH;
}

JABAS_API int jabas_sgd(const float* grad, float* param, float* momentum_buf, uint64_t numel, double lr,
                        double weight_decay, double momentum, double dampening, int32_t nesterov,
                        int32_t first_step, jabas_stream_t stream) {
    if (!grad || !param) return JABAS_ERR_NULL;
    JabasSpan sp;
    memset(&sp, 0, sizeof(sp));
    JabasStepArgs s;
    memset(&s, 0, sizeof(s));
    sp.grads[0] = grad;
    sp.param = param;
    sp.state1 = momentum_buf;
    sp.numel = numel;
    s.K = 1;
    s.grad_dtype = JABAS_F32;
    s.weight[0] = 1.0f;              // g * 1.0f is exact: the "aggregate" is the gradient itself
    s.opt_kind = JABAS_OPT_SGD;
    s.n_groups = 1;
    s.first_step = first_step;
    s.nesterov = nesterov;
    s.momentum = momentum;
    s.dampening = dampening;
    s.groups[0].lr = lr;
    s.groups[0].weight_decay = weight_decay;
    s.groups[0].step = 1;
    return jabas_sync_bucket(&sp, nullptr, &s, nullptr, nullptr, 0, stream);
}

JABAS_API int jabas_adam(const float* grad, float* param, float* exp_avg, float* exp_avg_sq, float* max_exp_avg_sq,
                         uint64_t numel, double lr, double weight_decay, double beta1, double beta2, double eps,
                         int64_t step, int32_t adamw, jabas_stream_t stream) {
    if (!grad || !param || !exp_avg || !exp_avg_sq) return JABAS_ERR_NULL;
    JabasSpan sp;
    memset(&sp, 0, sizeof(sp));
    JabasStepArgs s;
    memset(&s, 0, sizeof(s));
    sp.grads[0] = grad;
    sp.param = param;
    sp.state1 = exp_avg;
    sp.state2 = exp_avg_sq;
    sp.state3 = max_exp_avg_sq;
    sp.numel = numel;
    s.K = 1;
    s.grad_dtype = JABAS_F32;
    s.weight[0] = 1.0f;
    s.opt_kind = max_exp_avg_sq ? (adamw ? JABAS_OPT_ADAMW_AMSGRAD : JABAS_OPT_ADAM_AMSGRAD)
                                : (adamw ? JABAS_OPT_ADAMW : JABAS_OPT_ADAM);
    s.n_groups = 1;
    s.beta1 = beta1;
    s.beta2 = beta2;
    s.eps = eps;
    s.groups[0].lr = lr;
    s.groups[0].weight_decay = weight_decay;
    s.groups[0].step = step;
    return jabas_sync_bucket(&sp, nullptr, &s, nullptr, nullptr, 0, stream);
}
