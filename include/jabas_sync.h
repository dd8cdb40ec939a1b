/*
 * jabas_sync.h -- C ABI of libjabas_sync.so: the per-GPU gradient synchronisation
 * step of IIDP/JABAS on one MI355X (gfx950).
 *
 * One call covers, in a single pass over HBM:
 *   (1) the batch-weighted aggregate of the K virtual-stream-worker (VSW) gradient
 *       buckets,      acc = g_0*w_0; acc = acc + g_k*w_k  (k = 1..K-1),
 *       every product and sum individually rounded to fp32, bf16 inputs widened first;
 *   (2) the per-span gradient statistics used by similarity-based adaptive batching;
 *   (3) the weight update (SGD-momentum, Adam, AdamW) over the flat parameter span,
 *       optionally followed by the fan-out of the new weights to other VSW replicas.
 *
 * Conventions
 *   - plain C types only; every buffer is caller-owned device memory;
 *   - no entry point allocates, frees or synchronises the device; all work is queued
 *     on the stream passed in (jabas_stream_t is a hipStream_t);
 *   - the library keeps no mutable global state (jabas_sync_bucket_static apart, which says
 *     so), so calls from different threads on different streams do not interfere as long
 *     as they use different workspaces; the jabas_rdv_* calls work on a host object the caller
 *     creates (it and its HIP events are the only things the library ever allocates), under
 *     that object's own mutex;
 *   - return value: JABAS_OK (0) or a negative JabasStatus; nothing is launched when a
 *     negative status is returned (except JABAS_ERR_LAUNCH, reported after the fact).
 *     JABAS_ERR_LAUNCH is the return value of this call's own hipLaunchKernel: a HIP
 *     error an earlier call of the thread left unread is neither reported nor cleared;
 *
 * What each entry point stands in for in the reference is cited beside it
 * (paths relative to the JABAS repository).
 */
#ifndef JABAS_SYNC_H
#define JABAS_SYNC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JABAS_MAX_K 16          /* VSWs aggregated by one launch                      */
#define JABAS_MAX_GROUPS 16     /* optimizer parameter groups per launch              */
#define JABAS_STATS_STRIDE 40   /* doubles per span in stats_out: the widest row, 4 + 8 + 28 (GRAM, 8 VSWs) */
#define JABAS_GRAM_MAX_K 16     /* VSWs of one jabas_gram call                        */
#define JABAS_STATS_GRAM_MAX_K 8 /* VSWs of a launch with JABAS_STATS_GRAM             */
#define JABAS_GRAM_STRIDE 256   /* doubles per call in gram_out: JABAS_GRAM_MAX_K squared */
#define JABAS_STATIC_MAX_NUMEL (1ull << 26)  /* largest span of jabas_sync_bucket_static  */
#define JABAS_STEP_SCALARS_BYTES 688         /* size of a step-scalar block (jabas_step_scalars_encode) */

typedef void* jabas_stream_t;   /* hipStream_t */

typedef enum JabasStatus {
    JABAS_OK = 0,
    JABAS_ERR_NULL = -1,        /* a required pointer is NULL                          */
    JABAS_ERR_K = -2,           /* K outside 1..JABAS_MAX_K                            */
    JABAS_ERR_ALIGN = -3,       /* buffers of a span sit at different line positions   */
    JABAS_ERR_DTYPE = -4,       /* grad_dtype is neither JABAS_F32 nor JABAS_BF16      */
    JABAS_ERR_OPT = -5,         /* unknown optimizer kind or inconsistent state ptrs   */
    JABAS_ERR_GROUP = -6,       /* group index / count out of range, unsorted bounds   */
    JABAS_ERR_WORKSPACE = -7,   /* workspace missing or too small                      */
    JABAS_ERR_PLAN = -8,        /* plan blob malformed or too small                    */
    JABAS_ERR_SIZE = -9,        /* numel / span count out of range                     */
    JABAS_ERR_LAUNCH = -10,     /* the HIP runtime refused the launch                  */
    JABAS_ERR_ALIAS = -11,      /* a written buffer overlaps another buffer of the span */
    JABAS_ERR_STATE = -12       /* rendezvous: a VSW handed the same bucket over twice in one step,
                                   or a bucket was described again in the middle of a step */
} JabasStatus;

enum { JABAS_F32 = 0, JABAS_BF16 = 1 };
/* ..._AMSGRAD: Adam / AdamW with amsgrad=True (torch 1.8.1 _functional.adam: max_exp_avg_sq =
 * max(max_exp_avg_sq, exp_avg_sq), the denominator formed from the maximum), as
 * examples/gnmt/seq2seq/train/shard_optimizer.py:58-66,79-90 threads it into F.adam; the span
 * carries the maximum in state3. */
enum { JABAS_OPT_NONE = 0, JABAS_OPT_SGD = 1, JABAS_OPT_ADAM = 2, JABAS_OPT_ADAMW = 3,
       JABAS_OPT_ADAM_AMSGRAD = 4, JABAS_OPT_ADAMW_AMSGRAD = 5 };
/* Statistics level of a launch (JabasStepArgs.stats). SIMILARITY: the four sums the cosine
 * similarity between the halves and global-norm clipping read (slots DOT_AB .. NORM_AGG of a
 * row; the per-VSW slots are written as 0): the reference's adaptive batching consumes nothing
 * else (jabas/train/trainer.py:470-483), and the kernels that skip the K per-VSW norms keep more
 * loads in flight. FULL adds sum g_k^2 of every VSW. GRAM adds, to the full row, the products
 * sum g_a*g_b of every pair of VSWs a < b, i.e. the whole worker x worker Gram matrix from the
 * pass that aggregates and updates, with no byte read a second time; K <= JABAS_STATS_GRAM_MAX_K
 * (JABAS_ERR_K beyond: the K*(K-1)/2 extra sums per thread, fp64 for fp32 gradients and fp32
 * for bf16 ones, fit the registers of the fused kernel up to there; more workers use jabas_gram,
 * a pass of its own over the gradients). */
enum { JABAS_STATS_NONE = 0, JABAS_STATS_FULL = 1, JABAS_STATS_SIMILARITY = 2, JABAS_STATS_GRAM = 3 };

/* Slots of one stats_out row (JABAS_STATS_STRIDE doubles per span). A = VSWs with
 * half_id 0, B = VSWs with half_id 1; g_A = sum_{k in A} g_k*half_weight_k formed in
 * fp32 in increasing k (same rounding rule as the aggregate), g_B likewise. Products
 * and sums of the statistics themselves are fp64. */
enum {
    JABAS_STAT_DOT_AB = 0,      /* sum g_A * g_B                                       */
    JABAS_STAT_NORM_A = 1,      /* sum g_A^2                                           */
    JABAS_STAT_NORM_B = 2,      /* sum g_B^2                                           */
    JABAS_STAT_NORM_AGG = 3,    /* sum gbar^2 of the aggregate                         */
    JABAS_STAT_NORM_VSW0 = 4    /* + k: sum g_k^2 of VSW k                             */
};
/* JABAS_STATS_GRAM: slot of sum g_a*g_b, a < b < K (pairs in the order (0,1), (0,2), ..., (K-2,K-1),
 * after the K norms); the diagonal of the Gram matrix is the norms. */
#define JABAS_STAT_PAIR(K, a, b) (JABAS_STAT_NORM_VSW0 + (K) + (a) * (2 * (K) - (a) - 1) / 2 + ((b) - (a) - 1))

/* One contiguous stretch of the flat layout. All buffers hold `numel` elements and are
 * indexed alike. Element e of every fp32 buffer must fall at the same position of a
 * 16-byte line, and of every bf16 gradient buffer at the same position of an 8-byte line
 * ((address / element size) mod 4 equal for all buffers), which holds whenever they are
 * views at one element offset into 16-byte aligned arenas. That much is required
 * (JABAS_ERR_ALIGN otherwise). Spans run fastest when the same holds within 64 elements
 * ((address / element size) mod 64 equal for all buffers: views at one element offset into
 * 256-byte aligned arenas, which allocators of device memory give): the launch then starts its
 * element grid at that 256-byte line and moves whole cache lines; spans that start at arbitrary
 * elements lose 8-17 % of the rate without it.
 * agg_out may be exactly one of the fp32 gradient buffers (in-place bucket update); apart
 * from that every written buffer (agg_out, param, state1, state2, state3, fanout) must be disjoint
 * from every other buffer of the span, else JABAS_ERR_ALIAS. Overlap between different
 * spans of one plan is the caller's responsibility. Unused pointers are NULL.
 *
 * Interleaved moments (state_block_log2 != 0; Adam kinds only, JABAS_ERR_OPT otherwise): Adam's moments are
 * state only the optimizer touches, so where they live in HBM is this library's to choose, and one arena
 * that alternates blocks of T = 2^state_block_log2 elements of exp_avg and of exp_avg_sq (then of
 * max_exp_avg_sq for the ..._AMSGRAD kinds), [T of exp_avg][T of exp_avg_sq]..., streams 2-6 % faster than two
 * (three) arrays of their own (measured with T = 8192 and 16384, 32 and 64 KiB blocks, on the K = 4 fp32 and
 * K = 8 bf16 AdamW kernels): a workgroup's reads and writes of the moments then fall next to each other in
 * memory instead of at unrelated addresses. The span names its place in such an arena: state1 = address of
 * its first element's exp_avg, state_block_pos = that element's position inside its block (< T), state2 ==
 * state1 + T floats, state3 == state1 + 2 T floats (amsgrad), and state1 - 4 * state_block_pos, the start of
 * the block group, a multiple of 16 bytes (JABAS_ERR_ALIGN otherwise; a multiple of 256 for the fast element
 * grid). T from 2^8 to 2^24. Element i of the span has its exp_avg at float index
 * t + (ways - 1) * (t - t mod T), t = state_block_pos + i, from the start of the block group, ways = 2 or 3.
 * The alias rule treats everything from state1 to the last element's last moment as one written buffer.
 * No reference counterpart (torch keeps one tensor per parameter and moment,
 * examples/gnmt/seq2seq/train/shard_optimizer.py:50-66). */
typedef struct JabasSpan {
    const void* grads[JABAS_MAX_K];     /* K gradient buffers (fp32 or bf16)           */
    float*      agg_out;                /* aggregated fp32 gradient, or NULL           */
    float*      param;                  /* fp32 weights (optimizer kinds other than NONE) */
    float*      state1;                 /* SGD momentum buffer / Adam exp_avg          */
    float*      state2;                 /* Adam exp_avg_sq                             */
    float*      state3;                 /* Adam max_exp_avg_sq (the ..._AMSGRAD kinds only) */
    float*      fanout[JABAS_MAX_K - 1];/* replicas that receive the updated weights   */
    uint64_t    numel;
    uint32_t    n_fanout;
    uint32_t    bound_begin;            /* first entry of this span in the bounds table*/
    uint32_t    bound_count;            /* 0: the whole span is parameter group 0      */
    uint32_t    state_block_log2;       /* 0: state1/2/3 are arrays of their own; else interleaved moments */
    uint32_t    state_block_pos;        /* interleaved moments: position of the first element in its block */
    uint32_t    reserved;
} JabasSpan;

/* Parameter-group change inside a span: elements [start, next start) use `group`.
 * The first bound of a span has start 0; starts are strictly increasing. */
typedef struct JabasBound {
    uint64_t start;
    uint32_t group;
    uint32_t reserved;
} JabasBound;

/* Hyper-parameters of one parameter group, as the Python optimizer holds them
 * (doubles). `step` is the 1-based Adam step count of this call. */
typedef struct JabasGroup {
    double  lr;
    double  weight_decay;
    int64_t step;
} JabasGroup;

typedef struct JabasStepArgs {
    int32_t K;
    int32_t grad_dtype;                 /* JABAS_F32 / JABAS_BF16                      */
    float   weight[JABAS_MAX_K];        /* w_k = fp32(b_k / B); with A micro-batches summed
                                           into every bucket, fp32(b_k / (B*A))         */
    int32_t stats;                      /* JABAS_STATS_*: none / full row / similarity sums */
    uint8_t half_id[JABAS_MAX_K];       /* 0 = half A, 1 = half B                      */
    float   half_weight[JABAS_MAX_K];   /* fp32(b_k / sum of b over k's half)          */
    int32_t opt_kind;                   /* JABAS_OPT_*                                 */
    int32_t n_groups;
    int32_t first_step;                 /* SGD: momentum buffer not initialised yet    */
    int32_t nesterov;
    double  momentum, dampening;        /* SGD                                         */
    double  beta1, beta2, eps;          /* Adam / AdamW                                */
    JabasGroup groups[JABAS_MAX_GROUPS];
    const float* grad_scale;            /* device scalar c or NULL: when c < 1 the aggregate
                                           is multiplied by c (one fp32 product) before it is
                                           written and handed to the optimizer (clipping)  */
    const void* scalars_dev;            /* NULL, or a device block of JABAS_STEP_SCALARS_BYTES bytes,
                                           16-byte aligned, written by jabas_step_scalars_encode: the
                                           launch then reads weight, half_id, half_weight, first_step,
                                           nesterov, momentum, dampening, beta1, beta2, eps and the
                                           groups' lr, weight_decay and step from the block as it is
                                           when the kernel runs, not from this struct (which must
                                           still be filled in: it is what the call is checked
                                           against). SGD, ADAM and ADAMW only.                  */
} JabasStepArgs;

/* Library identification. No reference counterpart. */
const char* jabas_sync_version(void);
const char* jabas_status_string(int status);

/* The per-step scalars of `args` as the kernels read them (fp32 constants derived in double and
 * rounded once, exactly as a call without a block derives them), written to host_block
 * (JABAS_STEP_SCALARS_BYTES bytes). Pure host code. The caller moves the bytes to the device block
 * that JabasStepArgs.scalars_dev names, in stream order before the launch that reads them. What it
 * is for: a step recorded in a HIP graph has every by-value argument baked in, so an Adam step
 * (bias correction moves with the step count), an SGD step under a learning-rate schedule or under
 * the adaptive-batching LR modifier (jabas/train/trainer.py:693-700) could not be replayed; with
 * the scalars in a device block the recorded launch stays valid and only the block is refreshed
 * (a copy from pinned host memory recorded in the same graph, or a copy queued before the replay).
 * K, grad_dtype, stats, opt_kind and n_groups of the recorded call stay what they were; a block
 * encoded from arguments with another K or optimizer kind is the caller's error, unchecked. The
 * Adam / AdamW flag is part of the block. No reference counterpart. */
int jabas_step_scalars_encode(const JabasStepArgs* args, void* host_block, size_t block_bytes);

/* Encodes `args` and queues, on `stream`, a one-wave kernel that writes the bytes to the device block
 * scalars_dev (JABAS_STEP_SCALARS_BYTES bytes, 16-byte aligned): the refresh ahead of a replay, in stream
 * order with the launches that read the block, without pinned host memory and without a copy engine in
 * between. Only a kernel launch: may itself be recorded (its bytes are then baked in, which is what a
 * recording wants for launches whose scalars never move). No reference counterpart. */
int jabas_step_scalars_upload(const JabasStepArgs* args, void* scalars_dev, jabas_stream_t stream);

/* Bytes of device workspace a single-span call (jabas_sync_bucket, jabas_stats) over
 * numel elements needs when statistics are requested: one partial row per workgroup of
 * the two-level reduction. No reference counterpart. */
size_t jabas_sync_workspace_bytes(uint64_t numel, int32_t grad_dtype);

/* --- multi-span plan --------------------------------------------------------------
 * A plan is the launch-invariant description of a set of spans (pointer table, tile
 * chunk table, group bounds). jabas_plan_encode validates the spans and writes the
 * blob into host memory; the caller copies the same bytes to the device once and
 * passes both copies to jabas_sync_fused at every step. Pure host code: runs without
 * a GPU. The chunk tables are cut for the launch shapes of (K, grad_dtype, optimizer
 * class of opt_kind: none / SGD / Adam+AdamW), so a plan serves launches of exactly
 * that K, dtype and class (statistics on or off, any step, any learning rate);
 * anything else is JABAS_ERR_PLAN. jabas_plan_bytes is an upper bound over all
 * launch shapes; the blob (device copy 16-byte aligned) may be larger than used.
 * Stands in for the per-tensor Python loops that walk buckets and parameters at every
 * step in the reference: jabas/train/trainer.py:327-337 (hook registration per local
 * model), examples/gnmt/seq2seq/train/shard_optimizer.py:40-73 (per-parameter loop
 * matching gradients to parameters by .index). */
size_t jabas_plan_bytes(const JabasSpan* spans, uint32_t n_span, uint32_t n_bounds,
                        int32_t grad_dtype);
int jabas_plan_encode(const JabasSpan* spans, uint32_t n_span,
                      const JabasBound* bounds, uint32_t n_bounds,
                      int32_t K, int32_t grad_dtype, int32_t opt_kind,
                      void* host_blob, size_t blob_bytes);
/* Number of workgroups (chunks) one launch of the plan uses at statistics level `stats`
 * (JABAS_STATS_*): the levels may run different workgroup shapes, the plan holds a chunk
 * table for each shape. Negative JabasStatus on a malformed blob or an unknown level. */
int64_t jabas_plan_chunks(const void* host_blob, int32_t stats);
/* Bytes of device workspace jabas_sync_fused needs for this plan when statistics are
 * requested (0 on a malformed blob). */
size_t jabas_plan_workspace_bytes(const void* host_blob);

/* --- the fused sync step ------------------------------------------------------------
 * Aggregate + statistics + optimizer (+ fan-out) over every span of a plan, one
 * launch (plus a one-workgroup-per-span finalize launch when args->stats is set).
 * stats_out: n_span * JABAS_STATS_STRIDE doubles (device), required when stats != 0.
 * A launch with statistics takes a plan of at most 65535 spans (JABAS_ERR_SIZE beyond,
 * returned before anything is launched); without statistics up to 2^24.
 * Replaces, for one GPU:
 *   - the local aggregation of the K VSW buckets inside IIDPTrainer.compute()/step()
 *     and iidp_allreduce_hook's division by the worker count
 *     (call sites jabas/ddp_comm_hooks/similarity_allreduce.py:42,
 *      jabas/train/trainer.py:452-468, 594-599);
 *   - clone + sub-group sum + div_ of subgroup_allreduce_hook
 *     (jabas/ddp_comm_hooks/similarity_allreduce.py:20-35) and the cat + reductions of
 *     _compute_cosine_similarity (jabas/train/trainer.py:470-483);
 *   - torch.optim.SGD / Adam / AdamW and iidp.optim.ShardSGD / ShardAdam / ShardAdamW
 *     .step() (examples/resnet50/main.py:351-359, examples/vit/main.py:425-437,
 *      examples/gnmt/seq2seq/train/shard_optimizer.py:30-90);
 *   - the weight copy main VSW -> other VSWs (jabas/train/trainer.py:530-534). */
int jabas_sync_fused(const void* plan_host, const void* plan_dev,
                     const JabasStepArgs* args, double* stats_out,
                     void* workspace, size_t workspace_bytes, jabas_stream_t stream);

/* The same step over ONE span passed by value (no plan, no device table): what a
 * comm hook calls for the bucket it was handed. bounds_dev is a device array holding
 * the span's bound_count entries (span->bound_begin is ignored), or NULL when
 * bound_count == 0; its contents cannot be checked on the host and must obey the
 * JabasBound rules. stats_out: JABAS_STATS_STRIDE doubles or NULL.
 * Replaces hook_with_allreduce for one bucket
 * (jabas/ddp_comm_hooks/similarity_allreduce.py:38-45) and, with an optimizer kind,
 * the optimizer hook of the overlap weight-sync mode (jabas/train/trainer.py:327-333). */
int jabas_sync_bucket(const JabasSpan* span, const JabasBound* bounds_dev,
                      const JabasStepArgs* args, double* stats_out,
                      void* workspace, size_t workspace_bytes, jabas_stream_t stream);

/* jabas_sync_bucket without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc) and so cannot size a workspace for whatever bucket comes next. No counterpart
 * in the reference. The partial rows of the statistics reduction go to a static device
 * array of 5.25 MB that every GPU the process uses holds until the process ends; its
 * address is looked up once per GPU, on the first call with statistics made with that GPU
 * current (the stream must belong to the current device; make that one call outside any
 * graph capture: the lookup, like the first launch out of a code object, loads device code).
 * Calls neither allocate nor free anything.
 * span->numel above JABAS_STATIC_MAX_NUMEL (64 Mi elements, a 256 MB fp32 bucket) is refused
 * with JABAS_ERR_SIZE before anything is launched, and so is JABAS_STATS_GRAM with more than
 * five VSWs (rows of more than 4 + JABAS_MAX_K sums, wider than the array is sized for). All calls on one GPU share that GPU's
 * array: calls with statistics that overlap in time on one GPU (different streams or
 * threads) race on it and must be serialised by the caller; calls without statistics do
 * not touch it. Results are those of jabas_sync_bucket, bit for bit. */
int jabas_sync_bucket_static(const JabasSpan* span, const JabasBound* bounds_dev,
                             const JabasStepArgs* args, double* stats_out,
                             jabas_stream_t stream);

/* --- single-purpose entry points (thin fronts over the same kernels) ---------------- */

/* out = sum_k w_k g_k in the canonical order. out may alias grads[0] (fp32).
 * Local VSW aggregation only (jabas/train/trainer.py:452-468, 594-599). */
int jabas_aggregate(const void* const* grads, int32_t K, int32_t grad_dtype,
                    const float* weight, float* out, uint64_t numel,
                    jabas_stream_t stream);

/* Statistics row of one span without touching any output buffer
 * (jabas/ddp_comm_hooks/similarity_allreduce.py:20-35, jabas/train/trainer.py:470-483). */
int jabas_stats(const void* const* grads, int32_t K, int32_t grad_dtype,
                const float* weight, const uint8_t* half_id, const float* half_weight,
                uint64_t numel, double* stats_out,
                void* workspace, size_t workspace_bytes, jabas_stream_t stream);

/* K x K Gram matrix of the worker gradients, gram_out[a*JABAS_GRAM_MAX_K + b] = sum g_a*g_b
 * symmetric, JABAS_GRAM_STRIDE doubles. fp32 gradients, and bf16 gradients of up to 7 workers:
 * exact fp64 products and fp64 sums; bf16 gradients of 8 or more workers: exact fp32 products,
 * fp32 running sums over at most 4096 elements, then fp64 (about 1e-6 of |g_a||g_b|). The order of
 * operations is fixed: the same call gives the same bits. The "between
 * workers" statistics; no reference counterpart beyond the pairwise cosine of
 * jabas/train/trainer.py:478. K <= JABAS_GRAM_MAX_K. workspace: at least
 * 1024 * JABAS_GRAM_STRIDE doubles (one row of partial sums per workgroup); with 32 rows more
 * (1056 * JABAS_GRAM_STRIDE doubles) the rows are summed in two stages, which is faster and, since the
 * order of additions differs, may differ from the one-stage result in the last bits. */
int jabas_gram(const void* const* grads, int32_t K, int32_t grad_dtype,
               uint64_t numel, double* gram_out,
               void* workspace, size_t workspace_bytes, jabas_stream_t stream);

/* Global-norm clipping coefficient from statistics rows (device to device, no host sync):
 *   total = sum over the n_rows rows of slot JABAS_STAT_NORM_AGG (in row order, fp64),
 *   *coef_out = fp32(max_norm / (sqrt(total) + eps)).
 * Feed coef_out to a later call as JabasStepArgs.grad_scale: the gradient is scaled only
 * when the coefficient is below 1, as torch.nn.utils.clip_grad_norm_ does
 * (examples/gnmt/seq2seq/train/trainer.py:157-161; clip_grad_norm_for_overlap in
 * examples/gnmt/seq2seq/train/shard_optimizer.py:75-76). eps is 1e-6 there. */
int jabas_clip_coef(const double* stats_rows, uint32_t n_rows, double max_norm, double eps,
                    float* coef_out, jabas_stream_t stream);

/* SGD step with a ready fp32 gradient (torch 1.8.1 optim/_functional.sgd as used by
 * examples/resnet50/main.py:351-359, examples/faster_r_cnn/train.py:266-276).
 * momentum_buf may be NULL when momentum == 0. */
int jabas_sgd(const float* grad, float* param, float* momentum_buf, uint64_t numel,
              double lr, double weight_decay, double momentum, double dampening,
              int32_t nesterov, int32_t first_step, jabas_stream_t stream);

/* Adam (adamw == 0) / AdamW (adamw != 0) step with a ready fp32 gradient
 * (torch 1.8.1 optim/_functional.adam / adamw as called by
 * examples/gnmt/seq2seq/train/shard_optimizer.py:78-90, examples/vit/main.py:425-437).
 * max_exp_avg_sq: NULL, or the running maximum of the second moment (amsgrad=True). */
int jabas_adam(const float* grad, float* param, float* exp_avg, float* exp_avg_sq,
               float* max_exp_avg_sq, uint64_t numel, double lr, double weight_decay,
               double beta1, double beta2, double eps, int64_t step, int32_t adamw,
               jabas_stream_t stream);

/* ---- Rendezvous of the K VSW comm hooks of one GPU --------------------------------------------
 * In IIDP each VSW has its own DDP reducer, thread and stream, only VSW 0's hook communicates and
 * the others register dummy_hook (jabas/train/trainer.py:452-468, 494-514); where the K hooks of a
 * GPU meet is Python inside IIDP (absent from the JABAS repository), so these calls have no
 * counterpart there: they are the native form of that meeting point for buckets that are handed over
 * with the same buffers step after step. A hook's hand-over is one call (an event on its stream, a
 * counter under the object's mutex); the call that completes a bucket queues, on launch_stream, a wait
 * for every VSW's event and the jabas_sync_bucket launch described by jabas_rdv_set_bucket.
 * Thread-safe per object. The caller orders the VSW streams behind the launches at the end of the
 * step (one event on launch_stream) before any VSW hands a bucket over again. */
typedef struct JabasRendezvous JabasRendezvous;

enum {
    JABAS_RDV_WAITING = 0,        /* handed over; other VSWs are still missing              */
    JABAS_RDV_LAUNCHED = 1,       /* this call queued the launch, without statistics          */
    JABAS_RDV_LAUNCHED_ROW0 = 2,  /* ... with statistics into row 0 of the bucket's two rows  */
    JABAS_RDV_LAUNCHED_ROW1 = 3,  /* ... into row 1 (the rows alternate)                      */
    JABAS_RDV_UNKNOWN = 4         /* the bucket is not described: nothing was recorded        */
};

/* K VSWs; the object belongs to the current device (its events are created there). */
int jabas_rdv_create(int32_t K, JabasRendezvous** out);
void jabas_rdv_destroy(JabasRendezvous* r);

/* Describes the launch of bucket `bucket` (everything jabas_sync_bucket takes: the span with the K
 * gradient buffers the VSWs will hand over, the device bound table or NULL); stats_rows: two rows of
 * JABAS_STATS_STRIDE doubles and a workspace of jabas_sync_workspace_bytes, or NULL when the bucket
 * never takes statistics. last_row (0 or 1): the row the bucket's statistics were written to last,
 * by whoever launched it before (0 when nobody did): the launches queued from here go on alternating
 * from there, so a row handed out earlier stays untouched until the second-next statistics launch.
 * The struct is copied; the buffers stay the caller's and must outlive the
 * description. Creates the bucket's K events on first use (the only allocation). */
int jabas_rdv_set_bucket(JabasRendezvous* r, uint32_t bucket, const JabasSpan* span,
                         const JabasBound* bounds_dev, double* stats_rows,
                         void* workspace, size_t workspace_bytes, int32_t last_row);

/* Forgets the description; returns how many VSWs had handed the bucket over in the running step. */
int jabas_rdv_drop_bucket(JabasRendezvous* r, uint32_t bucket);

/* VSW k hands bucket `bucket` over on vsw_stream. want_stats counts from VSW 0 only (its hook knows
 * whether this is a statistics step); args: this step's arguments (args->stats is replaced by
 * stats_level or JABAS_STATS_NONE accordingly). launch_stream: where the launch goes if this
 * hand-over completes the bucket (only the completing call's word is used, so it may differ from
 * call to call: a launch stream of the caller's, VSW 0's stream, or vsw_stream itself to put the
 * launch behind the work of whichever VSW comes last; that VSW then records no event).
 * Returns a JABAS_RDV_* code or a negative JabasStatus (JABAS_ERR_STATE: handed over twice). */
int jabas_rdv_publish(JabasRendezvous* r, int32_t k, uint32_t bucket, int32_t want_stats,
                      jabas_stream_t vsw_stream, jabas_stream_t launch_stream,
                      const JabasStepArgs* args, int32_t stats_level);

/* End of a step or recovery from an error: clears what was handed over and returns the number of
 * buckets that were incomplete (0 after a healthy step). */
int jabas_rdv_reset(JabasRendezvous* r);

#ifdef __cplusplus
}
#endif
#endif /* JABAS_SYNC_H */
