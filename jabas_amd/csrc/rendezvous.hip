// Native rendezvous of the K VSW comm hooks of one GPU around the fused launch of a bucket.
//
// In IIDP every VSW runs its own DDP reducer on its own thread and stream and only VSW 0's hook
// communicates (jabas/train/trainer.py:452-468); the place where the K hooks of a GPU meet is Python there.
// Here the meeting point of a bucket that is handed over with the same buffers step after step is this
// object: a publish is one foreign call (an event record on the VSW's stream and a counter under a mutex),
// and the call that completes the bucket queues the K event waits and the prepared jabas_sync_bucket launch
// on the launch stream. Host code only: no kernel lives in this file.
#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "jabas_internal.h"

#define JABAS_API extern "C" __attribute__((visibility("default")))

struct JabasRendezvous {
    struct Bucket {
        bool set = false;
        JabasSpan span;
        const JabasBound* bounds_dev = nullptr;
        double* rows = nullptr;                 // two rows of JABAS_STATS_STRIDE doubles, used in turn
        void* workspace = nullptr;
        size_t workspace_bytes = 0;
        hipEvent_t events[JABAS_MAX_K] = {};
        hipStream_t streams[JABAS_MAX_K] = {};
        uint32_t arrived = 0;                   // bit k: VSW k handed its buffer over in this step
        uint32_t recorded = 0;                  // bit k: events[k] was recorded in this step
        int want_stats = 0;                     // VSW 0's word
        int flip = 0;
    };
    std::mutex mu;
    int K = 0;
    int device = 0;
    std::vector<Bucket> buckets;
};

namespace {

constexpr uint32_t kMaxBuckets = 1u << 16;

void destroy_events(JabasRendezvous::Bucket& b) {
    for (auto& e : b.events)
        if (e) {
            (void)hipEventDestroy(e);
            e = nullptr;
        }
}

}  // namespace

JABAS_API int jabas_rdv_create(int32_t K, JabasRendezvous** out) {
    if (!out) return JABAS_ERR_NULL;
    *out = nullptr;
    if (K < 1 || K > JABAS_MAX_K) return JABAS_ERR_K;
    JabasRendezvous* r = new (std::nothrow) JabasRendezvous;
    if (!r) return JABAS_ERR_SIZE;
    r->K = K;
    if (hipGetDevice(&r->device) != hipSuccess) {
        delete r;
        return JABAS_ERR_LAUNCH;
    }
    *out = r;
    return JABAS_OK;
}

JABAS_API void jabas_rdv_destroy(JabasRendezvous* r) {
    if (!r) return;
    for (auto& b : r->buckets) destroy_events(b);
    delete r;
}

JABAS_API int jabas_rdv_set_bucket(JabasRendezvous* r, uint32_t bucket, const JabasSpan* span, const JabasBound* bounds_dev,
                                   double* stats_rows, void* workspace, size_t workspace_bytes, int32_t last_row) {
    if (!r || !span) return JABAS_ERR_NULL;
    if (bucket >= kMaxBuckets || last_row < 0 || last_row > 1) return JABAS_ERR_SIZE;
    if (stats_rows && (!workspace || reinterpret_cast<uintptr_t>(stats_rows) % 8)) return JABAS_ERR_WORKSPACE;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev != r->device) return JABAS_ERR_LAUNCH;   // events belong to a device
    std::lock_guard<std::mutex> lock(r->mu);
    if (r->buckets.size() <= bucket) r->buckets.resize(bucket + 1);
    JabasRendezvous::Bucket& b = r->buckets[bucket];
    if (b.arrived) return JABAS_ERR_STATE;      // in the middle of a step
    for (int k = 0; k < r->K; ++k)
        if (!b.events[k] && hipEventCreateWithFlags(&b.events[k], hipEventDisableTiming) != hipSuccess) {
            destroy_events(b);
            b.set = false;
            return JABAS_ERR_LAUNCH;
        }
    b.span = *span;
    b.bounds_dev = bounds_dev;
    b.rows = stats_rows;
    b.workspace = workspace;
    b.workspace_bytes = workspace_bytes;
    b.recorded = 0;
    b.want_stats = 0;
    b.flip = last_row;                          // the next statistics launch takes the other row
    b.set = true;
    return JABAS_OK;
}

JABAS_API int jabas_rdv_drop_bucket(JabasRendezvous* r, uint32_t bucket) {
    if (!r) return JABAS_ERR_NULL;
    std::lock_guard<std::mutex> lock(r->mu);
    if (bucket >= r->buckets.size() || !r->buckets[bucket].set) return 0;
    JabasRendezvous::Bucket& b = r->buckets[bucket];
    const int arrived = __builtin_popcount(b.arrived);
    b.set = false;
    b.arrived = b.recorded = 0;
    return arrived;
}

JABAS_API int jabas_rdv_publish(JabasRendezvous* r, int32_t k, uint32_t bucket, int32_t want_stats,
                                jabas_stream_t vsw_stream, jabas_stream_t launch_stream, const JabasStepArgs* args,
                                int32_t stats_level) {
    if (!r || !args) return JABAS_ERR_NULL;
    if (k < 0 || k >= r->K || args->K != r->K) return JABAS_ERR_K;
    JabasRendezvous::Bucket snap;               // what the launch needs, copied under the lock (the table may grow)
    uint32_t recorded;
    int want, flip = 0;
    {
        std::lock_guard<std::mutex> lock(r->mu);
        if (bucket >= r->buckets.size() || !r->buckets[bucket].set) return JABAS_RDV_UNKNOWN;
        JabasRendezvous::Bucket* b = &r->buckets[bucket];
        const uint32_t bit = 1u << k;
        if (b->arrived & bit) return JABAS_ERR_STATE;
        hipStream_t mine = static_cast<hipStream_t>(vsw_stream);
        const bool complete = (b->arrived | bit) == (r->K >= 32 ? 0xffffffffu : (1u << r->K) - 1u);
        // The launch goes on the stream the completing hand-over names: only that hand-over knows it (callers
        // may put a bucket's launch on the stream of whichever VSW comes last), so every other one records an
        // event, and the completing one does unless the launch follows its own work on its own stream.
        if (!complete || vsw_stream != launch_stream) {
            if (hipEventRecord(b->events[k], mine) != hipSuccess) return JABAS_ERR_LAUNCH;
            b->recorded |= bit;
        }
        b->streams[k] = mine;
        b->arrived |= bit;
        if (k == 0) b->want_stats = want_stats != 0;
        if (!complete) return JABAS_RDV_WAITING;
        // complete: this call launches. The bucket is free for the next step from here on (its events are
        // waited for below, before any thread can record them again: the VSW streams are held back by the
        // caller's end-of-step event, which is queued after this launch).
        recorded = b->recorded;
        want = b->want_stats && b->rows != nullptr;
        if (want) flip = (b->flip ^= 1);
        snap = *b;
        b->arrived = b->recorded = 0;
        b->want_stats = 0;
    }
    hipStream_t main = static_cast<hipStream_t>(launch_stream);
    for (int j = 0; j < r->K; ++j)
        if ((recorded >> j & 1u) && snap.streams[j] != main)
            if (hipStreamWaitEvent(main, snap.events[j], 0) != hipSuccess) return JABAS_ERR_LAUNCH;
    JabasStepArgs a = *args;
    a.stats = want ? static_cast<uint32_t>(stats_level) : static_cast<uint32_t>(JABAS_STATS_NONE);
    double* row = want ? snap.rows + static_cast<size_t>(flip) * JABAS_STATS_STRIDE : nullptr;
    const int rc = jabas_sync_bucket(&snap.span, snap.bounds_dev, &a, row, want ? snap.workspace : nullptr,
                                     want ? snap.workspace_bytes : 0, launch_stream);
    if (rc != JABAS_OK) return rc;
    return want ? JABAS_RDV_LAUNCHED_ROW0 + flip : JABAS_RDV_LAUNCHED;
}

JABAS_API int jabas_rdv_reset(JabasRendezvous* r) {
    if (!r) return JABAS_ERR_NULL;
    std::lock_guard<std::mutex> lock(r->mu);
    int pending = 0;
    for (auto& b : r->buckets) {
        if (b.arrived) ++pending;
        b.arrived = b.recorded = 0;
        b.want_stats = 0;
    }
    return pending;
}
