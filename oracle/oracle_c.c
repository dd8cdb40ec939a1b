/*
 * Scalar C restatement of the per-GPU gradient-sync arithmetic. TEST INFRASTRUCTURE:
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it.
 *
 * Written independently of oracle.py (element loops instead of whole-tensor ops) so
 * that the two can be compared bit for bit; build with -ffp-contract=off so that no
 * product/sum pair is fused (see oracle/Makefile). fp32 arithmetic is SSE scalar code
 * on x86-64: no excess precision, IEEE sqrt and division.
 *
 * Reference files followed (JABAS repository):
 *   oc_aggregate*  jabas/train/trainer.py:452-468,594-599;
 *                  jabas/ddp_comm_hooks/similarity_allreduce.py:32
 *   oc_stats       jabas/ddp_comm_hooks/similarity_allreduce.py:20-35;
 *                  jabas/train/trainer.py:427-432,470-483
 *   oc_sgd         torch 1.8.1 optim/_functional.sgd (examples/resnet50/main.py:351-359)
 *   oc_adam        torch 1.8.1 optim/_functional.adam/adamw
 *                  (examples/gnmt/seq2seq/train/shard_optimizer.py:78-90, examples/vit/main.py:425-437)
 * The order of IIDP's own aggregation is not visible in the reference tree (un-vendored
 * submodule): parity of the aggregate order against the reference is unpinned.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static float elem(const void* base, int bf16, size_t i) {
    return bf16 ? bf16_to_f32(((const uint16_t*)base)[i]) : ((const float*)base)[i];
}

/* out[i] = ((g0*w0 + g1*w1) + g2*w2) + ...   every * and + rounded to fp32 */
void oc_aggregate(const void* const* g, int K, int bf16, const float* w, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        float acc = elem(g[0], bf16, i) * w[0];
        for (int k = 1; k < K; ++k) {
            float t = elem(g[k], bf16, i) * w[k];
            acc = acc + t;
        }
        out[i] = acc;
    }
}

/* row[0]=dot(gA,gB) row[1]=|gA|^2 row[2]=|gB|^2 row[3]=|gbar|^2 row[4+k]=|g_k|^2; fp64 sums */
void oc_stats(const void* const* g, int K, int bf16, const float* w, const uint8_t* half, const float* hw,
              size_t n, double* row) {
    for (int i = 0; i < 4 + K; ++i) row[i] = 0.0;      /* the caller's row holds at least 4 + K entries */
    for (size_t i = 0; i < n; ++i) {
        float acc = 0.0f, ga = 0.0f, gb = 0.0f;
        int seen_a = 0, seen_b = 0;
        for (int k = 0; k < K; ++k) {
            float x = elem(g[k], bf16, i);
            float t = x * w[k];
            acc = k ? acc + t : t;
            float th = x * hw[k];
            if (half[k]) { gb = seen_b ? gb + th : th; seen_b = 1; }
            else         { ga = seen_a ? ga + th : th; seen_a = 1; }
            row[4 + k] += (double)x * (double)x;
        }
        row[0] += (double)ga * (double)gb;
        row[1] += (double)ga * (double)ga;
        row[2] += (double)gb * (double)gb;
        row[3] += (double)acc * (double)acc;
    }
}

/* gram[a*K+b] = sum_i g_a[i]*g_b[i] */
void oc_gram(const void* const* g, int K, int bf16, size_t n, double* gram) {
    for (int a = 0; a < K * K; ++a) gram[a] = 0.0;
    for (size_t i = 0; i < n; ++i)
        for (int a = 0; a < K; ++a)
            for (int b = 0; b < K; ++b)
                gram[a * K + b] += (double)elem(g[a], bf16, i) * (double)elem(g[b], bf16, i);
}

/* fp32 scalars are what the Python doubles become inside an fp32 kernel */
void oc_sgd(float* p, const float* g, float* buf, size_t n, float wd, float neg_lr, float momentum,
            float one_minus_damp, int has_momentum, int first_step, int nesterov) {
    for (size_t i = 0; i < n; ++i) {
        float d = g[i];
        if (wd != 0.0f) { float t = p[i] * wd; d = d + t; }
        if (has_momentum) {
            if (first_step) buf[i] = d;
            else { float a = buf[i] * momentum; float b = d * one_minus_damp; buf[i] = a + b; }
            if (nesterov) { float t = buf[i] * momentum; d = d + t; }
            else d = buf[i];
        }
        float s = d * neg_lr;
        p[i] = p[i] + s;
    }
}

/* vmax: NULL, or max_exp_avg_sq of amsgrad (torch.maximum propagates NaN from either side) */
void oc_adam(float* p, const float* g, float* m, float* v, float* vmax, size_t n, float wd, float decay, float beta1,
             float one_minus_beta1, float beta2, float one_minus_beta2, float sqrt_bc2, float eps,
             float neg_step_size, int adamw) {
    for (size_t i = 0; i < n; ++i) {
        float gi = g[i];
        if (adamw) p[i] = p[i] * decay;
        else if (wd != 0.0f) { float t = p[i] * wd; gi = gi + t; }
        float a = m[i] * beta1, b = gi * one_minus_beta1;
        m[i] = a + b;
        float c = v[i] * beta2, e = gi * one_minus_beta2;
        e = e * gi;
        v[i] = c + e;
        float second = v[i];
        if (vmax) {
            float a0 = vmax[i], b0 = v[i];
            vmax[i] = (a0 != a0) ? a0 : ((b0 != b0) ? b0 : (a0 > b0 ? a0 : b0));
            second = vmax[i];
        }
        float denom = sqrtf(second);
        denom = denom / sqrt_bc2;
        denom = denom + eps;
        float num = m[i] * neg_step_size;
        num = num / denom;
        p[i] = p[i] + num;
    }
}
