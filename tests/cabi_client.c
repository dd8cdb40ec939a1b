/* Plain-C client of libjabas_sync.so: built with gcc by tests/test_cabi_host.py, it prints the layout a C
 * compiler gives the header's structs (compared with the ctypes mirror) and drives the pure-host entry
 * points (version, status strings, plan sizing and encoding). No GPU call is made. */
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "jabas_sync.h"

#define SHOW_SIZE(T) printf("sizeof " #T " %zu\n", sizeof(T))
#define SHOW_OFF(T, f) printf("offsetof " #T "." #f " %zu\n", offsetof(T, f))

int main(void) {
    SHOW_SIZE(JabasSpan);
    SHOW_OFF(JabasSpan, grads);
    SHOW_OFF(JabasSpan, agg_out);
    SHOW_OFF(JabasSpan, param);
    SHOW_OFF(JabasSpan, state1);
    SHOW_OFF(JabasSpan, state2);
    SHOW_OFF(JabasSpan, state3);
    SHOW_OFF(JabasSpan, fanout);
    SHOW_OFF(JabasSpan, numel);
    SHOW_OFF(JabasSpan, n_fanout);
    SHOW_OFF(JabasSpan, bound_begin);
    SHOW_OFF(JabasSpan, bound_count);
    SHOW_OFF(JabasSpan, state_block_log2);
    SHOW_OFF(JabasSpan, state_block_pos);
    SHOW_SIZE(JabasBound);
    SHOW_OFF(JabasBound, start);
    SHOW_OFF(JabasBound, group);
    SHOW_SIZE(JabasGroup);
    SHOW_OFF(JabasGroup, lr);
    SHOW_OFF(JabasGroup, weight_decay);
    SHOW_OFF(JabasGroup, step);
    SHOW_SIZE(JabasStepArgs);
    SHOW_OFF(JabasStepArgs, K);
    SHOW_OFF(JabasStepArgs, grad_dtype);
    SHOW_OFF(JabasStepArgs, weight);
    SHOW_OFF(JabasStepArgs, stats);
    SHOW_OFF(JabasStepArgs, half_id);
    SHOW_OFF(JabasStepArgs, half_weight);
    SHOW_OFF(JabasStepArgs, opt_kind);
    SHOW_OFF(JabasStepArgs, n_groups);
    SHOW_OFF(JabasStepArgs, first_step);
    SHOW_OFF(JabasStepArgs, nesterov);
    SHOW_OFF(JabasStepArgs, momentum);
    SHOW_OFF(JabasStepArgs, dampening);
    SHOW_OFF(JabasStepArgs, beta1);
    SHOW_OFF(JabasStepArgs, beta2);
    SHOW_OFF(JabasStepArgs, eps);
    SHOW_OFF(JabasStepArgs, groups);
    SHOW_OFF(JabasStepArgs, grad_scale);
    SHOW_OFF(JabasStepArgs, scalars_dev);

    /* slots of the pair products in a row of level JABAS_STATS_GRAM, as the header's macro places them */
    printf("pairs4 %d,%d,%d,%d,%d,%d\n", JABAS_STAT_PAIR(4, 0, 1), JABAS_STAT_PAIR(4, 0, 2), JABAS_STAT_PAIR(4, 0, 3),
           JABAS_STAT_PAIR(4, 1, 2), JABAS_STAT_PAIR(4, 1, 3), JABAS_STAT_PAIR(4, 2, 3));
    printf("pairs3 %d,%d,%d\n", JABAS_STAT_PAIR(3, 0, 1), JABAS_STAT_PAIR(3, 0, 2), JABAS_STAT_PAIR(3, 1, 2));
    printf("version %s\n", jabas_sync_version());
    printf("status0 %s\n", jabas_status_string(JABAS_OK));

    /* two spans of a K = 2 fp32 SGD step; the addresses are never dereferenced by the encoder */
    JabasSpan spans[2];
    JabasBound bounds[2];
    memset(spans, 0, sizeof spans);
    memset(bounds, 0, sizeof bounds);
    for (int i = 0; i < 2; ++i) {
        char* base = (char*)0x7f0000000000ull + (size_t)i * 0x10000000ull;
        spans[i].grads[0] = base;
        spans[i].grads[1] = base + 0x1000000;
        spans[i].agg_out = (float*)(base + 0x2000000);
        spans[i].param = (float*)(base + 0x3000000);
        spans[i].state1 = (float*)(base + 0x4000000);
        spans[i].numel = 5000 + 4096 * i;
    }
    spans[1].bound_begin = 0;
    spans[1].bound_count = 2;
    bounds[0].start = 0;
    bounds[0].group = 0;
    bounds[1].start = 4000;
    bounds[1].group = 1;
    size_t nbytes = jabas_plan_bytes(spans, 2, 2, JABAS_F32);
    void* blob = malloc(nbytes);
    if (!blob) return 2;
    int rc = jabas_plan_encode(spans, 2, bounds, 2, 2, JABAS_F32, JABAS_OPT_SGD, blob, nbytes);
    printf("encode %d\n", rc);
    printf("chunks %lld\n", (long long)jabas_plan_chunks(blob, 0));
    printf("chunks_stats %lld\n", (long long)jabas_plan_chunks(blob, 1));
    printf("workspace %zu\n", jabas_plan_workspace_bytes(blob));
    spans[1].grads[1] = (char*)spans[1].grads[1] + 4; /* breaks the 16-byte congruence rule */
    rc = jabas_plan_encode(spans, 2, bounds, 2, 2, JABAS_F32, JABAS_OPT_SGD, blob, nbytes);
    printf("encode_misaligned %d %s\n", rc, jabas_status_string(rc));
    free(blob);
    return 0;
}
