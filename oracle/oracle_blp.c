/*
 * CPU restatement of the reference's block-level-preemption (BLP) protocol.
 *
 * TEST INFRASTRUCTURE ONLY (see oracle_ops.c).  One POSIX thread stands for
 * one persistent workgroup.
 *
 * Reference lines restated here:
 *   - dispatcher loop .................. scripts/compile/convert_to_blp.py:40-69
 *   - extra argument order ............. scripts/compile/convert_to_blp.py:35
 *   - grid clamp / per-kernel counter .. src/model.cpp:366-396
 *   - execute (counters zeroed) ........ src/executor.cpp:211-232
 *   - getStopPoint / resume ............ src/executor.cpp:269-298
 *   - preempt-then-resume test shape ... src/tests/test-dnn-blp.cpp:36-42
 *
 * Parity status: pinned by invariants that hold for every interleaving
 * (tests/test_oracle_blp.py): each tile runs exactly once across any number
 * of preempt/resume rounds, the tile-id decode matches brute force, the stop
 * index is the first kernel that saw the flag, counters are reset only by
 * execute, and a preempted-then-resumed GEMM is memcmp-equal to an
 * uninterrupted one.
 */
#include <pthread.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* x = idx % sx, y = (idx / sx) % sy, z = idx / (sx*sy)   (convert_to_blp.py:52-54) */
void orc_blp_decode(int idx, int sx, int sy, int *x, int *y, int *z) {
    *x = idx % sx;
    *y = (idx / sx) % sy;
    *z = idx / (sx * sy);
}

typedef void (*orc_tile_fn)(void *user, int kernel_id, int x, int y, int z);

typedef struct {
    atomic_int flag;        /* *preempted : shared by every best-effort tenant */
    atomic_int stop_index;  /* *pStopIndex: one per executor, -1 = none        */
    atomic_int *executed;   /* one claim counter per kernel                    */
    int n_kernels;
    const int *total;       /* tiles per kernel = gx*gy*gz of the original grid */
    const int *shape;       /* 3 ints per kernel: original grid                */
    /* deterministic injection: when the claim that returns inject_claim in
     * kernel inject_kernel is made, that "workgroup" raises the flag itself,
     * after the claim, so exactly the tiles claimed so far are still owed. */
    int inject_kernel, inject_claim;
    orc_tile_fn body;
    void *user;
} orc_blp;

typedef struct { orc_blp *s; int kernel_id; } wg_arg;

/* One persistent workgroup: convert_to_blp.py:40-69. */
static void *wg_main(void *p) {
    wg_arg *a = (wg_arg *)p;
    orc_blp *s = a->s;
    int k = a->kernel_id;
    for (;;) {
        int stop = atomic_load(&s->flag);
        int x = 0, y = 0, z = 0;
        if (!stop) {
            int idx = atomic_fetch_add(&s->executed[k], 1);
            if (idx >= s->total[k]) stop = 1;
            else {
                orc_blp_decode(idx, s->shape[3 * k], s->shape[3 * k + 1], &x, &y, &z);
                if (k == s->inject_kernel && idx == s->inject_claim) atomic_store(&s->flag, 1);
            }
        } else {
            int expect = -1;
            atomic_compare_exchange_strong(&s->stop_index, &expect, k);
        }
        if (stop) return NULL;
        s->body(s->user, k, x, y, z);
    }
}

/* One kernel launch: grid = min(total, n_workers) x 1 x 1 (model.cpp:373-385);
 * returns when every workgroup has left, like a stream-ordered kernel. */
static void launch(orc_blp *s, int k, int n_workers) {
    int n = s->total[k] < n_workers ? s->total[k] : n_workers;
    if (n < 1) n = 1;
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * n);
    wg_arg a = {s, k};
    for (int i = 0; i < n; ++i) pthread_create(&th[i], NULL, wg_main, &a);
    for (int i = 0; i < n; ++i) pthread_join(th[i], NULL);
    free(th);
}

/* BLPExecutor::execute: zero the counters, launch every kernel in order
 * (executor.cpp:211-225). */
static void blp_execute(orc_blp *s, int n_workers) {
    for (int k = 0; k < s->n_kernels; ++k) atomic_store(&s->executed[k], 0);
    for (int k = 0; k < s->n_kernels; ++k) launch(s, k, n_workers);
}

/* BLPExecutor::getStopPoint + resume: read the stop index, reset it to -1,
 * relaunch kernels [stop, n) WITHOUT touching the counters
 * (executor.cpp:269-298).  Returns the stop index that was read. */
static int blp_resume(orc_blp *s, int n_workers) {
    int stop = atomic_load(&s->stop_index);
    if (stop == -1) return -1;
    atomic_store(&s->stop_index, -1);
    for (int k = stop; k < s->n_kernels; ++k) launch(s, k, n_workers);
    return stop;
}

/* ---- generic chain of kernels with visit counting ---------------------- */

typedef struct { atomic_int *visits; const int *offset; const int *shape; atomic_int bad_decode; } count_user;

static void count_body(void *u, int k, int x, int y, int z) {
    count_user *c = (count_user *)u;
    int sx = c->shape[3 * k], sy = c->shape[3 * k + 1], sz = c->shape[3 * k + 2];
    if (x >= sx || y >= sy || z >= sz) { atomic_fetch_add(&c->bad_decode, 1); return; }
    atomic_fetch_add(&c->visits[c->offset[k] + (z * sy + y) * sx + x], 1);
}

/* Runs execute, then for each injection i: (flag raised inside the run by the
 * claim inject_claim[i] of kernel inject_kernel[i]) -> host clears the flag ->
 * resume.  Injection i+1 is armed during resume i.  visits_out has one int per
 * tile of every kernel (concatenated); stop_out one int per injection (the
 * stop index read by that resume); executed_out the final counters.
 * Returns the number of out-of-range decodes (must be 0). */
int orc_blp_run_chain(int n_kernels, const int *shape, int n_workers, int n_inject,
                      const int *inject_kernel, const int *inject_claim, int *visits_out,
                      int *stop_out, int *executed_out) {
    int *total = (int *)malloc(sizeof(int) * n_kernels), *offset = (int *)malloc(sizeof(int) * n_kernels);
    int sum = 0;
    for (int k = 0; k < n_kernels; ++k) {
        total[k] = shape[3 * k] * shape[3 * k + 1] * shape[3 * k + 2];
        offset[k] = sum;
        sum += total[k];
    }
    atomic_int *visits = (atomic_int *)calloc(sum ? sum : 1, sizeof(atomic_int));
    atomic_int *executed = (atomic_int *)calloc(n_kernels, sizeof(atomic_int));
    count_user cu = {visits, offset, shape, 0};
    orc_blp s;
    atomic_init(&s.flag, 0);
    atomic_init(&s.stop_index, -1);
    s.executed = executed; s.n_kernels = n_kernels; s.total = total; s.shape = shape;
    s.body = count_body; s.user = &cu;
    s.inject_kernel = n_inject > 0 ? inject_kernel[0] : -1;
    s.inject_claim = n_inject > 0 ? inject_claim[0] : -1;
    blp_execute(&s, n_workers);
    for (int i = 0; i < n_inject; ++i) {
        atomic_store(&s.flag, 0);                     /* host: *flag = 0 (test-dnn-blp.cpp:41) */
        s.inject_kernel = i + 1 < n_inject ? inject_kernel[i + 1] : -1;
        s.inject_claim = i + 1 < n_inject ? inject_claim[i + 1] : -1;
        stop_out[i] = blp_resume(&s, n_workers);
    }
    for (int i = 0; i < sum; ++i) visits_out[i] = atomic_load(&visits[i]);
    for (int k = 0; k < n_kernels; ++k) executed_out[k] = atomic_load(&executed[k]);
    int bad = atomic_load(&cu.bad_decode);
    free(total); free(offset); free(visits); free(executed);
    return bad;
}

/* ---- config 1: preemptible fp32 GEMM + bias + ReLU on the CPU ----------- */

typedef struct {
    int M, N, K, tm, tn;
    const float *A, *B, *bias;
    float *C;
} gemm_user;

/* One output tile, fixed k order, fp32 accumulate: the result of a tile does
 * not depend on which worker or which launch computes it. */
static void gemm_tile(void *u, int kid, int x, int y, int z) {
    (void)kid; (void)z;
    gemm_user *g = (gemm_user *)u;
    int m0 = y * g->tm, n0 = x * g->tn;
    int m1 = m0 + g->tm < g->M ? m0 + g->tm : g->M, n1 = n0 + g->tn < g->N ? n0 + g->tn : g->N;
    for (int m = m0; m < m1; ++m)
        for (int n = n0; n < n1; ++n) {
            float acc = 0.f;
            for (int k = 0; k < g->K; ++k) acc += g->A[(size_t)m * g->K + k] * g->B[(size_t)k * g->N + n];
            acc += g->bias[n];
            g->C[(size_t)m * g->N + n] = acc > 0.f ? acc : 0.f;
        }
}

/* C = relu(A*B + bias) through the BLP dispatcher with n_inject preemptions at
 * the given claim counts.  Returns the number of resumes that found a stop
 * index (== preemptions that actually interrupted the kernel). */
int orc_blp_gemm(int M, int N, int K, const float *A, const float *B, const float *bias, float *C,
                 int tm, int tn, int n_workers, int n_inject, const int *inject_claim) {
    int shape[3] = {(N + tn - 1) / tn, (M + tm - 1) / tm, 1};
    int total = shape[0] * shape[1];
    atomic_int executed;
    atomic_init(&executed, 0);
    gemm_user gu = {M, N, K, tm, tn, A, B, bias, C};
    orc_blp s;
    atomic_init(&s.flag, 0);
    atomic_init(&s.stop_index, -1);
    s.executed = &executed; s.n_kernels = 1; s.total = &total; s.shape = shape;
    s.body = gemm_tile; s.user = &gu;
    s.inject_kernel = n_inject > 0 ? 0 : -1;
    s.inject_claim = n_inject > 0 ? inject_claim[0] : -1;
    blp_execute(&s, n_workers);
    int hits = 0;
    for (int i = 0; i < n_inject; ++i) {
        atomic_store(&s.flag, 0);
        s.inject_claim = i + 1 < n_inject ? inject_claim[i + 1] : -1;
        s.inject_kernel = i + 1 < n_inject ? 0 : -1;
        if (blp_resume(&s, n_workers) != -1) ++hits;
    }
    return hits;
}
