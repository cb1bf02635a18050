/*
 * CPU executor: whole model graphs run on the host cores through the block-level-preemption
 * tile loop, as the CPU baseline that sits beside the GPU numbers.
 *
 * TEST / MEASUREMENT INFRASTRUCTURE ONLY (see oracle_ops.c): used by tests/ and by the
 * cpu_baseline leg of bench.py, never by the product path.
 *
 * What is restated from the reference: the dispatcher of scripts/compile/convert_to_blp.py:40-69
 * (a persistent worker = one "workgroup": read the flag, claim the next tile index from the
 * kernel's atomic counter, decode it, run the body; on a raised flag record the kernel id in the
 * stop index and leave) and the launch loop of src/executor.cpp:211-232 (counters cleared, kernels
 * in order).  The operators are the same mathematics as oracle_ops.c in fp32 with vectorisable
 * inner loops, laid out like the GPU build (NHWC activations, [Cout][R][S][Cin] weights,
 * [units][in] dense weights), so that the host cores are not handicapped by scalar double loops.
 * Parity of this file is pinned by tests/test_oracle_exec.py against the compositions of
 * oracle/models.py (themselves pinned against torch on the CPU).
 *
 * One worker thread per core, pinned (the reference pins its client threads, src/util/util.cpp:3-10);
 * the workers stay alive across kernels and runs and meet at a barrier after every kernel, which
 * is what stream order is on the GPU.
 */
#define _GNU_SOURCE
#include <math.h>
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

enum { OX_GEMM = 0, OX_CONV = 1, OX_POOL = 2, OX_ELTWISE = 3, OX_SOFTMAX = 4, OX_LAYERNORM = 5, OX_EMBED = 6, OX_ATTENTION = 7 };
enum { OX_ACT_NONE = 0, OX_ACT_RELU = 1, OX_ACT_GELU = 2 };

typedef struct {
    int op, act;
    /* GEMM: c[M][N] = act(alpha * a[M][K] . b[N][K]^T + bias[N] + res[M][N]); rows lda / ldc / ldr apart */
    int M, N, K;
    long lda, ldc, ldr;
    const float *a, *b, *bias, *res;
    float *c;
    float alpha;
    /* CONV (NHWC, weights [cout][r][s][cin]): a = input, b = weights, c = output; pixel strides in floats */
    int n, h, w, cin, cout, r, s, stride, ph, pw, ho, wo;
    long in_ps, out_ps, res_ps;
    /* POOL (NHWC): mode 0 max, 1 average without padding, 2 global average, 3 average counting padding; window r x r */
    int mode;
    /* row operators: rows x cols; ELTWISE: c = act((a [+ b]) * gamma[col] + beta[col]) with strides lda, ldr (b), ldc */
    long rows;
    int cols;
    float eps, scale;
    const float *gamma, *beta;
    /* EMBED: c[t] = tok[ids[t]] + pos[t % seq] + seg[0] */
    const long long *ids;
    const float *tok, *pos, *seg;
    int seq, vocab;
    /* ATTENTION: per (batch, head): softmax(scale * q k^T) v; rows of q / k / v ld_qkv apart, head h at column h*head_dim */
    int batch, heads, head_dim;
    long ld_qkv;
    const float *q, *k, *v;
    /* planned */
    int tiles, sx, sy;
} ox_layer;

#define TM 16 /* GEMM / conv tile: rows (pixels) */
#define TN 64 /* GEMM / conv tile: columns (output channels) */
#define ROWS_PER_TILE 8

static float act_f(float v, int act) {
    if (act == OX_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == OX_ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
    return v;
}

/* dot products of one row x against four rows of y (K contiguous in all), vectorised */
__attribute__((target_clones("avx512f", "avx2,fma", "default")))
static void dot4(const float *x, const float *y0, const float *y1, const float *y2, const float *y3, int K, float *out) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma omp simd reduction(+ : s0, s1, s2, s3)
    for (int k = 0; k < K; ++k) {
        const float xv = x[k];
        s0 += xv * y0[k]; s1 += xv * y1[k]; s2 += xv * y2[k]; s3 += xv * y3[k];
    }
    out[0] += s0; out[1] += s1; out[2] += s2; out[3] += s3;
}

static void plan(ox_layer *L) {
    switch (L->op) {
        case OX_GEMM: L->sx = (L->N + TN - 1) / TN; L->sy = (L->M + TM - 1) / TM; break;
        case OX_CONV: L->ho = (L->h + 2 * L->ph - L->r) / L->stride + 1; L->wo = (L->w + 2 * L->pw - L->s) / L->stride + 1;
                      L->M = L->n * L->ho * L->wo; L->sx = (L->cout + TN - 1) / TN; L->sy = (L->M + TM - 1) / TM; break;
        case OX_POOL: if (L->mode == 2) { L->ho = L->wo = 1; } else { L->ho = (L->h + 2 * L->ph - L->r) / L->stride + 1; L->wo = (L->w + 2 * L->pw - L->r) / L->stride + 1; }
                      L->sx = 1; L->sy = (L->n * L->ho * L->wo + ROWS_PER_TILE - 1) / ROWS_PER_TILE; break;
        case OX_ATTENTION: L->sx = 1; L->sy = L->batch * L->heads * ((L->seq + TM - 1) / TM); break;
        default: L->sx = 1; L->sy = (int)((L->rows + ROWS_PER_TILE - 1) / ROWS_PER_TILE); break;
    }
    L->tiles = L->sx * L->sy;
}

/* ---- tile bodies ------------------------------------------------------------------------------ */
static void finish_tile(const ox_layer *L, float acc[TM][TN], int m0, int n0, int M, int N, long ldc, long ldr) {
    for (int i = 0; i < TM && m0 + i < M; ++i)
        for (int j = 0; j < TN && n0 + j < N; ++j) {
            float v = acc[i][j] * L->alpha + (L->bias ? L->bias[n0 + j] : 0.f);
            if (L->res) v += L->res[(long)(m0 + i) * ldr + n0 + j];
            L->c[(long)(m0 + i) * ldc + n0 + j] = act_f(v, L->act);
        }
}

static void gemm_tile(const ox_layer *L, int tx, int ty) {
    const int m0 = ty * TM, n0 = tx * TN;
    float acc[TM][TN];
    memset(acc, 0, sizeof acc);
    static const float zero[4] = {0};
    (void)zero;
    for (int i = 0; i < TM && m0 + i < L->M; ++i) {
        const float *x = L->a + (long)(m0 + i) * L->lda;
        int j = 0;
        for (; j + 4 <= TN && n0 + j + 4 <= L->N; j += 4)
            dot4(x, L->b + (long)(n0 + j) * L->K, L->b + (long)(n0 + j + 1) * L->K, L->b + (long)(n0 + j + 2) * L->K, L->b + (long)(n0 + j + 3) * L->K, L->K, &acc[i][j]);
        for (; j < TN && n0 + j < L->N; ++j) {
            const float *y = L->b + (long)(n0 + j) * L->K;
            float s = 0.f;
            for (int k = 0; k < L->K; ++k) s += x[k] * y[k];
            acc[i][j] = s;
        }
    }
    finish_tile(L, acc, m0, n0, L->M, L->N, L->ldc, L->ldr);
}

static void conv_tile(const ox_layer *L, int tx, int ty) {
    const int m0 = ty * TM, n0 = tx * TN;
    float acc[TM][TN];
    memset(acc, 0, sizeof acc);
    const long wrow = (long)L->r * L->s * L->cin;  /* floats per output channel of the weights */
    for (int i = 0; i < TM && m0 + i < L->M; ++i) {
        const int m = m0 + i, img = m / (L->ho * L->wo), rem = m - img * (L->ho * L->wo), oh = rem / L->wo, ow = rem - oh * L->wo;
        for (int r = 0; r < L->r; ++r) {
            const int ih = oh * L->stride - L->ph + r;
            if (ih < 0 || ih >= L->h) continue;
            for (int s = 0; s < L->s; ++s) {
                const int iw = ow * L->stride - L->pw + s;
                if (iw < 0 || iw >= L->w) continue;
                const float *x = L->a + (((long)img * L->h + ih) * L->w + iw) * L->in_ps;
                const float *wt = L->b + ((long)r * L->s + s) * L->cin;
                int j = 0;
                for (; j + 4 <= TN && n0 + j + 4 <= L->cout; j += 4)
                    dot4(x, wt + (n0 + j) * wrow, wt + (n0 + j + 1) * wrow, wt + (n0 + j + 2) * wrow, wt + (n0 + j + 3) * wrow, L->cin, &acc[i][j]);
                for (; j < TN && n0 + j < L->cout; ++j) {
                    const float *y = wt + (n0 + j) * wrow;
                    float sum = 0.f;
                    for (int k = 0; k < L->cin; ++k) sum += x[k] * y[k];
                    acc[i][j] += sum;
                }
            }
        }
    }
    finish_tile(L, acc, m0, n0, L->M, L->cout, L->out_ps, L->res_ps);
}

static void pool_tile(const ox_layer *L, int ty) {
    const int total = L->n * L->ho * L->wo, C = L->cin;
    for (int p = ty * ROWS_PER_TILE; p < (ty + 1) * ROWS_PER_TILE && p < total; ++p) {
        const int img = p / (L->ho * L->wo), rem = p - img * (L->ho * L->wo), oh = rem / L->wo, ow = rem - oh * L->wo;
        float *o = L->c + (long)p * L->out_ps;
        if (L->mode == 2) {
            for (int c = 0; c < C; ++c) o[c] = 0.f;
            for (int i = 0; i < L->h * L->w; ++i) {
                const float *x = L->a + ((long)img * L->h * L->w + i) * L->in_ps;
                for (int c = 0; c < C; ++c) o[c] += x[c];
            }
            for (int c = 0; c < C; ++c) o[c] /= (float)(L->h * L->w);
            continue;
        }
        for (int c = 0; c < C; ++c) o[c] = L->mode == 0 ? -INFINITY : 0.f;
        int cnt = 0;
        for (int r = 0; r < L->r; ++r) {
            const int ih = oh * L->stride - L->ph + r;
            if (ih < 0 || ih >= L->h) continue;
            for (int s = 0; s < L->r; ++s) {
                const int iw = ow * L->stride - L->pw + s;
                if (iw < 0 || iw >= L->w) continue;
                const float *x = L->a + (((long)img * L->h + ih) * L->w + iw) * L->in_ps;
                if (L->mode == 0) for (int c = 0; c < C; ++c) o[c] = x[c] > o[c] ? x[c] : o[c];
                else for (int c = 0; c < C; ++c) o[c] += x[c];
                ++cnt;
            }
        }
        if (L->mode == 3) cnt = L->r * L->r;
        if (L->mode != 0) for (int c = 0; c < C; ++c) o[c] /= (float)(cnt > 0 ? cnt : 1);
    }
}

static void row_tile(const ox_layer *L, int ty) {
    for (long row = (long)ty * ROWS_PER_TILE; row < (long)(ty + 1) * ROWS_PER_TILE && row < L->rows; ++row) {
        const int C = L->cols;
        float *o = L->c + row * L->ldc;
        if (L->op == OX_ELTWISE) {
            const float *x = L->a + row * L->lda, *y = L->b ? L->b + row * L->ldr : NULL;
            for (int c = 0; c < C; ++c) {
                float v = x[c] + (y ? y[c] : 0.f);
                if (L->gamma) v *= L->gamma[c];
                if (L->beta) v += L->beta[c];
                o[c] = act_f(v, L->act);
            }
        } else if (L->op == OX_SOFTMAX) {
            const float *x = L->a + row * L->lda;
            float mx = -INFINITY, sum = 0.f;
            for (int c = 0; c < C; ++c) mx = x[c] * L->scale > mx ? x[c] * L->scale : mx;
            for (int c = 0; c < C; ++c) { o[c] = expf(x[c] * L->scale - mx); sum += o[c]; }
            for (int c = 0; c < C; ++c) o[c] /= sum;
        } else if (L->op == OX_LAYERNORM) {
            const float *x = L->a + row * L->lda, *y = L->res ? L->res + row * L->ldr : NULL;
            float mean = 0.f, var = 0.f;
            for (int c = 0; c < C; ++c) { o[c] = x[c] + (y ? y[c] : 0.f); mean += o[c]; }
            mean /= (float)C;
            for (int c = 0; c < C; ++c) var += (o[c] - mean) * (o[c] - mean);
            const float inv = 1.f / sqrtf(var / (float)C + L->eps);
            for (int c = 0; c < C; ++c) o[c] = (o[c] - mean) * inv * L->gamma[c] + L->beta[c];
        } else { /* OX_EMBED */
            long long id = L->ids[row];
            if (id < 0) id = 0;
            if (id >= L->vocab) id = L->vocab - 1;
            const float *e = L->tok + id * C, *p = L->pos + (row % L->seq) * C;
            for (int c = 0; c < C; ++c) o[c] = e[c] + p[c] + (L->seg ? L->seg[c] : 0.f);
        }
    }
}

/* one tile = TM queries of one (batch, head): scores against every key, softmax, weighted values */
static void attention_tile(const ox_layer *L, int ty) {
    const int qt = (L->seq + TM - 1) / TM, bh = ty / qt, q0 = (ty - bh * qt) * TM, b = bh / L->heads, h = bh - b * L->heads, D = L->head_dim, S = L->seq;
    float *sc = (float *)malloc(sizeof(float) * (size_t)S);
    for (int i = q0; i < q0 + TM && i < S; ++i) {
        const float *q = L->q + ((long)b * S + i) * L->ld_qkv + h * D;
        float mx = -INFINITY, sum = 0.f;
        for (int j = 0; j < S; ++j) {
            const float *k = L->k + ((long)b * S + j) * L->ld_qkv + h * D;
            float s = 0.f;
            for (int d = 0; d < D; ++d) s += q[d] * k[d];
            sc[j] = s * L->scale;
            mx = sc[j] > mx ? sc[j] : mx;
        }
        for (int j = 0; j < S; ++j) { sc[j] = expf(sc[j] - mx); sum += sc[j]; }
        float *o = L->c + ((long)b * S + i) * L->ldc + h * D;
        for (int d = 0; d < D; ++d) o[d] = 0.f;
        for (int j = 0; j < S; ++j) {
            const float *v = L->v + ((long)b * S + j) * L->ld_qkv + h * D;
            const float p = sc[j] / sum;
            for (int d = 0; d < D; ++d) o[d] += p * v[d];
        }
    }
    free(sc);
}

static void run_tile(const ox_layer *L, int idx) {
    /* x = idx % sx, y = (idx / sx) % sy   (convert_to_blp.py:52-54; z = 0 here) */
    const int tx = idx % L->sx, ty = (idx / L->sx) % L->sy;
    switch (L->op) {
        case OX_GEMM: gemm_tile(L, tx, ty); break;
        case OX_CONV: conv_tile(L, tx, ty); break;
        case OX_POOL: pool_tile(L, ty); break;
        case OX_ATTENTION: attention_tile(L, ty); break;
        default: row_tile(L, ty); break;
    }
}

/* ---- the executor ------------------------------------------------------------------------------- */
typedef struct {
    ox_layer *layers;
    int n_layers, threads, passes;
    atomic_int *executed;      /* one claim counter per kernel (src/executor.cpp:333) */
    atomic_int flag;           /* *preempted */
    atomic_int stop_index;     /* *pStopIndex, -1 = none */
    int inject_kernel, inject_claim;
    int first_kernel;          /* resume: kernels [first_kernel, n) are launched, counters untouched */
    pthread_barrier_t bar;
    double *pass_ms;
} ox_exec;

typedef struct { ox_exec *x; int id; } ox_worker;

static double now_ms(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec * 1e3 + ts.tv_nsec / 1e6;
}

static void *worker_main(void *arg) {
    ox_worker *w = (ox_worker *)arg;
    ox_exec *x = w->x;
    cpu_set_t allowed, set;
    if (sched_getaffinity(0, sizeof allowed, &allowed) == 0 && CPU_COUNT(&allowed) > 0) {  /* the id-th core this process may use */
        int want = w->id % CPU_COUNT(&allowed), cpu = 0;
        for (; cpu < CPU_SETSIZE; ++cpu)
            if (CPU_ISSET(cpu, &allowed) && want-- == 0) break;
        CPU_ZERO(&set);
        CPU_SET(cpu, &set);
        pthread_setaffinity_np(pthread_self(), sizeof set, &set);  /* best effort */
    }
    for (int pass = 0; pass < x->passes; ++pass) {
        pthread_barrier_wait(&x->bar);
        double t0 = 0;
        if (w->id == 0) t0 = now_ms();
        for (int k = x->first_kernel; k < x->n_layers; ++k) {
            const ox_layer *L = &x->layers[k];
            /* one persistent "workgroup": convert_to_blp.py:40-69 */
            for (;;) {
                if (atomic_load_explicit(&x->flag, memory_order_relaxed)) {
                    int expect = -1;
                    atomic_compare_exchange_strong(&x->stop_index, &expect, k);
                    break;
                }
                const int idx = atomic_fetch_add_explicit(&x->executed[k], 1, memory_order_relaxed);
                if (idx >= L->tiles) break;
                if (k == x->inject_kernel && idx == x->inject_claim) atomic_store(&x->flag, 1);
                run_tile(L, idx);
            }
            pthread_barrier_wait(&x->bar);  /* stream order: the next kernel starts when this one has drained */
        }
        if (w->id == 0 && x->pass_ms) x->pass_ms[pass] = now_ms() - t0;
        pthread_barrier_wait(&x->bar);
        if (w->id == 0 && pass + 1 < x->passes)  /* execute(): counters cleared before the next submission */
            for (int k = 0; k < x->n_layers; ++k) atomic_store(&x->executed[k], 0);
    }
    return NULL;
}

static int ox_go(ox_exec *x) {
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)x->threads);
    ox_worker *ws = (ox_worker *)malloc(sizeof(ox_worker) * (size_t)x->threads);
    pthread_barrier_init(&x->bar, NULL, (unsigned)x->threads);
    for (int i = 0; i < x->threads; ++i) { ws[i].x = x; ws[i].id = i; pthread_create(&th[i], NULL, worker_main, &ws[i]); }
    for (int i = 0; i < x->threads; ++i) pthread_join(th[i], NULL);
    pthread_barrier_destroy(&x->bar);
    free(th); free(ws);
    return 0;
}

void orx_plan(ox_layer *layers, int n) { for (int i = 0; i < n; ++i) plan(&layers[i]); }
int orx_layer_bytes(void) { return (int)sizeof(ox_layer); }

/* Runs the kernel list `passes` times on `threads` pinned workers; pass_ms receives the wall time of every pass. */
int orx_run(ox_layer *layers, int n, int threads, int passes, double *pass_ms) {
    if (n < 1 || threads < 1 || passes < 1) return -1;
    orx_plan(layers, n);
    ox_exec x;
    memset(&x, 0, sizeof x);
    x.layers = layers; x.n_layers = n; x.threads = threads; x.passes = passes; x.pass_ms = pass_ms;
    x.executed = (atomic_int *)calloc((size_t)n, sizeof(atomic_int));
    atomic_store(&x.flag, 0); atomic_store(&x.stop_index, -1);
    x.inject_kernel = -1; x.inject_claim = -1; x.first_kernel = 0;
    ox_go(&x);
    free(x.executed);
    return 0;
}

/* One submission that is stopped when claim `inject_claim` of kernel `inject_kernel` is made, then
 * resumed from the stop index with the counters untouched (src/executor.cpp:269-298).  Returns the
 * stop index (-1: it ran to the end); claims_at_stop receives the claim counters at the stop. */
int orx_run_preempted(ox_layer *layers, int n, int threads, int inject_kernel, int inject_claim, int *claims_at_stop) {
    orx_plan(layers, n);
    ox_exec x;
    memset(&x, 0, sizeof x);
    x.layers = layers; x.n_layers = n; x.threads = threads; x.passes = 1;
    x.executed = (atomic_int *)calloc((size_t)n, sizeof(atomic_int));
    atomic_store(&x.flag, 0); atomic_store(&x.stop_index, -1);
    x.inject_kernel = inject_kernel; x.inject_claim = inject_claim;
    ox_go(&x);
    const int stop = atomic_load(&x.stop_index);
    if (claims_at_stop) for (int k = 0; k < n; ++k) claims_at_stop[k] = atomic_load(&x.executed[k]);
    if (stop >= 0) {
        /* every worker that saw the flag left after its claim check, so each claim below `total` was run;
         * workers that found the counter exhausted overshot it once each, as on the GPU */
        atomic_store(&x.flag, 0); atomic_store(&x.stop_index, -1);
        x.inject_kernel = -1; x.first_kernel = stop;
        ox_go(&x);
    }
    free(x.executed);
    return stop;
}
