/*
 * CPU oracle for the operator arithmetic of the preemptible executor.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing on the product path may link, import or
 * call this file; it exists so that tests, the smoke check and the CPU
 * baseline leg of the benchmark have an independent statement of the math.
 *
 * Provenance.  The reference (thustorage/GPreempt) holds no operator source:
 * its kernels are emitted by Apache TVM @ 513c2be0c3b853 (README.md:69-72,
 * scripts/compile/compile.py:33-57), which is not vendored, and its tests
 * assert no numerical result (src/tests/test-dnn.cpp:38-41).  The operators
 * here therefore restate the published, textbook definition of each relay op
 * the exported graphs contain (conv2d NCHW/OIHW with folded batch-norm,
 * dense, max/avg/global pooling, add, softmax, layer_norm, erf GELU, take,
 * batch_matmul).  Every function accumulates in double and rounds once to
 * float, so it is a tighter statement of the math than any fp32 kernel.
 *
 * Parity status: pinned against mathematics (closed forms, brute force on
 * tiny shapes, library routines of numpy/torch) in tests/test_oracle_ops.py.
 * Parity against the TVM-compiled numbers of the reference: UNPINNED (the
 * reference ships no outputs and TVM is absent).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_ACT_NONE 0
#define ORC_ACT_RELU 1
#define ORC_ACT_GELU 2

static inline double orc_act(double v, int act) {
    if (act == ORC_ACT_RELU) return v > 0.0 ? v : 0.0;
    if (act == ORC_ACT_GELU) return 0.5 * v * (1.0 + erf(v * 0.70710678118654752440));
    return v;
}

/* C[M,N] = act(A[M,K] * B + bias[n] + residual[M,N]).
 * b_is_nk == 0: B is K x N row-major (config 1 of the benchmark: "A 1024x1024
 * and B 1024x1024"); b_is_nk == 1: B is N x K row-major (relay nn.dense weight
 * layout, units x in_features).  bias / residual may be NULL. */
void orc_gemm_bias_act(int M, int N, int K, const float *A, long lda,
                       const float *B, long ldb, int b_is_nk, const float *bias,
                       const float *residual, long ldr, int act, float *C, long ldc) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        double *acc = (double *)malloc(sizeof(double) * (size_t)N);
        for (int n = 0; n < N; ++n) acc[n] = 0.0;
        if (b_is_nk) {
            for (int n = 0; n < N; ++n) {
                double s = 0.0;
                const float *a = A + (size_t)m * lda, *b = B + (size_t)n * ldb;
                for (int k = 0; k < K; ++k) s += (double)a[k] * (double)b[k];
                acc[n] = s;
            }
        } else {
            for (int k = 0; k < K; ++k) {
                double a = A[(size_t)m * lda + k];
                const float *b = B + (size_t)k * ldb;
                for (int n = 0; n < N; ++n) acc[n] += a * (double)b[n];
            }
        }
        for (int n = 0; n < N; ++n) {
            double v = acc[n];
            if (bias) v += bias[n];
            if (residual) v += residual[(size_t)m * ldr + n];
            C[(size_t)m * ldc + n] = (float)orc_act(v, act);
        }
        free(acc);
    }
}

/* batch_matmul: C[b] = alpha * A[b] (M x K) * op(B[b]); b_is_nk as above. */
void orc_bmm(int batch, int M, int N, int K, const float *A, long lda, long sa,
             const float *B, long ldb, long sb, int b_is_nk, float alpha, float *C,
             long ldc, long sc) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b)
        for (int m = 0; m < M; ++m)
            for (int n = 0; n < N; ++n) {
                double s = 0.0;
                for (int k = 0; k < K; ++k) {
                    double bv = b_is_nk ? B[(size_t)b * sb + (size_t)n * ldb + k]
                                        : B[(size_t)b * sb + (size_t)k * ldb + n];
                    s += (double)A[(size_t)b * sa + (size_t)m * lda + k] * bv;
                }
                C[(size_t)b * sc + (size_t)m * ldc + n] = (float)(s * (double)alpha);
            }
}

/* Direct convolution, NCHW activations, OIHW weights, groups = 1, dilation 1.
 * out[n,co,ho,wo] = act(sum_{ci,r,s} in[n,ci,ho*sh-ph+r,wo*sw-pw+s] * w[co,ci,r,s]
 *                       + bias[co] + residual[n,co,ho,wo]). */
void orc_conv2d_nchw(int N, int Cin, int H, int W, int Cout, int R, int S, int sh, int sw,
                     int ph, int pw, const float *in, const float *w, const float *bias,
                     const float *residual, int act, float *out) {
    int Ho = (H + 2 * ph - R) / sh + 1, Wo = (W + 2 * pw - S) / sw + 1;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int n = 0; n < N; ++n)
        for (int co = 0; co < Cout; ++co) {
            double *acc = (double *)calloc((size_t)Ho * Wo, sizeof(double));
            for (int ci = 0; ci < Cin; ++ci)
                for (int r = 0; r < R; ++r)
                    for (int s = 0; s < S; ++s) {
                        double wv = w[(((size_t)co * Cin + ci) * R + r) * S + s];
                        const float *plane = in + ((size_t)n * Cin + ci) * H * W;
                        for (int ho = 0; ho < Ho; ++ho) {
                            int hi = ho * sh - ph + r;
                            if (hi < 0 || hi >= H) continue;
                            for (int wo = 0; wo < Wo; ++wo) {
                                int wi = wo * sw - pw + s;
                                if (wi < 0 || wi >= W) continue;
                                acc[(size_t)ho * Wo + wo] += wv * (double)plane[(size_t)hi * W + wi];
                            }
                        }
                    }
            size_t base = ((size_t)n * Cout + co) * Ho * Wo;
            for (size_t i = 0; i < (size_t)Ho * Wo; ++i) {
                double v = acc[i];
                if (bias) v += bias[co];
                if (residual) v += residual[base + i];
                out[base + i] = (float)orc_act(v, act);
            }
            free(acc);
        }
}

/* Pooling, NCHW.  mode 0 = max (padding never wins), 1 = average with
 * count_include_pad = 0 (relay avg_pool2d default). */
void orc_pool2d_nchw(int N, int C, int H, int W, int R, int S, int sh, int sw, int ph, int pw,
                     int mode, const float *in, float *out) {
    int Ho = (H + 2 * ph - R) / sh + 1, Wo = (W + 2 * pw - S) / sw + 1;
#pragma omp parallel for schedule(static)
    for (long nc = 0; nc < (long)N * C; ++nc)
        for (int ho = 0; ho < Ho; ++ho)
            for (int wo = 0; wo < Wo; ++wo) {
                double best = -INFINITY, sum = 0.0;
                int cnt = 0;
                for (int r = 0; r < R; ++r)
                    for (int s = 0; s < S; ++s) {
                        int hi = ho * sh - ph + r, wi = wo * sw - pw + s;
                        if (hi < 0 || hi >= H || wi < 0 || wi >= W) continue;
                        double v = in[((size_t)nc * H + hi) * W + wi];
                        if (v > best) best = v;
                        sum += v;
                        ++cnt;
                    }
                if (mode == 3) cnt = R * S; /* padding counted as zeros */
                out[((size_t)nc * Ho + ho) * Wo + wo] = (float)(mode == 0 ? best : sum / (cnt ? cnt : 1));
            }
}

/* global_avg_pool2d: out[n,c] = mean over H*W. */
void orc_global_avgpool_nchw(int N, int C, int HW, const float *in, float *out) {
    for (long nc = 0; nc < (long)N * C; ++nc) {
        double s = 0.0;
        for (int i = 0; i < HW; ++i) s += in[(size_t)nc * HW + i];
        out[nc] = (float)(s / HW);
    }
}

/* out = act(a + b) elementwise; b may be NULL. */
void orc_add_act(long n, const float *a, const float *b, int act, float *out) {
    for (long i = 0; i < n; ++i) out[i] = (float)orc_act((double)a[i] + (b ? (double)b[i] : 0.0), act);
}

/* Per-channel affine + activation on NCHW: out = act(x*scale[c] + shift[c])
 * (an inference batch-norm that could not be folded into a preceding conv). */
void orc_scale_shift_act_nchw(int N, int C, int HW, const float *x, const float *scale,
                              const float *shift, int act, float *out) {
    for (long nc = 0; nc < (long)N * C; ++nc) {
        int c = (int)(nc % C);
        for (int i = 0; i < HW; ++i)
            out[(size_t)nc * HW + i] =
                (float)orc_act((double)x[(size_t)nc * HW + i] * scale[c] + shift[c], act);
    }
}

/* softmax over the last axis: rows x cols. */
void orc_softmax(long rows, int cols, const float *x, float *out) {
    for (long r = 0; r < rows; ++r) {
        const float *p = x + (size_t)r * cols;
        double mx = -INFINITY, s = 0.0;
        for (int c = 0; c < cols; ++c) if (p[c] > mx) mx = p[c];
        for (int c = 0; c < cols; ++c) s += exp((double)p[c] - mx);
        for (int c = 0; c < cols; ++c) out[(size_t)r * cols + c] = (float)(exp((double)p[c] - mx) / s);
    }
}

/* layer_norm over the last axis (biased variance), optional residual added first:
 * y = (x+res - mean) / sqrt(var + eps) * gamma + beta. */
void orc_layernorm(long rows, int cols, const float *x, const float *res, const float *gamma,
                   const float *beta, float eps, float *out) {
    for (long r = 0; r < rows; ++r) {
        double mean = 0.0, var = 0.0;
        for (int c = 0; c < cols; ++c)
            mean += (double)x[(size_t)r * cols + c] + (res ? (double)res[(size_t)r * cols + c] : 0.0);
        mean /= cols;
        for (int c = 0; c < cols; ++c) {
            double d = (double)x[(size_t)r * cols + c] + (res ? (double)res[(size_t)r * cols + c] : 0.0) - mean;
            var += d * d;
        }
        var /= cols;
        double inv = 1.0 / sqrt(var + (double)eps);
        for (int c = 0; c < cols; ++c) {
            double v = (double)x[(size_t)r * cols + c] + (res ? (double)res[(size_t)r * cols + c] : 0.0);
            out[(size_t)r * cols + c] = (float)((v - mean) * inv * gamma[c] + beta[c]);
        }
    }
}

/* take(table, ids, axis=0) summed with a position table: out[t,:] = tok[ids[t],:] + pos[t % seq,:]
 * (+ seg[0,:] if given).  ids are int64 as in the reference's BERT input
 * (src/tests/test-dnn.cpp:21-23). */
void orc_embed(long tokens, int seq, int hidden, const int64_t *ids, const float *tok,
               const float *pos, const float *seg, float *out) {
    for (long t = 0; t < tokens; ++t)
        for (int h = 0; h < hidden; ++h) {
            double v = (double)tok[(size_t)ids[t] * hidden + h] + (double)pos[(size_t)(t % seq) * hidden + h];
            if (seg) v += seg[h];
            out[(size_t)t * hidden + h] = (float)v;
        }
}

/* Inference batch-norm folded into the preceding convolution (what
 * relay.build(opt_level=3) does, scripts/compile/compile.py:55-56):
 *   w'[co,...] = w[co,...] * g[co]/sqrt(var[co]+eps);  b'[co] = beta[co] + (b[co]-mu[co]) * g/sqrt(var+eps). */
void orc_fold_bn(int Cout, long per_out, const float *w, const float *b, const float *gamma,
                 const float *beta, const float *mean, const float *var, float eps, float *w_out,
                 float *b_out) {
    for (int co = 0; co < Cout; ++co) {
        double k = (double)gamma[co] / sqrt((double)var[co] + (double)eps);
        for (long i = 0; i < per_out; ++i) w_out[(size_t)co * per_out + i] = (float)((double)w[(size_t)co * per_out + i] * k);
        b_out[co] = (float)((double)beta[co] + ((b ? (double)b[co] : 0.0) - (double)mean[co]) * k);
    }
}

/* Round-to-nearest-even float -> bf16 -> float, to model bf16 storage between
 * layers (fp16 rounding is done with numpy.float16 on the Python side). */
static inline float orc_bf16_round1(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return f;
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}
void orc_round_bf16(long n, const float *x, float *out) { for (long i = 0; i < n; ++i) out[i] = orc_bf16_round1(x[i]); }
