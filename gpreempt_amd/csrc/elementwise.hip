// Preemptible memory-bound operators: layout change, pooling, elementwise, softmax,
// layer-norm, embedding.  All are HBM-bound, so each thread moves 16 bytes per access,
// consecutive lanes touch consecutive 16-byte chunks (coalesced wave64 accesses), arithmetic is
// fp32, and row reductions stay inside one wavefront (cross-lane shuffles, no LDS round trip).
// Work is cut into tiles handed out by gp::tile_loop so that every operator can be stopped at
// a tile boundary and resumed without redoing or skipping a tile.
#include "common.hpp"

namespace gp {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct VecIO;
template <> struct VecIO<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ void load(const float *p, float (&f)[4]) {
        f32x4 v = *(const f32x4 *)p;
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = v[i];
    }
    static __device__ __forceinline__ void store(float *p, const float (&f)[4]) {
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = f[i];
        *(f32x4 *)p = v;
    }
    static __device__ __forceinline__ float ld1(const float *p) { return *p; }
    static __device__ __forceinline__ void st1(float *p, float v) { *p = v; }
};
template <> struct VecIO<_Float16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void load(const _Float16 *p, float (&f)[8]) {
        f16x8 v = *(const f16x8 *)p;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
    }
    static __device__ __forceinline__ void store(_Float16 *p, const float (&f)[8]) {
        f16x8 v;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (_Float16)f[i];
        *(f16x8 *)p = v;
    }
    static __device__ __forceinline__ float ld1(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void st1(_Float16 *p, float v) { *p = (_Float16)v; }
};
template <> struct VecIO<__bf16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void load(const __bf16 *p, float (&f)[8]) {
        bf16x8 v = *(const bf16x8 *)p;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
    }
    static __device__ __forceinline__ void store(__bf16 *p, const float (&f)[8]) {
        bf16x8 v;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (__bf16)f[i];
        *(bf16x8 *)p = v;
    }
    static __device__ __forceinline__ float ld1(const __bf16 *p) { return (float)*p; }
    static __device__ __forceinline__ void st1(__bf16 *p, float v) { *p = (__bf16)v; }
};

__device__ __forceinline__ float act_f(float v, int act) {
    if (act == GP_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == GP_ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

constexpr int NT = 256;

// ---- NCHW -> NHWC (channel padded) ---------------------------------------------------------
// tile = 256 pixels of one image; a thread owns one pixel: C strided reads (coalesced across
// the wave for each channel) and one contiguous c_pad-wide write.
template <typename TI, typename TO>
__global__ __launch_bounds__(NT) void nchw_to_nhwc_kernel(const TI *in, TO *out, int C, int HW, int c_pad, BlpArgs blp) {
    tile_loop(blp, [&](TileIdx t) {
        int pix = t.x * NT + threadIdx.x;
        if (pix >= HW) return;
        const TI *src = in + (long)t.y * C * HW + pix;
        TO *dst = out + ((long)t.y * HW + pix) * c_pad;
        if (c_pad == VecIO<TO>::VEC) {  // the usual case (3 channels padded to one vector): one 16-byte store
            float v[VecIO<TO>::VEC];
#pragma unroll
            for (int c = 0; c < VecIO<TO>::VEC; ++c) v[c] = c < C ? VecIO<TI>::ld1(src + (long)c * HW) : 0.f;
            VecIO<TO>::store(dst, v);
            return;
        }
        for (int c = 0; c < c_pad; ++c) {
            float v = c < C ? VecIO<TI>::ld1(src + (long)c * HW) : 0.f;
            VecIO<TO>::st1(dst + c, v);
        }
    });
}

// ---- pooling, NHWC -------------------------------------------------------------------------
// item = (output pixel, 16-byte channel chunk); tile = 256 items.
template <typename T>
__global__ __launch_bounds__(NT) void pool_kernel(gp_pool_params p, int Ho, int Wo, long items, BlpArgs blp) {
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.C / VEC;
    tile_loop(blp, [&](TileIdx t) {
        long item = (long)t.x * NT + threadIdx.x;
        if (item >= items) return;
        int ch = (int)(item % chunks);
        long pix = item / chunks;
        const T *in = (const T *)p.in;
        T *out = (T *)p.out;
        float acc[VEC];
        if (p.mode == 2) {  // global average: pix = n
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
            const T *src = in + pix * p.H * p.W * p.in_pix_stride + ch * VEC;
            for (int i = 0; i < p.H * p.W; ++i) {
                float f[VEC];
                VecIO<T>::load(src + (long)i * p.in_pix_stride, f);
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] += f[j];
            }
            float inv = 1.f / (float)(p.H * p.W);
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] *= inv;
            VecIO<T>::store(out + pix * p.out_pix_stride + ch * VEC, acc);
            return;
        }
        int wo = (int)(pix % Wo);
        long q = pix / Wo;
        int ho = (int)(q % Ho);
        long n = q / Ho;
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = p.mode == 0 ? -INFINITY : 0.f;
        int cnt = 0;
        for (int r = 0; r < p.R; ++r) {
            int hi = ho * p.stride - p.pad + r;
            if ((unsigned)hi >= (unsigned)p.H) continue;
            for (int s = 0; s < p.S; ++s) {
                int wi = wo * p.stride - p.pad + s;
                if ((unsigned)wi >= (unsigned)p.W) continue;
                float f[VEC];
                VecIO<T>::load(in + ((n * p.H + hi) * p.W + wi) * p.in_pix_stride + ch * VEC, f);
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = p.mode == 0 ? fmaxf(acc[j], f[j]) : acc[j] + f[j];
                ++cnt;
            }
        }
        if (p.mode == 1) {
            float inv = 1.f / (float)(cnt > 0 ? cnt : 1);
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] *= inv;
        }
        VecIO<T>::store(out + pix * p.out_pix_stride + ch * VEC, acc);
    });
}

// ---- elementwise ---------------------------------------------------------------------------
// item = (row, 16-byte chunk); tile = 1024 items (4 per thread, strided by 256 for coalescing).
constexpr int ELT_PER = 4;
template <typename T>
__global__ __launch_bounds__(NT) void eltwise_kernel(gp_eltwise_params p, long items, BlpArgs blp) {
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.cols / VEC;
    tile_loop(blp, [&](TileIdx t) {
#pragma unroll
        for (int u = 0; u < ELT_PER; ++u) {
            long item = ((long)t.x * ELT_PER + u) * NT + threadIdx.x;
            if (item >= items) continue;
            int ch = (int)(item % chunks);
            long row = item / chunks;
            float a[VEC];
            VecIO<T>::load((const T *)p.a + row * p.a_stride + ch * VEC, a);
            if (p.b) {
                float b[VEC];
                VecIO<T>::load((const T *)p.b + row * p.b_stride + ch * VEC, b);
#pragma unroll
                for (int j = 0; j < VEC; ++j) a[j] += b[j];
            }
            if (p.scale) {
                float sc[VEC];
                VecIO<T>::load((const T *)p.scale + ch * VEC, sc);
#pragma unroll
                for (int j = 0; j < VEC; ++j) a[j] *= sc[j];
            }
            if (p.shift) {
                float sh[VEC];
                VecIO<T>::load((const T *)p.shift + ch * VEC, sh);
#pragma unroll
                for (int j = 0; j < VEC; ++j) a[j] += sh[j];
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) a[j] = act_f(a[j], p.act);
            VecIO<T>::store((T *)p.out + row * p.out_stride + ch * VEC, a);
        }
    });
}

// ---- softmax -------------------------------------------------------------------------------
// one wavefront per row, 4 rows per tile; lane i reads elements i, i+64, ...
template <typename T>
__global__ __launch_bounds__(NT) void softmax_kernel(gp_softmax_params p, BlpArgs blp) {
    tile_loop(blp, [&](TileIdx t) {
        long row = (long)t.x * 4 + (threadIdx.x >> 6);
        if (row >= p.rows) return;
        const int lane = threadIdx.x & 63;
        const T *x = (const T *)p.x + row * p.cols;
        T *o = (T *)p.out + row * p.cols;
        float mx = -INFINITY;
        for (int c = lane; c < p.cols; c += 64) mx = fmaxf(mx, VecIO<T>::ld1(x + c) * p.scale);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int c = lane; c < p.cols; c += 64) sum += __expf(VecIO<T>::ld1(x + c) * p.scale - mx);
        sum = wave_sum(sum);
        float inv = 1.f / sum;
        for (int c = lane; c < p.cols; c += 64) VecIO<T>::st1(o + c, __expf(VecIO<T>::ld1(x + c) * p.scale - mx) * inv);
    });
}

// ---- layer norm ----------------------------------------------------------------------------
// one wavefront per row, 4 rows per tile; the row (plus residual) is kept in registers
// (up to MAXC 16-byte chunks per lane), so HBM sees one read and one write per element.
template <typename T, int MAXC>
__global__ __launch_bounds__(NT) void layernorm_kernel(gp_layernorm_params p, BlpArgs blp) {
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.cols / VEC;
    tile_loop(blp, [&](TileIdx t) {
        long row = (long)t.x * 4 + (threadIdx.x >> 6);
        if (row >= p.rows) return;
        const int lane = threadIdx.x & 63;
        const T *x = (const T *)p.x + row * p.cols;
        const T *r = p.residual ? (const T *)p.residual + row * p.cols : nullptr;
        float v[MAXC][VEC];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            int ch = lane + i * 64;
            if (ch < chunks) {
                VecIO<T>::load(x + ch * VEC, v[i]);
                if (r) {
                    float rr[VEC];
                    VecIO<T>::load(r + ch * VEC, rr);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) v[i][j] += rr[j];
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) sum += v[i][j];
            }
        }
        float mean = wave_sum(sum) / (float)p.cols;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            int ch = lane + i * 64;
            if (ch < chunks) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) { float d = v[i][j] - mean; sq += d * d; }
            }
        }
        float inv = rsqrtf(wave_sum(sq) / (float)p.cols + p.eps);
        T *o = (T *)p.out + row * p.cols;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            int ch = lane + i * 64;
            if (ch < chunks) {
                float ga[VEC], be[VEC], y[VEC];
                VecIO<T>::load((const T *)p.gamma + ch * VEC, ga);
                VecIO<T>::load((const T *)p.beta + ch * VEC, be);
#pragma unroll
                for (int j = 0; j < VEC; ++j) y[j] = (v[i][j] - mean) * inv * ga[j] + be[j];
                VecIO<T>::store(o + ch * VEC, y);
            }
        }
    });
}

// ---- embedding -----------------------------------------------------------------------------
// one wavefront per token, 4 tokens per tile.
template <typename T>
__global__ __launch_bounds__(NT) void embed_kernel(gp_embed_params p, BlpArgs blp) {
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.hidden / VEC;
    tile_loop(blp, [&](TileIdx t) {
        long tok = (long)t.x * 4 + (threadIdx.x >> 6);
        if (tok >= p.tokens) return;
        const int lane = threadIdx.x & 63;
        long id = p.ids[tok];
        if (id < 0) id = 0;
        if (id >= p.vocab) id = p.vocab - 1;  // clamp like relay take(mode="clip")
        const T *e = (const T *)p.tok + id * p.hidden;
        const T *ps = (const T *)p.pos + (tok % p.seq) * p.hidden;
        T *o = (T *)p.out + tok * p.hidden;
        for (int ch = lane; ch < chunks; ch += 64) {
            float a[VEC], b[VEC];
            VecIO<T>::load(e + ch * VEC, a);
            VecIO<T>::load(ps + ch * VEC, b);
#pragma unroll
            for (int j = 0; j < VEC; ++j) a[j] += b[j];
            if (p.seg) {
                VecIO<T>::load((const T *)p.seg + ch * VEC, b);
#pragma unroll
                for (int j = 0; j < VEC; ++j) a[j] += b[j];
            }
            VecIO<T>::store(o + ch * VEC, a);
        }
    });
}

template <class Kernel, class... Args>
static int launch_tiles(Kernel kern, int sx, int sy, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info, Args... args) {
    BlpArgs blp;
    int grid = 0;
    int rc = plan_launch(kern, NT, 0, sx, sy, 1, ctx, &blp, &grid, info);
    if (rc) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), 0, native(s), args..., blp);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

static bool al16(const void *p) { return ((uintptr_t)p & 15) == 0; }
static bool is_float(int dt) { return dt == GP_F32 || dt == GP_F16 || dt == GP_BF16; }
static int vec_of(int dt) { return dt == GP_F32 ? 4 : 8; }

#define GP_BY_DTYPE(dt, EXPR)                                    \
    switch (dt) {                                                \
        case GP_F32: { using T = float; return EXPR; }           \
        case GP_F16: { using T = _Float16; return EXPR; }        \
        case GP_BF16: { using T = __bf16; return EXPR; }         \
    }

}  // namespace gp

using namespace gp;

extern "C" int gp_launch_nchw_to_nhwc(const gp_layout_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->in && p->out, "null layout params");
    GP_REQUIRE(p->N > 0 && p->C > 0 && p->H > 0 && p->W > 0 && p->c_pad >= p->C, "layout shape");
    GP_REQUIRE(is_float(p->dtype_in) && is_float(p->dtype_out), "layout dtype");
    int HW = p->H * p->W, sx = (HW + NT - 1) / NT;
#define L(TI, TO) launch_tiles(nchw_to_nhwc_kernel<TI, TO>, sx, p->N, ctx, s, info, (const TI *)p->in, (TO *)p->out, p->C, HW, p->c_pad)
    if (p->dtype_in == GP_F32 && p->dtype_out == GP_F32) return L(float, float);
    if (p->dtype_in == GP_F32 && p->dtype_out == GP_F16) return L(float, _Float16);
    if (p->dtype_in == GP_F32 && p->dtype_out == GP_BF16) return L(float, __bf16);
    if (p->dtype_in == GP_F16 && p->dtype_out == GP_F16) return L(_Float16, _Float16);
    if (p->dtype_in == GP_BF16 && p->dtype_out == GP_BF16) return L(__bf16, __bf16);
#undef L
    set_error("layout: unsupported dtype pair %d -> %d", p->dtype_in, p->dtype_out);
    return GP_OUTOFRANGE;
}

extern "C" int gp_launch_pool2d(const gp_pool_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->in && p->out, "null pool params");
    GP_REQUIRE(is_float(p->dtype), "pool dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->N > 0 && p->H > 0 && p->W > 0 && p->C > 0 && p->C % vec == 0, "pool: C must be a positive multiple of %d", vec);
    GP_REQUIRE(p->mode >= 0 && p->mode <= 2, "pool mode %d", p->mode);
    GP_REQUIRE(p->in_pix_stride % vec == 0 && p->out_pix_stride % vec == 0 && p->in_pix_stride >= p->C && p->out_pix_stride >= p->C, "pool pixel strides");
    GP_REQUIRE(al16(p->in) && al16(p->out), "pool: 16-byte alignment");
    int Ho = 1, Wo = 1;
    if (p->mode != 2) {
        GP_REQUIRE(p->R > 0 && p->S > 0 && p->stride > 0 && p->pad >= 0, "pool window");
        Ho = (p->H + 2 * p->pad - p->R) / p->stride + 1;
        Wo = (p->W + 2 * p->pad - p->S) / p->stride + 1;
        GP_REQUIRE(Ho > 0 && Wo > 0, "pool: empty output");
    }
    long items = (long)p->N * Ho * Wo * (p->C / vec);
    int sx = (int)((items + NT - 1) / NT);
    GP_BY_DTYPE(p->dtype, launch_tiles(pool_kernel<T>, sx, 1, ctx, s, info, *p, Ho, Wo, items));
    return GP_OUTOFRANGE;
}

extern "C" int gp_launch_eltwise(const gp_eltwise_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->a && p->out, "null eltwise params");
    GP_REQUIRE(is_float(p->dtype), "eltwise dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->rows > 0 && p->cols > 0 && p->cols % vec == 0, "eltwise: cols must be a positive multiple of %d", vec);
    GP_REQUIRE(p->a_stride % vec == 0 && p->out_stride % vec == 0 && (!p->b || p->b_stride % vec == 0), "eltwise strides");
    GP_REQUIRE(al16(p->a) && al16(p->out) && al16(p->b) && al16(p->scale) && al16(p->shift), "eltwise: 16-byte alignment");
    long items = p->rows * (p->cols / vec);
    long tiles = (items + (long)NT * ELT_PER - 1) / ((long)NT * ELT_PER);
    GP_REQUIRE(tiles < (1L << 31), "eltwise: too large");
    GP_BY_DTYPE(p->dtype, launch_tiles(eltwise_kernel<T>, (int)tiles, 1, ctx, s, info, *p, items));
    return GP_OUTOFRANGE;
}

extern "C" int gp_launch_softmax(const gp_softmax_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->x && p->out, "null softmax params");
    GP_REQUIRE(is_float(p->dtype), "softmax dtype %d", p->dtype);
    GP_REQUIRE(p->rows > 0 && p->cols > 0, "softmax shape");
    gp_softmax_params q = *p;
    if (q.scale == 0.f) q.scale = 1.f;
    long tiles = (p->rows + 3) / 4;
    GP_REQUIRE(tiles < (1L << 31), "softmax: too many rows");
    GP_BY_DTYPE(p->dtype, launch_tiles(softmax_kernel<T>, (int)tiles, 1, ctx, s, info, q));
    return GP_OUTOFRANGE;
}

extern "C" int gp_launch_layernorm(const gp_layernorm_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->x && p->out && p->gamma && p->beta, "null layernorm params");
    GP_REQUIRE(is_float(p->dtype), "layernorm dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->rows > 0 && p->cols > 0 && p->cols % vec == 0, "layernorm: cols must be a positive multiple of %d", vec);
    GP_REQUIRE(p->cols <= 64 * vec * 16, "layernorm: at most %d columns", 64 * vec * 16);
    GP_REQUIRE(al16(p->x) && al16(p->out) && al16(p->residual) && al16(p->gamma) && al16(p->beta), "layernorm: 16-byte alignment");
    long tiles = (p->rows + 3) / 4;
    GP_REQUIRE(tiles < (1L << 31), "layernorm: too many rows");
    int chunks_per_lane = (p->cols / vec + 63) / 64;
    if (chunks_per_lane <= 2) { GP_BY_DTYPE(p->dtype, launch_tiles(layernorm_kernel<T, 2>, (int)tiles, 1, ctx, s, info, *p)); }
    else if (chunks_per_lane <= 8) { GP_BY_DTYPE(p->dtype, launch_tiles(layernorm_kernel<T, 8>, (int)tiles, 1, ctx, s, info, *p)); }
    else { GP_BY_DTYPE(p->dtype, launch_tiles(layernorm_kernel<T, 16>, (int)tiles, 1, ctx, s, info, *p)); }
    return GP_OUTOFRANGE;
}

extern "C" int gp_launch_embed(const gp_embed_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->ids && p->tok && p->pos && p->out, "null embed params");
    GP_REQUIRE(is_float(p->dtype), "embed dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->tokens > 0 && p->seq > 0 && p->vocab > 0 && p->hidden > 0 && p->hidden % vec == 0, "embed: hidden must be a positive multiple of %d", vec);
    GP_REQUIRE(al16(p->tok) && al16(p->pos) && al16(p->seg) && al16(p->out), "embed: 16-byte alignment");
    long tiles = (p->tokens + 3) / 4;
    GP_REQUIRE(tiles < (1L << 31), "embed: too many tokens");
    GP_BY_DTYPE(p->dtype, launch_tiles(embed_kernel<T>, (int)tiles, 1, ctx, s, info, *p));
    return GP_OUTOFRANGE;
}
