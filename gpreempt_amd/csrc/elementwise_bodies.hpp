// Tile bodies of the memory-bound operators: layout change, pooling, elementwise, softmax,
// layer-norm, embedding, copy.  All are HBM-bound, so each thread moves 16 bytes per access,
// consecutive lanes touch consecutive 16-byte chunks (coalesced wave64 accesses), arithmetic is
// fp32, and row reductions stay inside one wavefront (cross-lane shuffles, no LDS round trip).
// Each body processes one tile; the stand-alone kernels below and the whole-model program kernel
// hand tiles to them, so every operator can be stopped at a tile boundary and resumed without
// redoing or skipping a tile.
#pragma once
#include "common.hpp"
#include "out_store.hpp"
#include "mma.hpp"

namespace gp {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// A float that the compiler must materialise as such.  Conversions to fp16 go through it: otherwise
// the compiler may fold "multiply-add, then convert" into one v_fma_mixlo_f16, which rounds once
// where the two instructions round twice, and it decides that per instantiation: the same row
// would get different bits from two forms of one kernel.
__device__ __forceinline__ float pin_f32(float v) {
    asm("" : "+v"(v));
    return v;
}

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
        st_out128(p, __builtin_bit_cast(out_u32x4, v));
    }
    static __device__ __forceinline__ void unpack(out_u32x4 r, float (&f)[4]) {
        f32x4 v = __builtin_bit_cast(f32x4, r);
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = v[i];
    }
    static __device__ __forceinline__ out_u32x4 pack(const float (&f)[4]) {
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = f[i];
        return __builtin_bit_cast(out_u32x4, v);
    }
    static __device__ __forceinline__ float ld1(const float *p) { return *p; }
    static __device__ __forceinline__ void st1(float *p, float v) { st_elem<float>(p, v); }
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
        for (int i = 0; i < 8; ++i) v[i] = (_Float16)pin_f32(f[i]);
        st_out128(p, __builtin_bit_cast(out_u32x4, v));
    }
    static __device__ __forceinline__ void unpack(out_u32x4 r, float (&f)[8]) {
        f16x8 v = __builtin_bit_cast(f16x8, r);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
    }
    static __device__ __forceinline__ out_u32x4 pack(const float (&f)[8]) {
        f16x8 v;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (_Float16)pin_f32(f[i]);
        return __builtin_bit_cast(out_u32x4, v);
    }
    static __device__ __forceinline__ float ld1(const _Float16 *p) { return (float)*p; }
    static __device__ __forceinline__ void st1(_Float16 *p, float v) { st_elem<_Float16>(p, (_Float16)pin_f32(v)); }
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
        st_out128(p, __builtin_bit_cast(out_u32x4, v));
    }
    static __device__ __forceinline__ void unpack(out_u32x4 r, float (&f)[8]) {
        bf16x8 v = __builtin_bit_cast(bf16x8, r);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
    }
    static __device__ __forceinline__ out_u32x4 pack(const float (&f)[8]) {
        bf16x8 v;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (__bf16)f[i];
        return __builtin_bit_cast(out_u32x4, v);
    }
    static __device__ __forceinline__ float ld1(const __bf16 *p) { return (float)*p; }
    static __device__ __forceinline__ void st1(__bf16 *p, float v) { st_elem<__bf16>(p, (__bf16)v); }
};

// A tensor that cannot stay in the 256 MiB last-level cache is streamed: its loads and stores carry
// the nontemporal hint, so that lines nobody will read again do not push out ones that somebody will.
// Measured on 384 MiB buffers: copy 5.6 -> 6.2 TB/s, add (two reads, one write) 5.5 -> 6.3 TB/s.
constexpr long kStreamBytes = 256L << 20;
template <bool NTH> __device__ __forceinline__ out_u32x4 ld_raw128(const void *p) {
    if (NTH) return __builtin_nontemporal_load((const out_u32x4 *)p);
    return *(const out_u32x4 *)p;
}
template <bool NTH> __device__ __forceinline__ void st_raw128(void *p, out_u32x4 v) {
    if (NTH && !kCoherentStores) __builtin_nontemporal_store(v, (out_u32x4 *)p);
    else st_out128(p, v);
}

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
struct LayoutArgs { const void *in_; void *out_; int C, HW, c_pad; };
template <typename TI, typename TO>
__device__ __forceinline__ void layout_tile(const LayoutArgs &a, TileIdx t) {
    const TI *in = (const TI *)a.in_;
    TO *out = (TO *)a.out_;
    const int C = a.C, HW = a.HW, c_pad = a.c_pad;
    
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
}
// (LOOP: which dispatcher form the instantiation is built around, tile_loop.hpp)
template <typename TI, typename TO, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void nchw_to_nhwc_kernel(LayoutArgs a, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { layout_tile<TI, TO>(a, t); });
}

// ---- pooling, NHWC -------------------------------------------------------------------------
// item = (output pixel, 16-byte channel chunk); tile = 256 items.
// block2: a 3 x 3 / stride 2 max pool, an item is a 2 x 2 block of output pixels (one 16-byte channel
// chunk): its four windows overlap in a 5 x 5 input patch, 25 loads instead of 36.  The kernel is
// bound by the number of load requests (every input element is wanted by up to four windows), so
// fewer requests per output is what makes it faster: 2.7 -> 3.5 TB/s from issuing all taps without
// branches between them, and on to the figure in the profile with the shared patch.
struct PoolArgs { gp_pool_params p; int Ho, Wo; long items; int block2; };

// element-wise maximum of two 16-byte chunks, in the storage type (a maximum needs no wider arithmetic)
template <typename T> __device__ __forceinline__ u32x4 chunk_max(u32x4 a, u32x4 b);
template <> __device__ __forceinline__ u32x4 chunk_max<float>(u32x4 a, u32x4 b) {
    return __builtin_bit_cast(u32x4, __builtin_elementwise_max(__builtin_bit_cast(f32x4, a), __builtin_bit_cast(f32x4, b)));
}
template <> __device__ __forceinline__ u32x4 chunk_max<_Float16>(u32x4 a, u32x4 b) {
    return __builtin_bit_cast(u32x4, __builtin_elementwise_max(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b)));
}
template <> __device__ __forceinline__ u32x4 chunk_max<__bf16>(u32x4 a, u32x4 b) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // a bf16 is the upper half of a float
        const float al = __builtin_bit_cast(float, a[i] << 16), bl = __builtin_bit_cast(float, b[i] << 16);
        const float ah = __builtin_bit_cast(float, a[i] & 0xFFFF0000u), bh = __builtin_bit_cast(float, b[i] & 0xFFFF0000u);
        o[i] = (__builtin_bit_cast(unsigned, fmaxf(al, bl)) >> 16) | (__builtin_bit_cast(unsigned, fmaxf(ah, bh)) & 0xFFFF0000u);
    }
    return o;
}

// (max pooling only.  A tap outside the image is fetched from the clamped coordinate instead: that
// element lies inside the same window, so the maximum is unchanged and nothing has to be masked.)
template <typename T>
__device__ __forceinline__ void pool_tile_block2(const PoolArgs &a, TileIdx t) {
    const gp_pool_params &p = a.p;
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.C / VEC;
    const int Hb = (a.Ho + 1) / 2, Wb = (a.Wo + 1) / 2;
    const unsigned item = (unsigned)t.x * NT + threadIdx.x;
    if (item >= (unsigned)a.items) return;
    const unsigned ublk = item / (unsigned)chunks;
    const int ch = (int)(item - ublk * (unsigned)chunks);
    const unsigned q = ublk / (unsigned)Wb;
    const int wb = (int)(ublk - q * (unsigned)Wb);
    const long n = q / (unsigned)Hb;
    const int hb = (int)(q - (unsigned)n * (unsigned)Hb);
    const T *in = (const T *)p.in;
    T *out = (T *)p.out;
    const int h_first = hb * 4 - p.pad, w_first = wb * 4 - p.pad;  // input coordinate of the patch's corner
    u32x4 f[25];
#pragma unroll
    for (int r = 0; r < 5; ++r) {
#pragma unroll
        for (int s = 0; s < 5; ++s) {
            const int hi = h_first + r, wi = w_first + s;
            const int hc = hi < 0 ? 0 : (hi >= p.H ? p.H - 1 : hi), wc = wi < 0 ? 0 : (wi >= p.W ? p.W - 1 : wi);
            f[r * 5 + s] = *(const u32x4 *)(in + ((n * p.H + hc) * p.W + wc) * p.in_pix_stride + ch * VEC);
        }
    }
    // column maxima of the three row triples a window can take, then the windows
#pragma unroll
    for (int dy = 0; dy < 2; ++dy) {
        const int ho = hb * 2 + dy;
        if (ho >= a.Ho) continue;
        u32x4 col[5];
#pragma unroll
        for (int s = 0; s < 5; ++s) col[s] = chunk_max<T>(chunk_max<T>(f[(dy * 2) * 5 + s], f[(dy * 2 + 1) * 5 + s]), f[(dy * 2 + 2) * 5 + s]);
#pragma unroll
        for (int dx = 0; dx < 2; ++dx) {
            const int wo = wb * 2 + dx;
            if (wo >= a.Wo) continue;
            const u32x4 m = chunk_max<T>(chunk_max<T>(col[dx * 2], col[dx * 2 + 1]), col[dx * 2 + 2]);
            st_out128(out + ((n * a.Ho + ho) * a.Wo + wo) * p.out_pix_stride + ch * VEC, __builtin_bit_cast(out_u32x4, m));
        }
    }
}

template <typename T>
__device__ __forceinline__ void pool_tile(const PoolArgs &a, TileIdx t) {
    if (a.block2) { pool_tile_block2<T>(a, t); return; }
    const gp_pool_params &p = a.p;
    const int Ho = a.Ho, Wo = a.Wo;
    const long items = a.items;
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.C / VEC;
    
        // 32-bit index arithmetic (the planner bounds the item count): a 64-bit division is a
        // subroutine of a hundred instructions, and five of them per item made this kernel ALU-bound
        const unsigned item = (unsigned)t.x * NT + threadIdx.x;
        if (item >= (unsigned)items) return;
        const unsigned upix = item / (unsigned)chunks;
        const int ch = (int)(item - upix * (unsigned)chunks);
        const long pix = upix;
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
        const unsigned q = upix / (unsigned)Wo;
        const int wo = (int)(upix - q * (unsigned)Wo);
        const long n = q / (unsigned)Ho;
        const int ho = (int)(q - (unsigned)n * (unsigned)Ho);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = p.mode == 0 ? -INFINITY : 0.f;
        int cnt = 0;
        // The usual windows are unrolled so that all their loads are in flight together; with the
        // window size known only at run time every tap would wait for the one before.
        auto window = [&](auto RC, auto SC) {
            constexpr int R = decltype(RC)::value, S = decltype(SC)::value;
            float f[R * S][VEC];
            bool in_range[R * S];
            // every tap is loaded, from a clamped coordinate when it lies outside the image, and
            // dropped afterwards: no branch sits between the loads, so all R*S are in flight at once
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int s = 0; s < S; ++s) {
                    const int hi = ho * p.stride - p.pad + r, wi = wo * p.stride - p.pad + s;
                    in_range[r * S + s] = (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W;
                    const int hc = hi < 0 ? 0 : (hi >= p.H ? p.H - 1 : hi), wc = wi < 0 ? 0 : (wi >= p.W ? p.W - 1 : wi);
                    VecIO<T>::load(in + ((n * p.H + hc) * p.W + wc) * p.in_pix_stride + ch * VEC, f[r * S + s]);
                }
            }
#pragma unroll
            for (int i = 0; i < R * S; ++i) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float v = in_range[i] ? f[i][j] : (p.mode == 0 ? -INFINITY : 0.f);
                    acc[j] = p.mode == 0 ? fmaxf(acc[j], v) : acc[j] + v;
                }
                cnt += in_range[i];
            }
        };
        if (p.R == 3 && p.S == 3) window(IntC<3>{}, IntC<3>{});
        else if (p.R == 2 && p.S == 2) window(IntC<2>{}, IntC<2>{});
        else
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
        if (p.mode == 1 || p.mode == 3) {
            if (p.mode == 3) cnt = p.R * p.S;  // padding counts as zeros
            float inv = 1.f / (float)(cnt > 0 ? cnt : 1);
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] *= inv;
        }
        VecIO<T>::store(out + pix * p.out_pix_stride + ch * VEC, acc);
}
template <typename T, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void pool_kernel(PoolArgs a, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { pool_tile<T>(a, t); });
}

// ---- elementwise ---------------------------------------------------------------------------
// item = (row, 16-byte chunk); tile = 1024 items (4 per thread, strided by 256 for coalescing).
constexpr int ELT_PER = 4;
struct EltwiseArgs { gp_eltwise_params p; long items; int stream; };
template <typename T>
__device__ __forceinline__ void eltwise_finish(const gp_eltwise_params &p, int ch, float (&a)[VecIO<T>::VEC]) {
    constexpr int VEC = VecIO<T>::VEC;
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
}
// A tile whose 1024 items all exist: no bounds checks, so every load of the tile is in flight
// before the first value is needed (with the checks the compiler serialises the four items).
template <typename T, bool NTH>
__device__ __forceinline__ void eltwise_full_tile(const EltwiseArgs &a, unsigned base) {
    const gp_eltwise_params &p = a.p;
    constexpr int VEC = VecIO<T>::VEC;
    const unsigned chunks = (unsigned)(p.cols / VEC);
    long row[ELT_PER];
    int ch[ELT_PER];
    out_u32x4 ra[ELT_PER], rb[ELT_PER];
#pragma unroll
    for (int u = 0; u < ELT_PER; ++u) {
        const unsigned item = base + u * NT + threadIdx.x;
        const unsigned urow = item / chunks;
        ch[u] = (int)(item - urow * chunks);
        row[u] = urow;
        ra[u] = ld_raw128<NTH>((const T *)p.a + row[u] * p.a_stride + ch[u] * VEC);
    }
    if (p.b) {
#pragma unroll
        for (int u = 0; u < ELT_PER; ++u) rb[u] = ld_raw128<NTH>((const T *)p.b + row[u] * p.b_stride + ch[u] * VEC);
    }
#pragma unroll
    for (int u = 0; u < ELT_PER; ++u) {
        float x[VEC];
        VecIO<T>::unpack(ra[u], x);
        if (p.b) {
            float y[VEC];
            VecIO<T>::unpack(rb[u], y);
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[j] += y[j];
        }
        eltwise_finish<T>(p, ch[u], x);
        st_raw128<NTH>((T *)p.out + row[u] * p.out_stride + ch[u] * VEC, VecIO<T>::pack(x));
    }
}
template <typename T>
__device__ __forceinline__ void eltwise_tile(const EltwiseArgs &a, TileIdx t) {
    const gp_eltwise_params &p = a.p;
    const long items = a.items;
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.cols / VEC;
    const unsigned base = (unsigned)t.x * ELT_PER * NT;  // 32-bit: see pool_tile
    if ((long)base + ELT_PER * NT <= items) {
        if (a.stream) eltwise_full_tile<T, true>(a, base);
        else eltwise_full_tile<T, false>(a, base);
        return;
    }
#pragma unroll
    for (int u = 0; u < ELT_PER; ++u) {
        const unsigned item = base + u * NT + threadIdx.x;
        if (item >= (unsigned)items) continue;
        const unsigned urow = item / (unsigned)chunks;
        const int ch = (int)(item - urow * (unsigned)chunks);
        const long row = urow;
        float x[VEC];
        VecIO<T>::load((const T *)p.a + row * p.a_stride + ch * VEC, x);
        if (p.b) {
            float y[VEC];
            VecIO<T>::load((const T *)p.b + row * p.b_stride + ch * VEC, y);
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[j] += y[j];
        }
        eltwise_finish<T>(p, ch, x);
        VecIO<T>::store((T *)p.out + row * p.out_stride + ch * VEC, x);
    }
}
template <typename T, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void eltwise_kernel(EltwiseArgs a, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { eltwise_tile<T>(a, t); });
}

// ---- softmax -------------------------------------------------------------------------------
// A row is held in registers by G lanes (16-byte chunks, C per lane): one read and one write per
// element, reductions by xor-shuffles inside the lane group.  Short rows share a wavefront: with
// G = 16 a wave handles 4 rows at once (BERT's 128-wide score rows are 16 chunks of fp16).
// Rows whose length is not a multiple of the chunk, or longer than 256 chunks, take the scalar path.
__host__ __device__ inline int softmax_group(int cols, int vec) {  // lanes per row; 0 = scalar path
    if (cols % vec) return 0;
    const int chunks = cols / vec;
    return chunks <= 16 ? 16 : chunks <= 256 ? 64 : 0;
}
// lane groups of a large problem take RPW rows each at a time: with one 16-byte load per lane and row
// a wavefront has 1 KB in flight, too little to keep HBM busy
__host__ __device__ inline int softmax_rows_per_group(int cols, int vec, long rows) {
    return softmax_group(cols, vec) == 16 && rows >= 65536 ? 4 : 1;
}
__host__ __device__ inline int softmax_rows_per_tile(int cols, int vec, long rows) {
    const int g = softmax_group(cols, vec);
    return g ? 4 * (64 / g) * softmax_rows_per_group(cols, vec, rows) : 4;
}

template <typename T, int G, int C, bool NTH, int RPW = 1>
__device__ __forceinline__ void softmax_rows_grouped(const gp_softmax_params &p, TileIdx t) {
    constexpr int VEC = VecIO<T>::VEC;
    const int lane = threadIdx.x & 63, sub = lane % G;
    const int chunks = p.cols / VEC;
    out_u32x4 raw[RPW][C];
    long rowq[RPW];
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
        rowq[q] = (((long)t.x * 4 + (threadIdx.x >> 6)) * RPW + q) * (64 / G) + lane / G;
        const T *x = (const T *)p.x + (rowq[q] < p.rows ? rowq[q] : 0) * p.cols;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            const int ch = sub + i * G;
            if (rowq[q] < p.rows && ch < chunks) raw[q][i] = ld_raw128<NTH>(x + ch * VEC);
        }
    }
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
        const bool live = rowq[q] < p.rows;
        float v[C][VEC];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            const int ch = sub + i * G;
            if (live && ch < chunks) {
                VecIO<T>::unpack(raw[q][i], v[i]);
#pragma unroll
                for (int j = 0; j < VEC; ++j) { v[i][j] *= p.scale; mx = fmaxf(mx, v[i][j]); }
            }
        }
#pragma unroll
        for (int o = G / 2; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            const int ch = sub + i * G;
            if (live && ch < chunks) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) { v[i][j] = __expf(v[i][j] - mx); sum += v[i][j]; }
            }
        }
#pragma unroll
        for (int o = G / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        const float inv = 1.f / sum;
        T *out = (T *)p.out + (live ? rowq[q] : 0) * p.cols;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            const int ch = sub + i * G;
            if (live && ch < chunks) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[i][j] *= inv;
                st_raw128<NTH>(out + ch * VEC, VecIO<T>::pack(v[i]));
            }
        }
    }
}

template <typename T>
__device__ __forceinline__ void softmax_tile(const gp_softmax_params &p, TileIdx t) {
    constexpr int VEC = VecIO<T>::VEC;
    const int g = softmax_group(p.cols, VEC);  // uniform
    const bool stream = p.rows * (long)p.cols * (long)sizeof(T) * 2 > kStreamBytes;  // uniform
    if (g == 16) {
        if (softmax_rows_per_group(p.cols, VEC, p.rows) == 4) {
            if (stream) softmax_rows_grouped<T, 16, 1, true, 4>(p, t);
            else softmax_rows_grouped<T, 16, 1, false, 4>(p, t);
        } else {
            softmax_rows_grouped<T, 16, 1, false>(p, t);
        }
        return;
    }
    if (g == 64) {
        if (p.cols / VEC <= 64) softmax_rows_grouped<T, 64, 1, false>(p, t);
        else softmax_rows_grouped<T, 64, 4, false>(p, t);
        return;
    }
    // scalar path: one wavefront per row, 4 rows per tile; lane i reads elements i, i+64, ...
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
}
template <typename T, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void softmax_kernel(gp_softmax_params p, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { softmax_tile<T>(p, t); });
}

// ---- layer norm ----------------------------------------------------------------------------
// one wavefront per RPW rows, 4 * RPW rows per tile; the rows (plus residual) are kept in registers
// (up to MAXC 16-byte chunks per lane and row), so HBM sees one read and one write per element.
// R rows, each held by one wavefront as 16-byte chunks lane, lane + 64, ...: mean, variance and the
// normalised, packed rows.  The rows go through every step side by side, so that the cross-lane
// reductions of one row hide behind those of the others; a row's own arithmetic is the same whatever R
// is, and every kernel that normalises rows goes through this function, so that a row gets the same
// bits wherever it is computed.
// Sum over the 64 lanes, every lane getting the total.  The first four steps (partners 1, 2, 4 and 8 lanes
// apart, inside a row of 16) are DPP moves, which run in the vector ALU; only the last two cross rows
// and go through the LDS crossbar.  (Six crossbar shuffles per sum, from the sixteen wavefronts of a
// workgroup that all normalise rows, made the layer-norm prologue of gemm_ln.hpp wait for the LDS pipe.)
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int R>
__device__ __forceinline__ void wave_sum_rows(float (&s)[R]) {
    // quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror: after each step the lanes of a
    // group of 2, 4, 8, 16 hold the group's sum (a mirror pairs lane i with lane 7 - i or 15 - i, whose
    // groups differ in the bit that the step adds)
#pragma unroll
    for (int q = 0; q < R; ++q) s[q] += dpp_mov<0xB1>(s[q]);
#pragma unroll
    for (int q = 0; q < R; ++q) s[q] += dpp_mov<0x4E>(s[q]);
#pragma unroll
    for (int q = 0; q < R; ++q) s[q] += dpp_mov<0x141>(s[q]);
#pragma unroll
    for (int q = 0; q < R; ++q) s[q] += dpp_mov<0x140>(s[q]);
#pragma unroll
    for (int o = 16; o <= 32; o <<= 1) {
        float t[R];
#pragma unroll
        for (int q = 0; q < R; ++q) t[q] = __shfl_xor(s[q], o, 64);
#pragma unroll
        for (int q = 0; q < R; ++q) s[q] += t[q];
    }
}
// PRE: gamma and beta come as the lane's raw chunks (chunk lane + 64 i in slot i), fetched by the caller when
// it suits it; otherwise they are read here, chunk by chunk (long rows: no registers to spare for them).
template <typename T, int MAXC, int R, bool PRE>
__device__ __forceinline__ void ln_rows_math(const float (&v)[R][MAXC][VecIO<T>::VEC], int chunks, int lane, int cols, float eps,
                                             const T *gamma_p, const T *beta_p, const out_u32x4 (&gamma)[PRE ? MAXC : 1],
                                             const out_u32x4 (&beta)[PRE ? MAXC : 1], out_u32x4 (&y)[R][MAXC]) {
    constexpr int VEC = VecIO<T>::VEC;
    float sum[R], mean[R], sq[R], inv[R];
#pragma unroll
    for (int q = 0; q < R; ++q) {
        sum[q] = 0.f;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int ch = lane + i * 64;
            if (ch < chunks) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) sum[q] += v[q][i][j];
            }
        }
    }
    wave_sum_rows<R>(sum);
#pragma unroll
    for (int q = 0; q < R; ++q) {
        mean[q] = sum[q] / (float)cols;
        sq[q] = 0.f;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int ch = lane + i * 64;
            if (ch < chunks) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) { float d = v[q][i][j] - mean[q]; sq[q] += d * d; }
            }
        }
    }
    wave_sum_rows<R>(sq);
#pragma unroll
    for (int q = 0; q < R; ++q) inv[q] = rsqrtf(sq[q] / (float)cols + eps);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int ch = lane + i * 64;
        if (ch < chunks) {
            float ga[VEC], be[VEC];
            if constexpr (PRE) {
                VecIO<T>::unpack(gamma[i], ga);
                VecIO<T>::unpack(beta[i], be);
            } else {
                VecIO<T>::load(gamma_p + ch * VEC, ga);
                VecIO<T>::load(beta_p + ch * VEC, be);
            }
#pragma unroll
            for (int q = 0; q < R; ++q) {
                float o[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) o[j] = (v[q][i][j] - mean[q]) * inv[q] * ga[j] + be[j];
                y[q][i] = VecIO<T>::pack(o);
            }
        }
    }
}
// All loads of the wavefront's rows are issued before the first reduction.
constexpr int kLnTwoRows = 0x100;  // flag in the plan's `sub`: RPW = 2
template <typename T, int MAXC, int RPW, bool NTH>
__device__ __forceinline__ void layernorm_rows(const gp_layernorm_params &p, TileIdx t) {
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.cols / VEC;
    const int lane = threadIdx.x & 63;
    const long row0 = ((long)t.x * 4 + (threadIdx.x >> 6)) * RPW;
    if (row0 >= p.rows) return;
    constexpr bool PRE = MAXC <= 2;  // short rows: gamma and beta are fetched with the row
    out_u32x4 rx[RPW][MAXC], rr[RPW][MAXC], graw[PRE ? MAXC : 1], braw[PRE ? MAXC : 1];
    if constexpr (PRE) {
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int ch = lane + i * 64;
            graw[i] = braw[i] = out_u32x4{0, 0, 0, 0};
            if (ch < chunks) {
                graw[i] = *(const out_u32x4 *)((const T *)p.gamma + ch * VEC);
                braw[i] = *(const out_u32x4 *)((const T *)p.beta + ch * VEC);
            }
        }
    }
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
        const long row = row0 + q < p.rows ? row0 + q : row0;  // a missing second row re-reads the first and is not stored
        const T *x = (const T *)p.x + row * p.cols;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int ch = lane + i * 64;
            if (ch < chunks) rx[q][i] = ld_raw128<NTH>(x + ch * VEC);
        }
        if (p.residual) {
            const T *r = (const T *)p.residual + row * p.cols;
#pragma unroll
            for (int i = 0; i < MAXC; ++i) {
                const int ch = lane + i * 64;
                if (ch < chunks) rr[q][i] = ld_raw128<NTH>(r + ch * VEC);
            }
        }
    }
    float v[RPW][MAXC][VEC];
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int ch = lane + i * 64;
            if (ch < chunks) {
                VecIO<T>::unpack(rx[q][i], v[q][i]);
                if (p.residual) {
                    float r[VEC];
                    VecIO<T>::unpack(rr[q][i], r);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) v[q][i][j] += r[j];
                }
            }
        }
    }
    out_u32x4 y[RPW][MAXC];
    ln_rows_math<T, MAXC, RPW, PRE>(v, chunks, lane, p.cols, p.eps, (const T *)p.gamma, (const T *)p.beta, graw, braw, y);
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
        if (row0 + q >= p.rows) break;
        T *o = (T *)p.out + (row0 + q) * p.cols;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int ch = lane + i * 64;
            if (ch < chunks) st_raw128<NTH>(o + ch * VEC, y[q][i]);
        }
    }
}
template <typename T, int MAXC, int RPW = 1>
__device__ __forceinline__ void layernorm_tile(const gp_layernorm_params &p, TileIdx t) {
    const bool stream = p.rows * (long)p.cols * (long)sizeof(T) * (p.residual ? 3 : 2) > kStreamBytes;  // uniform
    if (stream) layernorm_rows<T, MAXC, RPW, true>(p, t);
    else layernorm_rows<T, MAXC, RPW, false>(p, t);
}
template <typename T, int MAXC, int RPW = 1, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void layernorm_kernel(gp_layernorm_params p, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { layernorm_tile<T, MAXC, RPW>(p, t); });
}

// ---- embedding -----------------------------------------------------------------------------
// one wavefront per token, 4 tokens per tile.
template <typename T>
__device__ __forceinline__ void embed_tile(const gp_embed_params &p, TileIdx t) {
    constexpr int VEC = VecIO<T>::VEC;
    const int chunks = p.hidden / VEC;
    
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
}
template <typename T, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void embed_kernel(gp_embed_params p, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { embed_tile<T>(p, t); });
}


// ---- copy ----------------------------------------------------------------------------------
// The reference's "nop" kernel (a device-to-device copy, src/executor.cpp:139-146) as a tiled
// operator: tile = 4096 bytes x 4 per thread.
struct CopyArgs { const void *src; void *dst; long bytes; };
constexpr int COPY_TILE_BYTES = NT * 16 * 4;
__device__ __forceinline__ void copy_tile(const CopyArgs &a, TileIdx t) {
    const char *s = (const char *)a.src;
    char *d = (char *)a.dst;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        long off = ((long)t.x * 4 + u) * NT * 16 + (long)threadIdx.x * 16;
        if (off + 16 <= a.bytes) st_out128(d + off, *(const u32x4 *)(s + off));
        else for (long i = off; i < a.bytes; ++i) st_out8(d + i, (unsigned char)s[i]);
    }
}
template <int UNUSED = 0, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(NT) void copy_kernel(CopyArgs a, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { copy_tile(a, t); });
}

}  // namespace gp
