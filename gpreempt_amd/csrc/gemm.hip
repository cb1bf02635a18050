// Preemptible GEMM and implicit-GEMM convolution on the gfx950 matrix cores.
//
// One workgroup owns one BM x BN output tile for the whole K range and walks K in a fixed
// order with fp32 accumulation, so the value of a tile does not depend on which workgroup or
// which launch computes it: a preempted-then-resumed run is bit-identical to an uninterrupted
// one.  Tiles are handed out by gp::tile_loop (tile_loop.hpp).
//
// Data movement: both operands are staged K-contiguous in LDS ([rows][BK + pad]) with 16-byte
// global loads that are issued one K-step ahead of the MFMAs (register prefetch).  A lane feeds
// v_mfma_f32_32x32x16_{f16,bf16} with one 16-byte LDS read per operand; for fp32 the same
// 16-byte read feeds four v_mfma_f32_32x32x2_f32 (K is consumed in a permuted but fixed order).
//
// The convolution is the same main loop with a gathered A operand: row m is output pixel
// (n, ho, wo) and column k is (r, s, ci) of an NHWC input, zero-filled outside the image.
#include "common.hpp"

namespace gp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ void mma(u32x4 a, u32x4 b, f32x16 &acc) {
        f32x4 fa = __builtin_bit_cast(f32x4, a), fb = __builtin_bit_cast(f32x4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[i], acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f(float v) { return v; }
    static __device__ __forceinline__ float from_f(float v) { return v; }
};
template <> struct Elem<_Float16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void mma(u32x4 a, u32x4 b, f32x16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f(_Float16 v) { return (float)v; }
    static __device__ __forceinline__ _Float16 from_f(float v) { return (_Float16)v; }
};
template <> struct Elem<__bf16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void mma(u32x4 a, u32x4 b, f32x16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f(__bf16 v) { return (float)v; }
    static __device__ __forceinline__ __bf16 from_f(float v) { return (__bf16)v; }
};

__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == GP_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == GP_ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
    return v;
}

struct MatArgs {
    // GEMM view: C[M,N] = A[M,K] * B ; conv fills the conv fields and M = N*Ho*Wo, K = R*S*Cin.
    int M, N, K;
    const void *A; long lda, stride_a, stride_a_outer;
    const void *B; long ldb, stride_b, stride_b_outer;
    void *C; long ldc, stride_c, stride_c_outer;
    const void *bias;
    const void *residual; long ldr;
    float alpha;
    int act;
    int batch_inner;
    // convolution geometry (CONV only)
    int H, W, Cin, S, Ho, Wo, sh, sw, ph, pw;
};

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool CONV, bool B_KN>
struct TileKernel {
    using elem = T;
    static constexpr int bm = BM, bn = BN;
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int NT = WGM * WGN * 64;
    static constexpr int LDK = BK + VEC;           // LDS row stride in elements (16-byte pad)
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int KSTEP = 2 * VEC;          // K consumed per mma() call
    static constexpr int A_CHUNKS = BM * BK / VEC, B_CHUNKS = BN * BK / VEC;
    static constexpr int A_PER = (A_CHUNKS + NT - 1) / NT, B_PER = (B_CHUNKS + NT - 1) / NT;
    static constexpr size_t LDS_BYTES = (size_t)(BM + BN) * LDK * sizeof(T);
    static_assert(BK % KSTEP == 0 && WM % 32 == 0 && WN % 32 == 0, "tile shape");
    static_assert(A_CHUNKS % NT == 0 && B_CHUNKS % NT == 0, "loader shape");

    static __device__ __forceinline__ void run(const MatArgs &g, TileIdx t, T *lds) {
        T *As = lds, *Bs = lds + BM * LDK;
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int wm = wave / WGN, wn = wave % WGN;
        const int l32 = lane & 31, half = lane >> 5;
        const int m0 = t.y * BM, n0 = t.x * BN;
        long offa = 0, offb = 0, offc = 0;
        if (g.batch_inner > 0) {
            int zo = t.z / g.batch_inner, zi = t.z - zo * g.batch_inner;
            offa = zo * g.stride_a_outer + zi * g.stride_a;
            offb = zo * g.stride_b_outer + zi * g.stride_b;
            offc = zo * g.stride_c_outer + zi * g.stride_c;
        } else {
            offa = t.z * g.stride_a; offb = t.z * g.stride_b; offc = t.z * g.stride_c;
        }
        const T *A = (const T *)g.A + offa, *B = (const T *)g.B + offb;

        // Per-thread loader slots: which (row, k-chunk) of the tile each 16-byte load covers.
        constexpr int KC = BK / VEC;  // chunks per tile row
        int a_row[A_PER], a_kc[A_PER];
        long a_base[A_PER];           // GEMM: element offset of the row; CONV: offset of image n
        int a_h0[A_PER], a_w0[A_PER]; // CONV: top-left input coordinate of the pixel's window
        bool a_ok[A_PER];
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            int c = tid + i * NT;
            a_row[i] = c / KC; a_kc[i] = c % KC;
            int m = m0 + a_row[i];
            a_ok[i] = m < g.M;
            if (CONV) {
                int mm = a_ok[i] ? m : 0;
                int n = mm / (g.Ho * g.Wo), rem = mm - n * (g.Ho * g.Wo);
                int ho = rem / g.Wo, wo = rem - ho * g.Wo;
                a_h0[i] = ho * g.sh - g.ph; a_w0[i] = wo * g.sw - g.pw;
                a_base[i] = (long)n * g.H * g.W * g.lda;
            } else {
                a_base[i] = (long)m * g.lda; a_h0[i] = a_w0[i] = 0;
            }
        }
        int b_row[B_PER], b_kc[B_PER];
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            int c = tid + i * NT;
            if (B_KN) { b_row[i] = c / (BN / VEC); b_kc[i] = c % (BN / VEC); }  // row = k, kc = n-chunk
            else { b_row[i] = c / KC; b_kc[i] = c % KC; }
        }

        u32x4 ra[A_PER], rb[B_PER];
        auto load_global = [&](int kt) {
            const int k0 = kt * BK;
#pragma unroll
            for (int i = 0; i < A_PER; ++i) {
                int k = k0 + a_kc[i] * VEC;
                u32x4 v = {0, 0, 0, 0};
                if (a_ok[i] && k < g.K) {
                    if (CONV) {
                        int rs = k / g.Cin, ci = k - rs * g.Cin;
                        int r = rs / g.S, s = rs - r * g.S;
                        int hi = a_h0[i] + r, wi = a_w0[i] + s;
                        if ((unsigned)hi < (unsigned)g.H && (unsigned)wi < (unsigned)g.W)
                            v = *(const u32x4 *)(A + a_base[i] + ((long)hi * g.W + wi) * g.lda + ci);
                    } else {
                        v = *(const u32x4 *)(A + a_base[i] + k);
                    }
                }
                ra[i] = v;
            }
#pragma unroll
            for (int i = 0; i < B_PER; ++i) {
                u32x4 v = {0, 0, 0, 0};
                if (B_KN) {
                    int k = k0 + b_row[i], n = n0 + b_kc[i] * VEC;
                    if (k < g.K && n < g.N) v = *(const u32x4 *)(B + (long)k * g.ldb + n);
                } else {
                    int k = k0 + b_kc[i] * VEC, n = n0 + b_row[i];
                    if (k < g.K && n < g.N) v = *(const u32x4 *)(B + (long)n * g.ldb + k);
                }
                rb[i] = v;
            }
        };
        auto store_lds = [&]() {
#pragma unroll
            for (int i = 0; i < A_PER; ++i) *(u32x4 *)(As + a_row[i] * LDK + a_kc[i] * VEC) = ra[i];
#pragma unroll
            for (int i = 0; i < B_PER; ++i) {
                if (B_KN) {
                    // transpose on the way in: element j of the chunk is B[k][n + j]
                    T tmp[VEC];
                    *(u32x4 *)tmp = rb[i];
#pragma unroll
                    for (int j = 0; j < VEC; ++j) Bs[(b_kc[i] * VEC + j) * LDK + b_row[i]] = tmp[j];
                } else {
                    *(u32x4 *)(Bs + b_row[i] * LDK + b_kc[i] * VEC) = rb[i];
                }
            }
        };

        f32x16 acc[MI][NI];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

        const int KT = (g.K + BK - 1) / BK;
        load_global(0);
        __syncthreads();  // the previous tile of this workgroup may still be reading LDS
        store_lds();
        __syncthreads();
        for (int kt = 0; kt < KT; ++kt) {
            if (kt + 1 < KT) load_global(kt + 1);
#pragma unroll
            for (int ks = 0; ks < BK / KSTEP; ++ks) {
                u32x4 fa[MI], fb[NI];
#pragma unroll
                for (int i = 0; i < MI; ++i)
                    fa[i] = *(const u32x4 *)(As + (wm * WM + i * 32 + l32) * LDK + ks * KSTEP + half * VEC);
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    fb[j] = *(const u32x4 *)(Bs + (wn * WN + j * 32 + l32) * LDK + ks * KSTEP + half * VEC);
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j) Elem<T>::mma(fa[i], fb[j], acc[i][j]);
            }
            if (kt + 1 < KT) {
                __syncthreads();
                store_lds();
                __syncthreads();
            }
        }

        // Epilogue: lane holds column n = l32 and rows 8*(v/4) + 4*half + v%4 of each 32x32 block.
        T *C = (T *)g.C + offc;
        const T *R = g.residual ? (const T *)g.residual + offc : nullptr;
        const T *bias = (const T *)g.bias;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            int n = n0 + wn * WN + j * 32 + l32;
            if (n >= g.N) continue;
            float bv = bias ? Elem<T>::to_f(bias[n]) : 0.f;
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int m = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                    if (m >= g.M) continue;
                    float x = acc[i][j][v] * g.alpha + bv;
                    if (R) x += Elem<T>::to_f(R[(long)m * g.ldr + n]);
                    C[(long)m * g.ldc + n] = Elem<T>::from_f(apply_act(x, g.act));
                }
            }
        }
    }
};

template <class TK>
__global__ __launch_bounds__(TK::NT) void mat_kernel(MatArgs g, BlpArgs blp) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    auto *lds = reinterpret_cast<typename TK::elem *>(lds_raw);
    tile_loop(blp, [&](TileIdx t) { TK::run(g, t, lds); });
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool CONV, bool B_KN>
using TK = TileKernel<T, BM, BN, BK, WGM, WGN, CONV, B_KN>;

template <class K>
static int launch_mat(const MatArgs &g, int batch, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    int sx = (g.N + K::bn - 1) / K::bn, sy = (g.M + K::bm - 1) / K::bm;
    BlpArgs blp;
    int grid = 0;
    auto kern = mat_kernel<K>;
    if (K::LDS_BYTES > 48 * 1024) {
        static bool once = false;  // benign race: idempotent attribute
        if (!once) {
            GP_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)K::LDS_BYTES));
            once = true;
        }
    }
    int rc = plan_launch(kern, K::NT, K::LDS_BYTES, sx, sy, batch, ctx, &blp, &grid, info);
    if (rc) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(K::NT), K::LDS_BYTES, native(s), g, blp);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

// Tile choice: the largest tile that still yields at least one tile per compute unit; small
// problems fall back to 64x64 so that more of the chip takes part.
template <typename T, bool CONV, bool B_KN>
static int dispatch_tile(const MatArgs &g, int batch, int tile_m, int tile_n, const gp_preempt_ctx *ctx,
                         gp_stream s, gp_launch_info *info) {
    constexpr int BK = sizeof(T) == 4 ? 16 : 32;
    long t128 = (long)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
    int tm = tile_m, tn = tile_n;
    if (tm == 0 || tn == 0) {
        if (t128 >= device_cus()) tm = tn = 128; else tm = tn = 64;
    }
    if (tm == 128 && tn == 128) return launch_mat<TK<T, 128, 128, BK, 2, 2, CONV, B_KN>>(g, batch, ctx, s, info);
    if (tm == 64 && tn == 64) return launch_mat<TK<T, 64, 64, BK, 2, 2, CONV, B_KN>>(g, batch, ctx, s, info);
    set_error("unsupported tile %dx%d (supported: 128x128, 64x64)", tm, tn);
    return GP_OUTOFRANGE;
}

template <bool CONV>
static int dispatch_dtype(int dtype, bool b_kn, const MatArgs &g, int batch, int tm, int tn,
                          const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    if (CONV) {
        switch (dtype) {
            case GP_F32: return dispatch_tile<float, true, false>(g, batch, tm, tn, ctx, s, info);
            case GP_F16: return dispatch_tile<_Float16, true, false>(g, batch, tm, tn, ctx, s, info);
            case GP_BF16: return dispatch_tile<__bf16, true, false>(g, batch, tm, tn, ctx, s, info);
        }
    } else if (b_kn) {
        switch (dtype) {
            case GP_F32: return dispatch_tile<float, false, true>(g, batch, tm, tn, ctx, s, info);
            case GP_F16: return dispatch_tile<_Float16, false, true>(g, batch, tm, tn, ctx, s, info);
            case GP_BF16: return dispatch_tile<__bf16, false, true>(g, batch, tm, tn, ctx, s, info);
        }
    } else {
        switch (dtype) {
            case GP_F32: return dispatch_tile<float, false, false>(g, batch, tm, tn, ctx, s, info);
            case GP_F16: return dispatch_tile<_Float16, false, false>(g, batch, tm, tn, ctx, s, info);
            case GP_BF16: return dispatch_tile<__bf16, false, false>(g, batch, tm, tn, ctx, s, info);
        }
    }
    set_error("unsupported dtype %d for matrix kernels", dtype);
    return GP_OUTOFRANGE;
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace gp

using namespace gp;

extern "C" int gp_launch_gemm(const gp_gemm_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p != nullptr, "null gemm params");
    GP_REQUIRE(p->dtype == GP_F32 || p->dtype == GP_F16 || p->dtype == GP_BF16, "gemm dtype %d", p->dtype);
    const int vec = p->dtype == GP_F32 ? 4 : 8;
    GP_REQUIRE(p->M > 0 && p->N > 0 && p->K > 0, "gemm shape %dx%dx%d", p->M, p->N, p->K);
    GP_REQUIRE(p->A && p->B && p->C, "gemm needs A, B and C");
    GP_REQUIRE(p->K % vec == 0 && p->lda % vec == 0 && p->ldb % vec == 0, "gemm: K, lda, ldb must be multiples of %d elements", vec);
    GP_REQUIRE(!p->b_is_nk ? (p->N % vec == 0) : true, "gemm: N must be a multiple of %d when B is K x N", vec);
    GP_REQUIRE(aligned16(p->A) && aligned16(p->B), "gemm: A and B must be 16-byte aligned");
    const int batch = p->batch > 0 ? p->batch : 1;
    if (batch > 1) {
        GP_REQUIRE(p->stride_a % vec == 0 && p->stride_b % vec == 0, "gemm: batch strides of A and B must be multiples of %d elements", vec);
        if (p->batch_inner > 0)
            GP_REQUIRE(p->stride_a_outer % vec == 0 && p->stride_b_outer % vec == 0, "gemm: outer batch strides must be multiples of %d elements", vec);
    }
    GP_REQUIRE(p->lda >= p->K && p->ldc >= p->N && p->ldb >= (p->b_is_nk ? p->K : p->N), "gemm: leading dimension smaller than the row");
    MatArgs g{};
    g.M = p->M; g.N = p->N; g.K = p->K;
    g.A = p->A; g.lda = p->lda; g.stride_a = p->stride_a; g.stride_a_outer = p->stride_a_outer;
    g.B = p->B; g.ldb = p->ldb; g.stride_b = p->stride_b; g.stride_b_outer = p->stride_b_outer;
    g.C = p->C; g.ldc = p->ldc; g.stride_c = p->stride_c; g.stride_c_outer = p->stride_c_outer;
    g.bias = p->bias; g.residual = p->residual; g.ldr = p->ldc;
    g.alpha = p->alpha == 0.f ? 1.f : p->alpha;
    g.act = p->act; g.batch_inner = batch > 1 ? p->batch_inner : 0;
    return dispatch_dtype<false>(p->dtype, !p->b_is_nk, g, batch, p->tile_m, p->tile_n, ctx, s, info);
}

extern "C" int gp_launch_conv2d(const gp_conv_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p != nullptr, "null conv params");
    GP_REQUIRE(p->dtype == GP_F32 || p->dtype == GP_F16 || p->dtype == GP_BF16, "conv dtype %d", p->dtype);
    const int vec = p->dtype == GP_F32 ? 4 : 8;
    GP_REQUIRE(p->N > 0 && p->H > 0 && p->W > 0 && p->Cin > 0 && p->Cout > 0 && p->R > 0 && p->S > 0, "conv shape");
    GP_REQUIRE(p->stride_h > 0 && p->stride_w > 0 && p->pad_h >= 0 && p->pad_w >= 0, "conv stride/pad");
    GP_REQUIRE(p->Cin % vec == 0, "conv: Cin must be a multiple of %d (pad the channels)", vec);
    GP_REQUIRE(p->in && p->weight && p->out, "conv needs in, weight and out");
    GP_REQUIRE(p->in_pix_stride >= p->Cin && p->in_pix_stride % vec == 0, "conv: input pixel stride");
    GP_REQUIRE(p->out_pix_stride >= p->Cout, "conv: output pixel stride");
    GP_REQUIRE(aligned16(p->in) && aligned16(p->weight), "conv: in and weight must be 16-byte aligned");
    int Ho = (p->H + 2 * p->pad_h - p->R) / p->stride_h + 1, Wo = (p->W + 2 * p->pad_w - p->S) / p->stride_w + 1;
    GP_REQUIRE(Ho > 0 && Wo > 0, "conv: empty output");
    long M = (long)p->N * Ho * Wo;
    GP_REQUIRE(M < (1L << 31), "conv: too many output pixels");
    MatArgs g{};
    g.M = (int)M; g.N = p->Cout; g.K = p->R * p->S * p->Cin;
    g.A = p->in; g.lda = p->in_pix_stride;
    g.B = p->weight; g.ldb = g.K;
    g.C = p->out; g.ldc = p->out_pix_stride;
    g.bias = p->bias; g.residual = p->residual; g.ldr = p->residual ? p->res_pix_stride : 0;
    GP_REQUIRE(!p->residual || p->res_pix_stride >= p->Cout, "conv: residual pixel stride");
    g.alpha = 1.f; g.act = p->act; g.batch_inner = 0;
    g.H = p->H; g.W = p->W; g.Cin = p->Cin; g.S = p->S; g.Ho = Ho; g.Wo = Wo;
    g.sh = p->stride_h; g.sw = p->stride_w; g.ph = p->pad_h; g.pw = p->pad_w;
    return dispatch_dtype<true>(p->dtype, false, g, 1, p->tile_m, p->tile_n, ctx, s, info);
}
