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
#include "gemm_tile.hpp"
#include "gemm_pipe.hpp"

namespace gp {

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

enum { VAR_AUTO = 0, VAR_STAGED = 1, VAR_PIPE = 2, VAR_PIPE_SPLITK = 3 };

template <typename T, bool CONV, bool B_KN>
static int dispatch_staged(const MatArgs &g, int batch, int tm, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    constexpr int BK = sizeof(T) == 4 ? 16 : 32;
    if (tm == 128) return launch_mat<TK<T, 128, 128, BK, 2, 2, CONV, B_KN>>(g, batch, ctx, s, info);
    if (tm == 64) return launch_mat<TK<T, 64, 64, BK, 2, 2, CONV, B_KN>>(g, batch, ctx, s, info);
    set_error("unsupported tile %d for the register-staged kernel (128, 64)", tm);
    return GP_OUTOFRANGE;
}

template <typename T, bool CONV>
static int dispatch_pipe(const MatArgs &g, int batch, int tm, bool splitk, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    if (!splitk) {
        if (tm == 128) return launch_mat<PipeKernel<T, 128, 128, 3, CONV, false>>(g, batch, ctx, s, info);
        if (tm == 64) return launch_mat<PipeKernel<T, 64, 64, 4, CONV, false>>(g, batch, ctx, s, info);
    } else {
        if (tm == 64) return launch_mat<PipeKernel<T, 64, 64, 4, CONV, true>>(g, batch, ctx, s, info);
        if (tm == 32) return launch_mat<PipeKernel<T, 32, 32, 4, CONV, true>>(g, batch, ctx, s, info);
    }
    set_error("unsupported tile %d for the pipelined kernel%s", tm, splitk ? " with split K (64, 32)" : " (128, 64)");
    return GP_OUTOFRANGE;
}

// Kernel and tile choice.  B stored K x N needs the transposing, register-staged kernel.
// Otherwise the pipelined kernel is used with the largest tile that still gives every compute
// unit work; problems too small for that split K across the waves of a workgroup so that the
// serial K loop shrinks instead.
template <typename T, bool CONV>
static int dispatch_any(bool b_kn, const MatArgs &g, int batch, int tile, int variant, const gp_preempt_ctx *ctx,
                        gp_stream s, gp_launch_info *info) {
    auto tiles = [&](int t) { return (long)((g.M + t - 1) / t) * ((g.N + t - 1) / t) * batch; };
    const long cus = device_cus();
    if (b_kn || variant == VAR_STAGED) {
        int tm = tile ? tile : (tiles(128) >= cus ? 128 : 64);
        if (CONV) return dispatch_staged<T, CONV, false>(g, batch, tm, ctx, s, info);
        return b_kn ? dispatch_staged<T, false, true>(g, batch, tm, ctx, s, info) : dispatch_staged<T, false, false>(g, batch, tm, ctx, s, info);
    }
    if (variant == VAR_PIPE) return dispatch_pipe<T, CONV>(g, batch, tile ? tile : (tiles(128) >= cus ? 128 : 64), false, ctx, s, info);
    if (variant == VAR_PIPE_SPLITK) return dispatch_pipe<T, CONV>(g, batch, tile ? tile : (tiles(64) >= cus / 2 ? 64 : 32), true, ctx, s, info);
    if (tile == 128 || (tile == 0 && tiles(128) >= cus)) return dispatch_pipe<T, CONV>(g, batch, 128, false, ctx, s, info);
    if (tile == 64 || (tile == 0 && (tiles(64) >= cus || g.K < 512))) return dispatch_pipe<T, CONV>(g, batch, 64, false, ctx, s, info);
    if (tile == 0 && tiles(64) >= cus / 2) return dispatch_pipe<T, CONV>(g, batch, 64, true, ctx, s, info);
    return dispatch_pipe<T, CONV>(g, batch, 32, true, ctx, s, info);
}

template <bool CONV>
static int dispatch_dtype(int dtype, bool b_kn, const MatArgs &g, int batch, int tile, int variant,
                          const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    switch (dtype) {
        case GP_F32: return dispatch_any<float, CONV>(b_kn, g, batch, tile, variant, ctx, s, info);
        case GP_F16: return dispatch_any<_Float16, CONV>(b_kn, g, batch, tile, variant, ctx, s, info);
        case GP_BF16: return dispatch_any<__bf16, CONV>(b_kn, g, batch, tile, variant, ctx, s, info);
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
    GP_REQUIRE(p->tile_m == p->tile_n, "gemm: square tiles only");
    return dispatch_dtype<false>(p->dtype, !p->b_is_nk, g, batch, p->tile_m, p->variant, ctx, s, info);
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
    GP_REQUIRE(p->tile_m == p->tile_n, "conv: square tiles only");
    return dispatch_dtype<true>(p->dtype, false, g, 1, p->tile_m, p->variant, ctx, s, info);
}
