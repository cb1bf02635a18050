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
#include <cstdlib>
#include <mutex>
#include "gemm_tile.hpp"
#include "gemm_pipe.hpp"
#include "gemm_wide.hpp"
#include "gemm_ln.hpp"
#include "plans.hpp"

namespace gp {

// LOOP: which dispatcher loop the instantiation is built around (tile_loop.hpp)
constexpr int LOOP_LOOKS = 3;
template <class TK, int LOOP>
__global__ __launch_bounds__(TK::NT) void mat_kernel(MatArgs g, BlpArgs blp) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    auto *lds = reinterpret_cast<typename TK::elem *>(lds_raw);
    if constexpr (LOOP == LOOP_LOOKS)  // long tiles: fixed claims, and the body looks at the stop word every few K-stages
        tile_fixed_early<true>(blp, [&](TileIdx t, int *stop) {
            CkptCtx cc{stop, nullptr, nullptr, 0};
            if (stop && blp.done) cc.announce = done_counter(blp);
            return TK::template run<true>(g, t, lds, cc);
        });
    else if constexpr (LOOP == LOOP_FIXED && TK::early_stop)
        tile_fixed_early(blp, [&](TileIdx t, int *stop) { return TK::run(g, t, lds, CkptCtx{stop, nullptr, nullptr, 0}); });
    else
        tiles<LOOP>(blp, [&](TileIdx t) { TK::run(g, t, lds); });
}

// bodies that can leave a tile between two K-steps (tile_loop_ckpt)
template <class TK>
__global__ __launch_bounds__(TK::NT) void mat_kernel_ckpt(MatArgs g, BlpArgs blp) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    auto *lds = reinterpret_cast<typename TK::elem *>(lds_raw);
    const CkptCtx cc = {blp.executed && blp.ckpt ? blp.stop_index : nullptr, blp.flag, blp.ckpt, blp.kernel_id, blp.stamps};
    tile_loop_ckpt(blp, [&](TileIdx t, int tile_index, int kt0) { return TK::run(g, t, lds, cc, tile_index, kt0); });
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool CONV, bool B_KN>
using TK = TileKernel<T, BM, BN, BK, WGM, WGN, CONV, B_KN>;

template <class K> struct K_is_ckpt { static constexpr bool value = false; };
template <typename T, int BM, int BN, int ST, bool CV, int W> struct K_is_ckpt<PipeKernel<T, BM, BN, ST, CV, false, true, W>> { static constexpr bool value = true; };
template <class K> struct KernelOf {
    static constexpr auto fn = mat_kernel<K, LOOP_ANY>;
    static constexpr auto plain = mat_kernel<K, LOOP_PLAIN>;
    static constexpr auto fixed = mat_kernel<K, LOOP_FIXED>;
#ifdef GP_NO_LOOKS  // (experiment switch: no instantiations that look more than once)
    static constexpr auto looks = fixed;
#else
    static constexpr auto looks = mat_kernel<K, K::can_look ? LOOP_LOOKS : LOOP_FIXED>;
#endif
};
template <typename T, int BM, int BN, int ST, bool CV, int W> struct KernelOf<PipeKernel<T, BM, BN, ST, CV, false, true, W>> {
    static constexpr auto fn = mat_kernel_ckpt<PipeKernel<T, BM, BN, ST, CV, false, true, W>>;
    static constexpr auto plain = fn;
    static constexpr auto fixed = fn;
    static constexpr auto looks = fn;
};

// bytes of checkpoint workspace a launch of body K needs (0: the body always finishes its tiles)
static size_t ckpt_workspace_bytes(size_t slot_bytes, int workgroups) {
    return (size_t)CKPT_MAX_WGS * CKPT_HEADER_INTS * 4 + (size_t)workgroups * slot_bytes;
}

template <class K>
static int launch_mat(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    BlpArgs blp;
    int grid = 0;
    auto kern = KernelOf<K>::fn;  // the launch is planned for the general form; the others need no more resources
    if (K::LDS_BYTES > 48 * 1024) {
        // several tenant threads launch concurrently: the attribute is set by exactly one of them
        static std::once_flag once;
        static hipError_t once_rc = hipSuccess;
        std::call_once(once, [] {
            for (const void *f : {(const void *)KernelOf<K>::fn, (const void *)KernelOf<K>::plain, (const void *)KernelOf<K>::fixed, (const void *)KernelOf<K>::looks}) {
                hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)K::LDS_BYTES);
                if (e != hipSuccess) once_rc = e;
            }
        });
        GP_HIP(once_rc);
    }
    // Long tiles (1.8 * 10^7 multiply-adds of the 16-bit rate and more, 10-40 us depending on how many workgroups share a
    // compute unit): what a stopped tenant would otherwise finish before it leaves.  The bodies that look at the stop
    // word every few K-stages can give such a tile up (tile_fixed_early).  Measured with the threshold at 0.8 / 2 / 4 * 10^7:
    // ResNet-50 fp32 b1 under a 500 req/s probe drains in 35 / 42 / 57 us (p99) and keeps 1046 / 1095 / 1094 req/s
    // (a launch in this mode is about a microsecond longer).  The 64x64 tiles with K = 4608 and the 128x128 tiles with
    // K = 1152 of VGG-16 have 1.89 * 10^7 each: with them in, BERT's drains of VGG-16 end within 48 us (p99) instead of
    // 60, and a VGG-16 pass takes 4 % longer (those launches 13 %: the instantiation that looks runs its K-steps that
    // much slower than the one that does not, although the two execute the same instructions per K-step to within a
    // few scalar ones).  GPREEMPT_LONG_TILE_MACS overrides it.
    static const double long_macs = [] { const char *e = getenv("GPREEMPT_LONG_TILE_MACS"); return e && atof(e) > 0 ? atof(e) : 1.8e7; }();
    const bool long_tiles = K::can_look && (double)K::bm * K::bn * pl.g.K * (pl.dtype == GP_F32 ? 8.0 : 1.0) >= long_macs;
    int rc = plan_launch(kern, K::NT, K::LDS_BYTES, pl.sx, pl.sy, pl.batch, ctx, &blp, &grid, info, 1, K::LDS_BYTES <= 64 * 1024 ? 4 : 1, long_tiles);
    if (rc) return rc;
    blp.order = pl.order;
    if constexpr (K_is_ckpt<K>::value) {
        if (info) info->fixed_claims = 0;  // tile_loop_ckpt always claims through the counters
        if (blp.spare || blp.front) { grid -= blp.spare + blp.front; blp.spare = blp.front = 0; blp.done = nullptr; set_poll_slices(&blp, grid); if (info) { info->grid = grid; info->front = 0; } }
        // mid-tile checkpoints need the caller's workspace and a slot per workgroup
        if (ctx && ctx->ckpt && ctx->ckpt_bytes >= ckpt_workspace_bytes(K::CKPT_SLOT_BYTES, grid) && grid <= CKPT_MAX_WGS) blp.ckpt = ctx->ckpt;
    }
    // one tile per claim here (plan_launch's default), which is what the two special forms assume
    if (!ctx) kern = KernelOf<K>::plain;
    else if (fixed_claims(true, blp.groups, grid - blp.front, blp.total)) kern = blp.done ? KernelOf<K>::looks : KernelOf<K>::fixed;  // (not for checkpointing bodies: theirs is fn)
    hipLaunchKernelGGL(kern, dim3(grid), dim3(K::NT), K::LDS_BYTES, native(s), pl.g, blp);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

// ring depth per tile size (deeper rings were measured: no gain, lower occupancy)
#ifndef GP_S128
#define GP_S128 3
#endif
#ifndef GP_W256
#define GP_W256 8  // wavefronts of the 256 x 256 body
#endif
#ifndef GP_S64
#define GP_S64 4
#endif
#ifndef GP_S32
#define GP_S32 4
#endif
// The large-GEMM body.  Experiment switch GP_BIG_BM / GP_BIG_BN / GP_BIG_STAGES: another tile shape and ring depth
// for it (128 x 256 with three stages has a prefetch distance of two stages in 144 KB of LDS).
#ifndef GP_BIG_BM
#define GP_BIG_BM 256
#define GP_BIG_BN 256
#define GP_BIG_STAGES 2
#endif
template <typename T, bool CK> using BigPipe = PipeKernel<T, GP_BIG_BM, GP_BIG_BN, GP_BIG_STAGES, false, false, CK, GP_W256>;
template <typename T, int TILE, int STAGES, bool SPLITK>
static int pipe_case(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    if (pl.conv) return launch_mat<PipeKernel<T, TILE, TILE, STAGES, true, SPLITK>>(pl, ctx, s, info);
    return launch_mat<PipeKernel<T, TILE, TILE, STAGES, false, SPLITK>>(pl, ctx, s, info);
}
static size_t plan_ckpt_bytes(const MatPlan &pl);
// the instantiation that can leave a tile between two K-steps, when the caller brought a workspace big enough for it
template <typename T, int TILE, int STAGES>
static int pipe_case_ckpt(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    if (!(ctx && ctx->ckpt && ctx->ckpt_bytes >= plan_ckpt_bytes(pl))) return pipe_case<T, TILE, STAGES, false>(pl, ctx, s, info);
    if (pl.conv) return launch_mat<PipeKernel<T, TILE, TILE, STAGES, true, false, true>>(pl, ctx, s, info);
    return launch_mat<PipeKernel<T, TILE, TILE, STAGES, false, false, true>>(pl, ctx, s, info);
}

// Ring depth of a wide body: three stages, four for the GEMM form of the 32 x 32 tile on 16 wavefronts (a
// stage is (WAVES / 4) K-blocks of BM + BN rows of 128 bytes: 32 KB there).  128 x 768 x 3072 went from
// 7.96 to 7.67 us per launch with the fourth stage; given to every body that has room for it, it cost the
// convolution chain of ResNet-152 1 us per launch (10.2 -> 11.2), and so did two stages instead of three for
// the convolution form (10.05 -> 10.98).
constexpr int wide_stages(int bm, int bn, int waves, bool conv) { return (!conv && bm == 32 && bn == 32 && waves == 16) ? 4 : 3; }
template <typename T, int BM, int BN, int WAVES, bool CONV = false>
using WideK = WideKernel<T, BM, BN, WAVES, wide_stages(BM, BN, WAVES, CONV), CONV>;

template <typename T, int BM, int BN, int WAVES>
static int wide_case(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    if (pl.conv) return launch_mat<WideK<T, BM, BN, WAVES, true>>(pl, ctx, s, info);
    return launch_mat<WideK<T, BM, BN, WAVES, false>>(pl, ctx, s, info);
}

template <typename T>
static int launch_typed(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    constexpr int SBK = sizeof(T) == 4 ? 16 : 32;
    switch (pl.body) {
        case MB_PIPE256:  // GEMM only: the gathered A operand of a convolution does not fit its register budget
            if (ctx && ctx->ckpt) return launch_mat<BigPipe<T, true>>(pl, ctx, s, info);
            return launch_mat<BigPipe<T, false>>(pl, ctx, s, info);
        case MB_PIPE128: return pipe_case_ckpt<T, 128, GP_S128>(pl, ctx, s, info);
        case MB_PIPE64:
            // A layer of at most four K-steps is all prologue and epilogue, and what hides those is more workgroups
            // per compute unit: with a ring of two stages (32 KB of LDS instead of 64) four fit instead of two.
            // 25088 x 256 x 64 with a residual (ResNet-152 b8, 56 x 56): 15.5 -> 10.7 us plain, 19.4 -> 13.6 us
            // preemptible; 6272 x 512 x 128: 10.0 -> 7.6 us.  Deep layers keep four stages (K = 4608 on 392 tiles:
            // 22.5 us with four, 38.6 with two).
            if (pl.g.K <= 256) return pipe_case<T, 64, 2, false>(pl, ctx, s, info);
            return pipe_case<T, 64, GP_S64, false>(pl, ctx, s, info);
        case MB_PIPE64_SK: return pipe_case<T, 64, GP_S64, true>(pl, ctx, s, info);
        case MB_PIPE32_SK: return pipe_case<T, 32, GP_S32, true>(pl, ctx, s, info);
        case MB_WIDE32x32_16: return wide_case<T, 32, 32, 16>(pl, ctx, s, info);
        case MB_WIDE32x32_8: return wide_case<T, 32, 32, 8>(pl, ctx, s, info);
        case MB_WIDE64x32_16: return wide_case<T, 64, 32, 16>(pl, ctx, s, info);
        case MB_WIDE64x64_8: return wide_case<T, 64, 64, 8>(pl, ctx, s, info);
        case MB_LNWIDE32x64_16:
            if constexpr (sizeof(T) == 2) return launch_mat<LnWideKernel<T, 32, 64, 16, 3>>(pl, ctx, s, info);
            break;
        case MB_STAGED128:
            if (pl.conv) return launch_mat<TK<T, 128, 128, SBK, 2, 2, true, false>>(pl, ctx, s, info);
            return pl.b_kn ? launch_mat<TK<T, 128, 128, SBK, 2, 2, false, true>>(pl, ctx, s, info)
                           : launch_mat<TK<T, 128, 128, SBK, 2, 2, false, false>>(pl, ctx, s, info);
        case MB_STAGED64:
            if (pl.conv) return launch_mat<TK<T, 64, 64, SBK, 2, 2, true, false>>(pl, ctx, s, info);
            return pl.b_kn ? launch_mat<TK<T, 64, 64, SBK, 2, 2, false, true>>(pl, ctx, s, info)
                           : launch_mat<TK<T, 64, 64, SBK, 2, 2, false, false>>(pl, ctx, s, info);
    }
    set_error("unknown matrix kernel body %d", pl.body);
    return GP_FAIL;
}

int launch_mat_plan(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    switch (pl.dtype) {
        case GP_F32: return launch_typed<float>(pl, ctx, s, info);
        case GP_F16: return launch_typed<_Float16>(pl, ctx, s, info);
        case GP_BF16: return launch_typed<__bf16>(pl, ctx, s, info);
    }
    set_error("unsupported dtype %d for matrix kernels", pl.dtype);
    return GP_OUTOFRANGE;
}

static size_t body_lds_bytes(int body, int dtype) {
    const size_t es = dtype == GP_F32 ? 4 : 2;
    switch (body) {
        case MB_PIPE256: return BigPipe<_Float16, false>::LDS_BYTES;
        case MB_PIPE128: return GP_S128 * (128 + 128) * 128;
        case MB_PIPE64: return GP_S64 * (64 + 64) * 128;
        case MB_PIPE64_SK: return GP_S64 * (64 + 64) * 128;   // at least the reduction buffer (4 waves x 4 blocks x 16 x 64 x 4 = 64 KB)
        case MB_PIPE32_SK: return GP_S32 * (32 + 32) * 128;
        case MB_WIDE32x32_16: return WideK<_Float16, 32, 32, 16>::LDS_BYTES;
        case MB_WIDE32x32_8: return WideK<_Float16, 32, 32, 8>::LDS_BYTES;
        case MB_WIDE64x32_16: return WideK<_Float16, 64, 32, 16>::LDS_BYTES;
        case MB_WIDE64x64_8: return WideK<_Float16, 64, 64, 8>::LDS_BYTES;
        case MB_LNWIDE32x64_16: return LnWideKernel<_Float16, 32, 64, 16, 3>::LDS_BYTES;
        case MB_STAGED128: return (128 + 128) * ((es == 4 ? 16 : 32) + (es == 4 ? 4 : 8)) * es;
        case MB_STAGED64: return (64 + 64) * ((es == 4 ? 16 : 32) + (es == 4 ? 4 : 8)) * es;
    }
    return 0;
}

// Kernel and tile choice.  B stored K x N needs the transposing, register-staged kernel.
// Otherwise the pipelined kernel is used with the largest tile that still gives every compute
// unit work; problems too small for that split K across the waves of a workgroup so that the
// serial K loop shrinks instead.
// the wide split-K bodies (gemm_wide.hpp) and their tiles
struct WideChoice { int body, bm, bn, waves; size_t lds; };
static const WideChoice kWide[4] = {
    {MB_WIDE32x32_16, 32, 32, 16, WideK<_Float16, 32, 32, 16>::LDS_BYTES},
    {MB_WIDE32x32_8, 32, 32, 8, WideK<_Float16, 32, 32, 8>::LDS_BYTES},
    {MB_WIDE64x32_16, 64, 32, 16, WideK<_Float16, 64, 32, 16>::LDS_BYTES},
    {MB_WIDE64x64_8, 64, 64, 8, WideK<_Float16, 64, 64, 8>::LDS_BYTES}};
static const WideChoice *wide_of(int body) {
    for (const WideChoice &w : kWide) if (w.body == body) return &w;
    return nullptr;
}
// Which wide body, if any: measured on MI355X (launch to launch, fp16, against the best of the
// four-wavefront bodies): they win where one round of workgroups covers the problem and K is deep
// enough to pay for the larger first stage.  128 x 768 x 3072: 10.2 -> 7.9 us; 392 x 512 x 4608:
// 14.0 -> 10.4; 1568 x 256 x 2304: 10.0 -> 8.3; 1568 x 256 x 1024: 6.6 -> 6.1; 128 x 768 x 768: 5.1 -> 4.7;
// 6272 x 128 x 1152: 8.9 -> 8.0; 392 x 2048 x 512: 6.4 -> 5.9.
static int wide_pick(const MatArgs &g, int batch, long cus, int dtype) {
    auto tiles = [&](int tm, int tn) { return (long)((g.M + tm - 1) / tm) * ((g.N + tn - 1) / tn) * batch; };
    // fp32 runs on MFMAs an eighth as fast, so a small layer is bound by them and not by its operands: as many
    // tiles as there are compute units to take them (ResNet-50 b1 fp32, launch to launch: 7 x 7 x 512 -> 2048
    // 13.1 -> 6.7 us, 3 x 3 at 56 x 56 x 64 16.2 -> 9.1 us; these tiles are also what a preempted tenant
    // finishes before it leaves)
    if (dtype == GP_F32 && tiles(32, 32) <= cus) return g.K >= 768 ? MB_WIDE32x32_16 : MB_WIDE32x32_8;
    if (g.K >= 768 && tiles(32, 32) <= cus) return MB_WIDE32x32_16;
    if (g.K >= 768 && tiles(64, 32) <= cus) return MB_WIDE64x32_16;
    if (g.K >= 512 && tiles(64, 64) <= cus && g.N > 32) return MB_WIDE64x64_8;
    return -1;
}

static int choose_body(MatPlan *pl, int tile, int tile_n, int variant) {
    const MatArgs &g = pl->g;
    auto tiles = [&](int t) { return (long)((g.M + t - 1) / t) * ((g.N + t - 1) / t) * pl->batch; };
    const long cus = device_cus();
    // both operands K-contiguous; a convolution, whose A operand is gathered, when a K-block never straddles
    // two filter taps and a bit per tap fits a word
    const int wide_bk = pl->dtype == GP_F32 ? 32 : 64;
    const bool wide_ok = !pl->b_kn && (!pl->conv || (g.Cin % wide_bk == 0 && g.K / g.Cin <= 32 && g.S < 32));
    int body = -1;
    if (g.ln_gamma) body = MB_LNWIDE32x64_16;  // (plan_gemm has checked that the shape fits)
    else if (pl->b_kn || variant == GP_MAT_STAGED) {
        int tm = tile ? tile : (tiles(128) >= cus ? 128 : 64);
        body = tm == 128 ? MB_STAGED128 : tm == 64 ? MB_STAGED64 : -1;
    } else if (variant == GP_MAT_PIPE) {
        int tm = tile ? tile : (tiles(128) >= cus ? 128 : 64);
        body = (tm == 256 && !pl->conv) ? MB_PIPE256 : tm == 128 ? MB_PIPE128 : tm == 64 ? MB_PIPE64 : -1;
    } else if (variant == GP_MAT_PIPE_SPLITK) {
        int tm = tile ? tile : (tiles(64) >= cus / 2 ? 64 : 32);
        body = tm == 64 ? MB_PIPE64_SK : tm == 32 ? MB_PIPE32_SK : -1;
    } else if (variant == GP_MAT_WIDE || variant == GP_MAT_WIDE8) {
        if (wide_ok) {
            const int tn = tile_n ? tile_n : tile;
            if (tile == 32 && tn == 32) body = variant == GP_MAT_WIDE ? MB_WIDE32x32_16 : MB_WIDE32x32_8;
            else if (tile == 64 && tn == 32) body = MB_WIDE64x32_16;
            else if (tile == 64 && tn == 64) body = MB_WIDE64x64_8;
        }
    } else if (variant == GP_MAT_AUTO) {
        // a tile wider than the problem multiplies zero columns: N <= 64 never takes the larger tiles
        if (!pl->conv && (tile == 256 || (tile == 0 && tiles(256) >= cus && g.N > 128 && g.M > 128))) body = MB_PIPE256;
        // (a problem of one or two K-steps is all epilogue, i.e. memory-bound: the 128 x 128 body runs one workgroup
        // per CU, too few threads for that; 25088 x 256 x 64 with a residual: 19.8 us on 128 x 128, 15.0 on 64 x 64)
        else if (tile == 128 || (tile == 0 && tiles(128) >= cus && g.N > 64 && g.M > 64 && g.K > 128)) body = MB_PIPE128;
        else if (tile == 0 && wide_ok && wide_pick(g, pl->batch, cus, pl->dtype) >= 0) body = wide_pick(g, pl->batch, cus, pl->dtype);
        else if (tile == 64 || (tile == 0 && (tiles(64) >= cus || g.K < 512))) body = MB_PIPE64;
        else if (tile == 0 && tiles(64) >= cus / 2) body = MB_PIPE64_SK;
        else if (tile == 0 || tile == 32) body = MB_PIPE32_SK;
    }
    if (body < 0) {
        set_error("no matrix kernel for tile %d x %d with variant %d (tiles: 256, 128, 64; 64, 32 with split K; wide: 32x32, 64x32, 64x64, N x K operands; convolutions with Cin a multiple of the K-block and at most 32 taps)", tile, tile_n ? tile_n : tile, variant);
        return GP_OUTOFRANGE;
    }
    int t = body == MB_PIPE256 ? GP_BIG_BM : (body == MB_PIPE128 || body == MB_STAGED128) ? 128 : (body == MB_PIPE32_SK ? 32 : 64);
    int tn = body == MB_PIPE256 ? GP_BIG_BN : t;
    if (const WideChoice *w = wide_of(body)) { t = w->bm; tn = w->bn; }
    if (body == MB_LNWIDE32x64_16) { t = 32; tn = 64; }
    pl->body = body;
    pl->sx = (g.N + tn - 1) / tn;
    pl->sy = (g.M + t - 1) / t;
    pl->lds_bytes = body_lds_bytes(body, pl->dtype);
    // Each XCD works on a contiguous eighth of the tile order (util/slice_map.h).  With x fastest
    // that is a band of tile rows: every XCD fetches its share of A and all of B; with y fastest
    // it is a band of tile columns: all of A and a share of B.  Take the cheaper one.
    const double a_elems = pl->conv ? (double)(g.M / (g.Ho * g.Wo > 0 ? g.Ho * g.Wo : 1)) * g.H * g.W * g.Cin : (double)g.M * g.K;
    const double b_elems = (double)g.N * g.K;
    pl->order = b_elems > a_elems ? 1 : 0;
    // Large GEMMs on the 256 x 256 tiles: an XCD runs 32 of them side by side, and a single tile row
    // with 32 column panels means 33 distinct operand panels streaming through its 4 MB L2; taken
    // as bands of two tile rows it is 18.  Measured at 8192^3 bf16, plain launches: constant
    // operands 889 -> 718 us, U[-1,1) operands 956 -> 928 us (those are bounded by power, see the
    // profile of this kernel); bands of 4, 8 and 16 rows were level or worse.
    if (!pl->conv && body == MB_PIPE256 && pl->sx >= 16 && pl->sy >= 16) pl->order = 2;
    return GP_SUCC;
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// shapes the layer-norm prologue body takes (the tile count bounds how often a row is re-normalised)
static bool ln_shape_ok(const gp_gemm_params *p) {
    if (!p || (p->dtype != GP_F16 && p->dtype != GP_BF16) || p->batch > 1 || !p->b_is_nk) return false;
    if (p->M <= 0 || p->N <= 0 || p->K <= 0 || p->lda != p->K || p->K % 64 != 0 || p->K > LnWideKernel<_Float16, 32, 64, 16, 3>::MAXK) return false;
    // one round of workgroups: every workgroup normalises its own 32 rows, which pays while that hides
    // behind the fetch of B and not when a compute unit does it twice
    const long tiles = (long)((p->M + 31) / 32) * ((p->N + 63) / 64);
    return tiles <= device_cus();
}
int plan_gemm(const gp_gemm_params *p, MatPlan *out);
// ... and the body the launcher would pick for the plain GEMM sums K in the prologue body's order (K-steps
// dealt to four wavefronts, partial tiles added in wavefront order), so that fusing changes no bit
extern "C" int gp_gemm_ln_supported(const gp_gemm_params *p) {
    if (!ln_shape_ok(p)) return 0;
    gp_gemm_params q = *p;
    q.ln_gamma = q.ln_beta = nullptr; q.ln_out = nullptr;
    q.tile_m = q.tile_n = q.variant = 0;
    MatPlan pl;
    if (!q.A || !q.B || !q.C || plan_gemm(&q, &pl) != GP_SUCC) return 0;
    return (is_wide_body(pl.body) || pl.body == MB_PIPE64_SK || pl.body == MB_PIPE32_SK) ? 1 : 0;
}

int plan_gemm(const gp_gemm_params *p, MatPlan *out) {
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
    GP_REQUIRE(p->tile_m == p->tile_n || p->variant == GP_MAT_WIDE || p->variant == GP_MAT_WIDE8, "gemm: square tiles only (the wide variants also take 64 x 32)");
    MatPlan &pl = *out;
    pl = MatPlan{};
    MatArgs &g = pl.g;
    g.M = p->M; g.N = p->N; g.K = p->K;
    g.A = p->A; g.lda = p->lda; g.stride_a = p->stride_a; g.stride_a_outer = p->stride_a_outer;
    g.B = p->B; g.ldb = p->ldb; g.stride_b = p->stride_b; g.stride_b_outer = p->stride_b_outer;
    g.C = p->C; g.ldc = p->ldc; g.stride_c = p->stride_c; g.stride_c_outer = p->stride_c_outer;
    g.bias = p->bias; g.residual = p->residual; g.ldr = p->ldc;
    g.alpha = p->alpha == 0.f ? 1.f : p->alpha;
    g.act = p->act; g.batch_inner = batch > 1 ? p->batch_inner : 0;
    pl.dtype = p->dtype; pl.conv = 0; pl.b_kn = !p->b_is_nk; pl.batch = batch;
    if (p->ln_gamma) {
        GP_REQUIRE(ln_shape_ok(p), "gemm: no layer-norm prologue for this shape (16-bit, batch 1, B as N x K, lda == K, K a multiple of 64 up to %d)", LnWideKernel<_Float16, 32, 64, 16, 3>::MAXK);
        GP_REQUIRE(p->ln_beta && p->ln_out, "gemm: the layer-norm prologue needs gamma, beta and ln_out");
        GP_REQUIRE(aligned16(p->ln_gamma) && aligned16(p->ln_beta) && aligned16(p->ln_out), "gemm: ln_gamma, ln_beta and ln_out must be 16-byte aligned");
        g.ln_gamma = p->ln_gamma; g.ln_beta = p->ln_beta; g.ln_out = p->ln_out; g.ln_eps = p->ln_eps;
    }
    return choose_body(&pl, p->tile_m, p->tile_n, p->variant);
}

int plan_conv2d(const gp_conv_params *p, MatPlan *out) {
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
    GP_REQUIRE((long)p->N * (p->H + 2L * p->pad_h) * (p->W + 2L * p->pad_w) < (1L << 31), "conv: too many input pixels");
    GP_REQUIRE(!p->residual || p->res_pix_stride >= p->Cout, "conv: residual pixel stride");
    GP_REQUIRE(p->tile_m == p->tile_n || p->variant == GP_MAT_WIDE || p->variant == GP_MAT_WIDE8, "conv: square tiles only (the wide variants also take 64 x 32)");
    MatPlan &pl = *out;
    pl = MatPlan{};
    MatArgs &g = pl.g;
    if (p->R == 1 && p->S == 1 && p->stride_h == 1 && p->stride_w == 1 && p->pad_h == 0 && p->pad_w == 0) {
        // A pointwise convolution IS a GEMM over the pixels (rows in_pix_stride apart); the GEMM
        // bodies need no window arithmetic and were measured about 1 us per launch faster at
        // ResNet-152's shapes (1568 x 256 x 1024: 7.7 -> 6.6 us with the same tile body).
        g.M = (int)M; g.N = p->Cout; g.K = p->Cin;
        g.A = p->in; g.lda = p->in_pix_stride;
        g.B = p->weight; g.ldb = g.K;
        g.C = p->out; g.ldc = p->out_pix_stride;
        g.bias = p->bias; g.residual = p->residual; g.ldr = p->residual ? p->res_pix_stride : 0;
        g.alpha = 1.f; g.act = p->act; g.batch_inner = 0;
        pl.dtype = p->dtype; pl.conv = 0; pl.b_kn = 0; pl.batch = 1;
        // an explicit variant keeps its meaning; the staged variant of a convolution has no K x N weights
        return choose_body(&pl, p->tile_m, p->tile_n, p->variant);
    }
    g.M = (int)M; g.N = p->Cout; g.K = p->R * p->S * p->Cin;
    g.A = p->in; g.lda = p->in_pix_stride;
    g.B = p->weight; g.ldb = g.K;
    g.C = p->out; g.ldc = p->out_pix_stride;
    g.bias = p->bias; g.residual = p->residual; g.ldr = p->residual ? p->res_pix_stride : 0;
    g.alpha = 1.f; g.act = p->act; g.batch_inner = 0;
    g.H = p->H; g.W = p->W; g.Cin = p->Cin; g.S = p->S; g.Ho = Ho; g.Wo = Wo;
    g.sh = p->stride_h; g.sw = p->stride_w; g.ph = p->pad_h; g.pw = p->pad_w;
    pl.dtype = p->dtype; pl.conv = 1; pl.b_kn = 0; pl.batch = 1;
    return choose_body(&pl, p->tile_m, p->tile_n, p->variant);
}

}  // namespace gp

using namespace gp;

extern "C" int gp_launch_gemm(const gp_gemm_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    MatPlan pl;
    int rc = plan_gemm(p, &pl);
    return rc ? rc : launch_mat_plan(pl, ctx, s, info);
}

extern "C" int gp_launch_conv2d(const gp_conv_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    MatPlan pl;
    int rc = plan_conv2d(p, &pl);
    if (rc) return rc;
    // A preemptible launch finishes the tiles it holds before it leaves, so a tenant's preemption latency is its
    // longest tile.  A 128 x 128 tile of a deep layer runs 45-65 us (VGG-16 b16: K = 2304 at 56 x 56, K = 4608
    // at 28 x 28); four 64 x 64 tiles in its place finish one by one.  Launch to launch the smaller tiles
    // cost nothing at K = 2304 (131 against 132 us) and 13 % at K = 4608 (132 against 117 us), 2 % of the
    // network; same summation per element, so the bits do not change.  Not when the caller chose the tile,
    // and not when it brought a checkpoint workspace (then long tiles are left between two K-steps instead).
    if (ctx && pl.body == MB_PIPE128 && pl.g.K >= 2304 && p->tile_m == 0 && p->variant == 0 && !(ctx->ckpt && ctx->ckpt_bytes >= plan_ckpt_bytes(pl))) {
        gp_conv_params q = *p;
        q.tile_m = q.tile_n = 64;
        q.variant = GP_MAT_PIPE;
        MatPlan small;
        if (plan_conv2d(&q, &small) == GP_SUCC) pl = small;
    }
    return launch_mat_plan(pl, ctx, s, info);
}

#ifdef GP_TILE_PROF
extern "C" int gp_debug_tile_prof(unsigned long long *out, int n) {
    GP_HIP(hipDeviceSynchronize());
    const int body = n < 256 * 8 ? n : 256 * 8;
    GP_HIP(hipMemcpyFromSymbol(out, HIP_SYMBOL(gp::g_tile_prof), sizeof(unsigned long long) * (size_t)body));
    if (n > body) GP_HIP(hipMemcpyFromSymbol(out + body, HIP_SYMBOL(gp::g_disp_prof), sizeof(unsigned long long) * (size_t)std::min(n - body, 256 * 8)));
    return GP_SUCC;
}
#endif

// Checkpoint workspace of the bodies that can leave a tile half-way (the 256 x 256 and 128 x 128
// bodies): headers plus one accumulator slot per resident workgroup.
namespace gp {
static size_t plan_ckpt_bytes(const MatPlan &pl) {
    if (pl.body == MB_PIPE256) return ckpt_workspace_bytes(BigPipe<float, true>::CKPT_SLOT_BYTES, (int)device_cus());
    if (pl.body == MB_PIPE128) return ckpt_workspace_bytes(PipeKernel<float, 128, 128, GP_S128, false, false, true>::CKPT_SLOT_BYTES, 2 * (int)device_cus());
    return 0;
}
}  // namespace gp
extern "C" int gp_gemm_ckpt_bytes(const gp_gemm_params *p, size_t *bytes) {
    GP_REQUIRE(bytes != nullptr, "null bytes");
    MatPlan pl;
    int rc = plan_gemm(p, &pl);
    if (rc) return rc;
    *bytes = plan_ckpt_bytes(pl);
    return GP_SUCC;
}
extern "C" int gp_conv_ckpt_bytes(const gp_conv_params *p, size_t *bytes) {
    GP_REQUIRE(bytes != nullptr, "null bytes");
    MatPlan pl;
    int rc = plan_conv2d(p, &pl);
    if (rc) return rc;
    *bytes = plan_ckpt_bytes(pl);
    return GP_SUCC;
}

extern "C" int gp_ckpt_reset_async(void *ckpt, gp_stream s) {
    GP_REQUIRE(ckpt != nullptr, "null checkpoint workspace");
    return gp_fill32_async(ckpt, 0, (size_t)CKPT_MAX_WGS * CKPT_HEADER_INTS, s);
}

// ---- a preemptible GEMM launch that allocates nothing -----------------------------------------------
// gp_launch_gemm takes its claim counters and stop index from the caller's context, which somebody
// had to allocate.  Callers that cannot allocate (code under HIP graph capture, tight serving loops,
// harnesses that forbid it) get the same launch with that state in a file-scope device array: 64
// kernel slots of 32 counters (one per 64-byte line), then one line that holds the stop index.
// The array exists once per GPU for the life of the process; every call on a GPU shares it and it
// keeps the last call's contents, so calls that overlap on one GPU race.
namespace gp {
constexpr int kStaticSlots = 64;      // kernels whose counters the array can hold at once
constexpr int kStaticGroups = 32;     // claim counters per kernel, as BLPExecutor uses
constexpr int kStaticSlotInts = kStaticGroups * COUNTER_STRIDE;
constexpr int kStaticInts = kStaticSlots * kStaticSlotInts + COUNTER_STRIDE;   // 131 136 bytes
constexpr int kStaticMaxDevices = 16;
static __device__ __align__(256) int scratch[kStaticInts];

// `scratch` is only a host-side stand-in here: the array's address on each device comes from
// hipGetSymbolAddress, once per device, with that device current.
static std::mutex g_scratch_mu;
static int *g_scratch_ptr[kStaticMaxDevices] = {nullptr};

int static_scratch_setup(int **out) {
    int dev = -1;
    GP_HIP(hipGetDevice(&dev));
    GP_REQUIRE(dev >= 0 && dev < kStaticMaxDevices, "device %d is beyond the %d the static scratch serves", dev, kStaticMaxDevices);
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        GP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        GP_REQUIRE(p != nullptr, "hipGetSymbolAddress returned no address for the static scratch");
        g_scratch_ptr[dev] = (int *)p;
    }
    if (out) *out = g_scratch_ptr[dev];
    return GP_SUCC;
}

// Clears one slot's counter lines and re-arms the stop index (a kernel, not a memset: the call may
// be recorded into a graph).
__global__ void static_reset_kernel(int *counters, int n, int *stop) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (counters && i < n) counters[i] = 0;
    if (stop && i == 0) *stop = -1;
}
__global__ void static_report_kernel(const int *stop, int *out) {
    if (threadIdx.x == 0) __hip_atomic_store(out, *stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
}  // namespace gp

extern "C" int gp_launch_gemm_noalloc(const gp_gemm_params *p, int *flag, int slot, int mode, int inject_at, int *stop_index_out,
                                      gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(mode >= 0 && mode <= (GP_NOALLOC_CLEAR | GP_NOALLOC_REARM), "mode %d", mode);
    GP_REQUIRE(slot >= 0 && slot < kStaticSlots, "slot %d: the static scratch holds the counters of %d kernels (slots 0..%d)", slot, kStaticSlots, kStaticSlots - 1);
    MatPlan pl;
    int rc = plan_gemm(p, &pl);
    if (rc) return rc;
    // every claim must be countable in the slot: the tile grid is bounded like a launch's
    GP_REQUIRE((long)pl.sx * pl.sy * pl.batch <= (1L << 24), "gemm of %ld tiles: the static scratch serves at most %ld per launch", (long)pl.sx * pl.sy * pl.batch, 1L << 24);
    int *base = nullptr;
    rc = static_scratch_setup(&base);
    if (rc) return rc;
    int *counters = base + (size_t)slot * kStaticSlotInts, *stop = base + (size_t)kStaticSlots * kStaticSlotInts;
    if (mode) {
        hipLaunchKernelGGL(static_reset_kernel, dim3((kStaticSlotInts + 255) / 256), dim3(256), 0, native(s),
                           (mode & GP_NOALLOC_CLEAR) ? counters : (int *)nullptr, kStaticSlotInts, (mode & GP_NOALLOC_REARM) ? stop : (int *)nullptr);
        GP_HIP(hipGetLastError());
    }
    gp_preempt_ctx ctx{};
    ctx.flag = flag; ctx.stop_index = stop; ctx.executed = counters; ctx.kernel_id = slot; ctx.inject_at = inject_at;
    ctx.counter_groups = kStaticGroups;
    ctx.fresh = (mode & GP_NOALLOC_CLEAR) != 0;
    rc = launch_mat_plan(pl, &ctx, s, info);
    if (rc) return rc;
    if (stop_index_out) {
        hipLaunchKernelGGL(static_report_kernel, dim3(1), dim3(64), 0, native(s), (const int *)stop, stop_index_out);
        GP_HIP(hipGetLastError());
    }
    return GP_SUCC;
}
