#include <algorithm>
// Stand-alone launchers of the memory-bound operators (C ABI); the tile bodies live in
// elementwise_bodies.hpp.
#include "plans.hpp"
#include "stencil_bodies.hpp"
#include "graph_bodies.hpp"

namespace gp {

// the three instantiations of one kernel: general dispatcher loop, no counters, fixed claims
template <class Kernel> struct KernelSet { Kernel any, plain, fixed; };
template <class Kernel> static KernelSet<Kernel> kernel_set(Kernel a, Kernel p, Kernel f) { return {a, p, f}; }
#define GP_KSET(...) kernel_set(__VA_ARGS__, LOOP_ANY>, __VA_ARGS__, LOOP_PLAIN>, __VA_ARGS__, LOOP_FIXED>)

template <class Kernel, class Arg>
static int launch_tiles(KernelSet<Kernel> ks, int sx, int sy, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info, const Arg &arg, size_t lds_bytes = 0, int max_batch = 16) {
    BlpArgs blp;
    int grid = 0;
    // several tiles per claim once there are far more tiles than workgroups that could hold them
    const long tiles = (long)sx * sy;
    const int batch = (int)std::min<long>(max_batch, std::max<long>(1, tiles / (32L * device_cus())));
    if (lds_bytes > 48 * 1024) {
        GP_HIP(hipFuncSetAttribute((const void *)ks.any, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        GP_HIP(hipFuncSetAttribute((const void *)ks.plain, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        GP_HIP(hipFuncSetAttribute((const void *)ks.fixed, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    }
    // planned for the general form; the special ones need no more resources
    int rc = plan_launch(ks.any, NT, lds_bytes, sx, sy, 1, ctx, &blp, &grid, info, batch, batch == 1 ? 4 : 1);
    if (rc) return rc;
    Kernel kern = ks.any;
    if (batch == 1) {  // the special forms call the body once: one tile per claim only
        if (!ctx) kern = ks.plain;
        else if (fixed_claims(true, blp.groups, grid - blp.front, blp.total)) kern = ks.fixed;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds_bytes, native(s), arg, blp);
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

int plan_layout(const gp_layout_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->in && p->out, "null layout params");
    GP_REQUIRE(p->N > 0 && p->C > 0 && p->H > 0 && p->W > 0 && p->c_pad >= p->C, "layout shape");
    GP_REQUIRE(is_float(p->dtype_in) && is_float(p->dtype_out), "layout dtype");
    GP_REQUIRE(p->dtype_in == p->dtype_out || p->dtype_in == GP_F32, "layout: unsupported dtype pair %d -> %d", p->dtype_in, p->dtype_out);
    int HW = p->H * p->W;
    *out = EltPlan{};
    out->op = OP_LAYOUT; out->dtype = p->dtype_out; out->sub = p->dtype_in * 4 + p->dtype_out;
    out->sx = (HW + NT - 1) / NT; out->sy = p->N;
    out->u.layout = LayoutArgs{p->in, p->out, p->C, HW, p->c_pad};
    return GP_SUCC;
}

int plan_pool2d(const gp_pool_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->in && p->out, "null pool params");
    GP_REQUIRE(is_float(p->dtype), "pool dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->N > 0 && p->H > 0 && p->W > 0 && p->C > 0 && p->C % vec == 0, "pool: C must be a positive multiple of %d", vec);
    GP_REQUIRE(p->mode >= 0 && p->mode <= 3, "pool mode %d", p->mode);
    GP_REQUIRE(p->in_pix_stride % vec == 0 && p->out_pix_stride % vec == 0 && p->in_pix_stride >= p->C && p->out_pix_stride >= p->C, "pool pixel strides");
    GP_REQUIRE(al16(p->in) && al16(p->out), "pool: 16-byte alignment");
    int Ho = 1, Wo = 1;
    if (p->mode != 2) {
        GP_REQUIRE(p->R > 0 && p->S > 0 && p->stride > 0 && p->pad >= 0, "pool window");
        Ho = (p->H + 2 * p->pad - p->R) / p->stride + 1;
        Wo = (p->W + 2 * p->pad - p->S) / p->stride + 1;
        GP_REQUIRE(Ho > 0 && Wo > 0, "pool: empty output");
    }
    // a 3 x 3 maximum window moving by 2: four neighbouring outputs per item (pool_tile_block2)
    const int block2 = p->mode == 0 && p->R == 3 && p->S == 3 && p->stride == 2 && p->pad <= 1 && Ho >= 2 && Wo >= 2;
    long items = block2 ? (long)p->N * ((Ho + 1) / 2) * ((Wo + 1) / 2) * (p->C / vec) : (long)p->N * Ho * Wo * (p->C / vec);
    GP_REQUIRE(items < (1L << 31), "pool: too large (2^31 16-byte items at most)");
    *out = EltPlan{};
    out->op = OP_POOL; out->dtype = p->dtype;
    out->sx = (int)((items + NT - 1) / NT); out->sy = 1;
    out->u.pool = PoolArgs{*p, Ho, Wo, items, block2};
    return GP_SUCC;
}

int plan_eltwise(const gp_eltwise_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->a && p->out, "null eltwise params");
    GP_REQUIRE(is_float(p->dtype), "eltwise dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->rows > 0 && p->cols > 0 && p->cols % vec == 0, "eltwise: cols must be a positive multiple of %d", vec);
    GP_REQUIRE(p->a_stride % vec == 0 && p->out_stride % vec == 0 && (!p->b || p->b_stride % vec == 0), "eltwise strides");
    GP_REQUIRE(al16(p->a) && al16(p->out) && al16(p->b) && al16(p->scale) && al16(p->shift), "eltwise: 16-byte alignment");
    long items = p->rows * (p->cols / vec);
    long tiles = (items + (long)NT * ELT_PER - 1) / ((long)NT * ELT_PER);
    GP_REQUIRE(items < (1L << 31), "eltwise: too large (2^31 16-byte items at most)");
    *out = EltPlan{};
    out->op = OP_ELTWISE; out->dtype = p->dtype; out->sx = (int)tiles; out->sy = 1;
    const long bytes = p->rows * p->cols * (long)dtype_size(p->dtype) * (p->b ? 3 : 2);
    out->u.elt = EltwiseArgs{*p, items, bytes > kStreamBytes};
    return GP_SUCC;
}

int plan_softmax(const gp_softmax_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->x && p->out, "null softmax params");
    GP_REQUIRE(is_float(p->dtype), "softmax dtype %d", p->dtype);
    GP_REQUIRE(p->rows > 0 && p->cols > 0, "softmax shape");
    // rows made of whole 16-byte chunks are read as vectors
    GP_REQUIRE(softmax_group(p->cols, vec_of(p->dtype)) == 0 || (al16(p->x) && al16(p->out)), "softmax: 16-byte alignment");
    const int rpt = softmax_rows_per_tile(p->cols, vec_of(p->dtype), p->rows);
    long tiles = (p->rows + rpt - 1) / rpt;
    GP_REQUIRE(tiles < (1L << 31), "softmax: too many rows");
    *out = EltPlan{};
    out->op = OP_SOFTMAX; out->dtype = p->dtype; out->sx = (int)tiles; out->sy = 1;
    out->u.softmax = *p;
    if (out->u.softmax.scale == 0.f) out->u.softmax.scale = 1.f;
    return GP_SUCC;
}

int plan_layernorm(const gp_layernorm_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->x && p->out && p->gamma && p->beta, "null layernorm params");
    GP_REQUIRE(is_float(p->dtype), "layernorm dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->rows > 0 && p->cols > 0 && p->cols % vec == 0, "layernorm: cols must be a positive multiple of %d", vec);
    GP_REQUIRE(p->cols <= 64 * vec * 16, "layernorm: at most %d columns", 64 * vec * 16);
    GP_REQUIRE(al16(p->x) && al16(p->out) && al16(p->residual) && al16(p->gamma) && al16(p->beta), "layernorm: 16-byte alignment");
    int chunks_per_lane = (p->cols / vec + 63) / 64;
    // short rows of a large problem: a wavefront takes two rows at a time, so that twice the bytes are in flight
    const int rpw = (chunks_per_lane <= 2 && p->rows >= 16384) ? 2 : 1;
    long tiles = (p->rows + 4 * rpw - 1) / (4 * rpw);
    GP_REQUIRE(tiles < (1L << 31), "layernorm: too many rows");
    *out = EltPlan{};
    out->op = OP_LAYERNORM; out->dtype = p->dtype; out->sx = (int)tiles; out->sy = 1;
    out->sub = (chunks_per_lane <= 2 ? 2 : chunks_per_lane <= 8 ? 8 : 16) | (rpw == 2 ? kLnTwoRows : 0);
    out->u.ln = *p;
    return GP_SUCC;
}

int plan_embed(const gp_embed_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->ids && p->tok && p->pos && p->out, "null embed params");
    GP_REQUIRE(is_float(p->dtype), "embed dtype %d", p->dtype);
    const int vec = vec_of(p->dtype);
    GP_REQUIRE(p->tokens > 0 && p->seq > 0 && p->vocab > 0 && p->hidden > 0 && p->hidden % vec == 0, "embed: hidden must be a positive multiple of %d", vec);
    GP_REQUIRE(al16(p->tok) && al16(p->pos) && al16(p->seg) && al16(p->out), "embed: 16-byte alignment");
    long tiles = (p->tokens + 3) / 4;
    GP_REQUIRE(tiles < (1L << 31), "embed: too many tokens");
    *out = EltPlan{};
    out->op = OP_EMBED; out->dtype = p->dtype; out->sx = (int)tiles; out->sy = 1;
    out->u.embed = *p;
    return GP_SUCC;
}

int plan_attention(const gp_attention_params *p, EltPlan *out) {
    GP_REQUIRE(p && p->q && p->k && p->v && p->out, "null attention params");
    GP_REQUIRE(p->dtype == GP_F16 || p->dtype == GP_BF16, "attention: fp16 or bf16 only (dtype %d)", p->dtype);
    GP_REQUIRE(p->head_dim == ATT_D, "attention: head_dim must be %d", ATT_D);
    GP_REQUIRE(p->batch > 0 && p->heads > 0 && p->seq > 0 && p->seq <= 512, "attention: seq must be 1..512");
    GP_REQUIRE(p->ld_qkv % 8 == 0 && p->ld_out > 0, "attention: row strides must be multiples of 8 elements");
    GP_REQUIRE(al16(p->q) && al16(p->k) && al16(p->v), "attention: 16-byte alignment");
    *out = EltPlan{};
    out->op = OP_ATTENTION; out->dtype = p->dtype;
    const int qb = attention_queries_per_tile(p->seq);
    out->sx = (p->seq + qb - 1) / qb; out->sy = p->batch * p->heads;
    out->lds_bytes = attention_class_lds_bytes(p->seq);
    out->u.attn = AttnArgs{*p};
    if (out->u.attn.p.scale == 0.f) out->u.attn.p.scale = 1.f;
    return GP_SUCC;
}

int plan_copy(const void *src, void *dst, long bytes, EltPlan *out) {
    GP_REQUIRE(src && dst && bytes > 0, "copy arguments");
    GP_REQUIRE(al16(src) && al16(dst), "copy: 16-byte alignment");
    long tiles = (bytes + COPY_TILE_BYTES - 1) / COPY_TILE_BYTES;
    GP_REQUIRE(tiles < (1L << 31), "copy: too large");
    *out = EltPlan{};
    out->op = OP_COPY; out->dtype = GP_F32; out->sx = (int)tiles; out->sy = 1;
    out->u.copy = CopyArgs{src, dst, bytes};
    return GP_SUCC;
}

int launch_elt_plan(const EltPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    switch (pl.op) {
        case OP_LAYOUT: {
            const int di = pl.sub / 4, dout = pl.sub % 4;
#define L(TI, TO) launch_tiles(GP_KSET(nchw_to_nhwc_kernel<TI, TO), pl.sx, pl.sy, ctx, s, info, pl.u.layout)
            if (di == GP_F32 && dout == GP_F32) return L(float, float);
            if (di == GP_F32 && dout == GP_F16) return L(float, _Float16);
            if (di == GP_F32 && dout == GP_BF16) return L(float, __bf16);
            if (di == GP_F16 && dout == GP_F16) return L(_Float16, _Float16);
            if (di == GP_BF16 && dout == GP_BF16) return L(__bf16, __bf16);
#undef L
            break;
        }
        case OP_POOL: GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(pool_kernel<T), pl.sx, pl.sy, ctx, s, info, pl.u.pool)); break;
        case OP_ELTWISE: GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(eltwise_kernel<T), pl.sx, pl.sy, ctx, s, info, pl.u.elt)); break;
        case OP_SOFTMAX: GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(softmax_kernel<T), pl.sx, pl.sy, ctx, s, info, pl.u.softmax)); break;
        case OP_LAYERNORM:
            if (pl.sub == (2 | kLnTwoRows)) { GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(layernorm_kernel<T, 2, 2), pl.sx, pl.sy, ctx, s, info, pl.u.ln)); }
            else if (pl.sub == 2) { GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(layernorm_kernel<T, 2, 1), pl.sx, pl.sy, ctx, s, info, pl.u.ln)); }
            else if (pl.sub == 8) { GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(layernorm_kernel<T, 8, 1), pl.sx, pl.sy, ctx, s, info, pl.u.ln)); }
            else { GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(layernorm_kernel<T, 16, 1), pl.sx, pl.sy, ctx, s, info, pl.u.ln)); }
            break;
        case OP_EMBED: GP_BY_DTYPE(pl.dtype, launch_tiles(GP_KSET(embed_kernel<T), pl.sx, pl.sy, ctx, s, info, pl.u.embed)); break;
        case OP_COPY: return launch_tiles(GP_KSET(copy_kernel<0), pl.sx, pl.sy, ctx, s, info, pl.u.copy);
        case OP_ATTENTION:
            switch (attention_nb_class(pl.u.attn.p.seq) * 2 + (pl.dtype == GP_F16)) {
#define GP_ATT(NB)                                                                                                            \
    case NB * 2 + 1: return launch_tiles(GP_KSET(attention_kernel<_Float16, NB), pl.sx, pl.sy, ctx, s, info, pl.u.attn, pl.lds_bytes); \
    case NB * 2: return launch_tiles(GP_KSET(attention_kernel<__bf16, NB), pl.sx, pl.sy, ctx, s, info, pl.u.attn, pl.lds_bytes);
                GP_ATT(4) GP_ATT(8) GP_ATT(12) GP_ATT(16)
#undef GP_ATT
            }
            return GP_OUTOFRANGE;
    }
    set_error("unsupported elementwise plan (op %d dtype %d)", pl.op, pl.dtype);
    return GP_OUTOFRANGE;
}

}  // namespace gp

using namespace gp;

#define GP_PLAN_AND_LAUNCH(PLAN_CALL)                     \
    EltPlan pl;                                           \
    int rc = PLAN_CALL;                                   \
    return rc ? rc : launch_elt_plan(pl, ctx, s, info);

extern "C" int gp_launch_nchw_to_nhwc(const gp_layout_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_layout(p, &pl)) }
extern "C" int gp_launch_miniweather(const gp_miniweather_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->hydro, "null miniweather params");
    GP_REQUIRE(p->kernel >= GP_MW_HALO_X && p->kernel <= GP_MW_UPDATE_Z, "miniweather kernel %d", p->kernel);
    GP_REQUIRE(p->nx >= 4 && p->nz >= 4 && (long)p->nx * p->nz <= (1L << 27), "miniweather grid %d x %d", p->nx, p->nz);
    GP_REQUIRE(p->dt > 0 && p->dx > 0 && p->dz > 0, "miniweather steps must be positive");
    const bool update = p->kernel == GP_MW_UPDATE_X || p->kernel == GP_MW_UPDATE_Z;
    const bool flux = p->kernel == GP_MW_FLUX_X || p->kernel == GP_MW_FLUX_Z;
    GP_REQUIRE(p->state || p->kernel == GP_MW_UPDATE_X, "miniweather: state missing");
    GP_REQUIRE(!(update || flux) || p->flux, "miniweather: flux missing");
    GP_REQUIRE(!update || (p->state_init && p->state_out), "miniweather: update operands missing");
    const int tiles = (int)((mw_ids(p->kernel, p->nx, p->nz) + MW_TILE - 1) / MW_TILE);
    switch (p->kernel) {
#define GP_MW(K) case K: return launch_tiles(GP_KSET(miniweather_kernel<K), tiles, 1, ctx, s, info, *p);
        GP_MW(GP_MW_HALO_X) GP_MW(GP_MW_FLUX_X) GP_MW(GP_MW_UPDATE_X) GP_MW(GP_MW_HALO_Z) GP_MW(GP_MW_FLUX_Z) GP_MW(GP_MW_UPDATE_Z)
#undef GP_MW
    }
    return GP_OUTOFRANGE;
}
extern "C" int gp_launch_graph(const gp_graph_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->vertex_list, "null graph params");
    GP_REQUIRE(p->kernel >= GP_GRAPH_BFS_STEP && p->kernel <= GP_GRAPH_CC_INIT, "graph kernel %d", p->kernel);
    GP_REQUIRE(p->vertex_count > 0 && p->vertex_count < (1ULL << 32), "graph: vertex count out of range");
    GP_REQUIRE(p->changed || p->kernel == GP_GRAPH_CC_INIT || p->kernel == GP_GRAPH_PR_INIT || p->kernel == GP_GRAPH_PR_PUSH || p->kernel == GP_GRAPH_SSSP_RELAX, "graph: changed word missing");
    GP_REQUIRE(!graph_kernel_is_edge_parallel(p->kernel) || p->edge_list, "graph: edge list missing");
    switch (p->kernel) {
        case GP_GRAPH_BFS_STEP: GP_REQUIRE(p->label, "bfs: label missing"); break;
        case GP_GRAPH_CC_STEP: case GP_GRAPH_CC_INIT: GP_REQUIRE(p->active && p->next_active && p->comp, "cc: operands missing"); break;
        case GP_GRAPH_PR_INIT: case GP_GRAPH_PR_PUSH: case GP_GRAPH_PR_UPDATE:
            GP_REQUIRE(p->active && p->delta && p->residual && p->value, "pagerank: operands missing"); break;
        case GP_GRAPH_SSSP_RELAX: GP_REQUIRE(p->weight_list && p->active && p->new_cost, "sssp: operands missing"); break;
        case GP_GRAPH_SSSP_UPDATE: GP_REQUIRE(p->active && p->cost && p->new_cost, "sssp: operands missing"); break;
    }
    GP_REQUIRE(p->lanes_per_vertex == 0 || p->lanes_per_vertex == 16 || p->lanes_per_vertex == 32 || p->lanes_per_vertex == 64, "graph: lanes_per_vertex must be 0, 16, 32 or 64");
    const int lanes = graph_kernel_is_edge_parallel(p->kernel) ? graph_lanes(p->lanes_per_vertex) : 64;
    const int tiles = (int)graph_kernel_tiles(p->kernel, p->vertex_count, lanes);
    // a tile of an edge-parallel kernel is a few hundred scattered accesses or atomics (microseconds):
    // claims stay small so that a stop is honoured quickly
    const int max_batch = graph_kernel_is_edge_parallel(p->kernel) ? 4 : 16;
    switch (p->kernel * 100 + lanes) {
#define GP_GR(K, L) case K * 100 + L: return launch_tiles(GP_KSET(graph_kernel<K, L), tiles, 1, ctx, s, info, *p, 0, max_batch);
#define GP_GR_EDGE(K) GP_GR(K, 16) GP_GR(K, 32) GP_GR(K, 64)
        GP_GR_EDGE(GP_GRAPH_BFS_STEP) GP_GR_EDGE(GP_GRAPH_CC_STEP) GP_GR_EDGE(GP_GRAPH_PR_PUSH) GP_GR_EDGE(GP_GRAPH_SSSP_RELAX)
        GP_GR(GP_GRAPH_PR_INIT, 64) GP_GR(GP_GRAPH_PR_UPDATE, 64) GP_GR(GP_GRAPH_SSSP_UPDATE, 64) GP_GR(GP_GRAPH_CC_INIT, 64)
#undef GP_GR_EDGE
#undef GP_GR
    }
    return GP_OUTOFRANGE;
}
extern "C" int gp_launch_attention(const gp_attention_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_attention(p, &pl)) }
extern "C" int gp_launch_pool2d(const gp_pool_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_pool2d(p, &pl)) }
extern "C" int gp_launch_eltwise(const gp_eltwise_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_eltwise(p, &pl)) }
extern "C" int gp_launch_softmax(const gp_softmax_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_softmax(p, &pl)) }
extern "C" int gp_launch_layernorm(const gp_layernorm_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_layernorm(p, &pl)) }
extern "C" int gp_launch_embed(const gp_embed_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info) { GP_PLAN_AND_LAUNCH(plan_embed(p, &pl)) }
