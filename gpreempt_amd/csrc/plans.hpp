// Launch plans: the validated, resolved form of an operator call (argument block, tile grid,
// kernel body).  The stand-alone launchers (gp_launch_*) launch a plan at once; the whole-model
// program (program.hip) stores plans as layer descriptors of one persistent kernel.
#pragma once
#include "elementwise_bodies.hpp"
#include "mma.hpp"
#include "attention_bodies.hpp"

namespace gp {

enum MatBody { MB_PIPE128 = 0, MB_PIPE64 = 1, MB_PIPE64_SK = 2, MB_PIPE32_SK = 3, MB_STAGED128 = 4, MB_STAGED64 = 5, MB_PIPE256 = 6,
               // wide split-K bodies (gemm_wide.hpp): tile rows x columns _ wavefronts
               MB_WIDE32x32_16 = 7, MB_WIDE32x32_8 = 8, MB_WIDE64x32_16 = 9, MB_WIDE64x64_8 = 10,
               // a wide 32 x 64 body with a layer-norm prologue over the rows of A (gemm_ln.hpp)
               MB_LNWIDE32x64_16 = 11 };
inline bool is_wide_body(int b) { return b >= MB_WIDE32x32_16 && b <= MB_WIDE64x64_8; }

struct MatPlan {
    MatArgs g;
    int dtype, body, conv, b_kn, batch;
    int sx, sy;        // tile grid (x over N, y over M, z = batch)
    int order;         // tile order handed to the dispatcher: 0 = x fastest, 1 = y fastest, G >= 2 = bands of G tile rows
    size_t lds_bytes;
};

enum EltOp { OP_MAT = 0, OP_LAYOUT, OP_POOL, OP_ELTWISE, OP_SOFTMAX, OP_LAYERNORM, OP_EMBED, OP_COPY, OP_ATTENTION };

struct EltPlan {
    int op, dtype, sub;  // sub: layout -> (dtype_in * 4 + dtype_out); layernorm -> chunks kept per lane (2, 8, 16)
    int sx, sy;
    size_t lds_bytes;    // dynamic LDS of the body (attention only; 0 otherwise)
    union {
        AttnArgs attn;
        LayoutArgs layout;
        PoolArgs pool;
        EltwiseArgs elt;
        gp_softmax_params softmax;
        gp_layernorm_params ln;
        gp_embed_params embed;
        CopyArgs copy;
    } u;
};

int plan_gemm(const gp_gemm_params *p, MatPlan *out);
int plan_conv2d(const gp_conv_params *p, MatPlan *out);
int launch_mat_plan(const MatPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

int plan_layout(const gp_layout_params *p, EltPlan *out);
int plan_pool2d(const gp_pool_params *p, EltPlan *out);
int plan_eltwise(const gp_eltwise_params *p, EltPlan *out);
int plan_softmax(const gp_softmax_params *p, EltPlan *out);
int plan_layernorm(const gp_layernorm_params *p, EltPlan *out);
int plan_embed(const gp_embed_params *p, EltPlan *out);
int plan_copy(const void *src, void *dst, long bytes, EltPlan *out);
int plan_attention(const gp_attention_params *p, EltPlan *out);
int launch_elt_plan(const EltPlan &pl, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

}  // namespace gp
