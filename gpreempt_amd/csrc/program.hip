// Whole-model program: every layer of a model runs inside ONE persistent kernel.
//
// Why: with one launch (or graph node) per layer, a preempted model still has to push every
// remaining node through the queue, each leaving at its first flag check; at 4-9 us per node
// that drain, not the kernels, sets the preemption latency (hundreds of microseconds for a
// 160-layer network), and a small high-priority model is launch-bound for the same reason.
// Here the layer list lives in device memory and the resident workgroups walk it themselves:
//
//   * a workgroup claims the next tile of the current layer from that layer's counter
//     (executed[l]); when the counter is exhausted it moves to layer l+1;
//   * before running a tile of layer l it waits until done[l-1] == total[l-1], i.e. until every
//     tile of the previous layer has been written (layer-granular dependency); the tiles it
//     waits for were all claimed by workgroups that are running, so the wait always ends;
//   * it polls the preempt flag exactly as the per-kernel dispatcher does (tile_loop.hpp); when
//     the flag is up it records the layer in *stop_index and leaves.  Everything it had claimed
//     is finished first, so afterwards done[l] == min(executed[l], total[l]) for every layer and
//     a relaunch continues at the first unclaimed tile: nothing is redone or skipped, and a tile
//     is still computed by one workgroup in a fixed K order, so the result stays bit-exact.
//
// This is the in-kernel form of the reference's host protocol: executed[] are the counters of
// src/model.cpp:366-396, *stop_index is pStopIndex of scripts/compile/convert_to_blp.py:56-58,
// execute/resume of src/executor.cpp:211-232,280-298 become "reset state + launch" and "launch".
//
// Memory ordering across the 8 XCDs (each has its own L2): a workgroup makes its tile visible
// with an agent-scope release fence before it increments done[l]; a workgroup that has seen
// done[l-1] complete issues an agent-scope acquire fence before it reads layer l-1's output.
#include "gemm_pipe.hpp"
#include "gemm_tile.hpp"
#include "plans.hpp"

#include <vector>

namespace gp {

struct LayerDesc {
    int op, dtype, body, sub, conv, b_kn;
    int total, sx, sy;
    int pad_;
    union {
        MatArgs mat;
        LayoutArgs layout;
        PoolArgs pool;
        EltwiseArgs elt;
        gp_softmax_params softmax;
        gp_layernorm_params ln;
        gp_embed_params embed;
        CopyArgs copy;
    } u;
};

struct ProgArgs {
    const LayerDesc *layers;
    int n_layers;
    int *executed;     // [n_layers] claim counters
    int *done;         // [n_layers] finished-tile counters
    int *cursor;       // first layer that may still have unclaimed tiles (hint for a relaunch)
    int *error;        // set to 1 when a dependency wait exceeded spin_limit
    int *flag;         // host flag, may be null
    int *stop_index;   // never null (an internal word when the caller passes no context)
    int inject_layer, inject_claim;
    int poll_mask;
    unsigned spin_limit;
};

template <typename T>
__device__ __forceinline__ void run_mat(const LayerDesc &d, TileIdx t, T *lds) {
    // Copy the argument block out of the descriptor first: the loads are wave-uniform, and the
    // tile bodies then index registers instead of memory inside their K loops.
    const MatArgs g = d.u.mat;
    constexpr int SBK = sizeof(T) == 4 ? 16 : 32;
    if (d.conv) {
        switch (d.body) {
            case MB_PIPE128: PipeKernel<T, 128, 128, 3, true, false>::run(g, t, lds); break;
            case MB_PIPE64: PipeKernel<T, 64, 64, 4, true, false>::run(g, t, lds); break;
            case MB_PIPE64_SK: PipeKernel<T, 64, 64, 4, true, true>::run(g, t, lds); break;
            case MB_PIPE32_SK: PipeKernel<T, 32, 32, 4, true, true>::run(g, t, lds); break;
        }
    } else if (d.b_kn) {
        switch (d.body) {
            case MB_STAGED128: TileKernel<T, 128, 128, SBK, 2, 2, false, true>::run(g, t, lds); break;
            case MB_STAGED64: TileKernel<T, 64, 64, SBK, 2, 2, false, true>::run(g, t, lds); break;
        }
    } else {
        switch (d.body) {
            case MB_PIPE128: PipeKernel<T, 128, 128, 3, false, false>::run(g, t, lds); break;
            case MB_PIPE64: PipeKernel<T, 64, 64, 4, false, false>::run(g, t, lds); break;
            case MB_PIPE64_SK: PipeKernel<T, 64, 64, 4, false, true>::run(g, t, lds); break;
            case MB_PIPE32_SK: PipeKernel<T, 32, 32, 4, false, true>::run(g, t, lds); break;
        }
    }
}

template <typename T>
__device__ __forceinline__ void run_layer(const LayerDesc &d, TileIdx t, T *lds) {
    switch (d.op) {
        case OP_MAT: run_mat<T>(d, t, lds); break;
        case OP_LAYOUT: {
            const LayoutArgs a = d.u.layout;
            if (d.sub == GP_F32 * 4 + (int)GP_F32 || d.sub / 4 != GP_F32) layout_tile<T, T>(a, t);  // same type in and out
            else layout_tile<float, T>(a, t);                                                  // fp32 "data", 16-bit model
            break;
        }
        case OP_POOL: { const PoolArgs a = d.u.pool; pool_tile<T>(a, t); break; }
        case OP_ELTWISE: { const EltwiseArgs a = d.u.elt; eltwise_tile<T>(a, t); break; }
        case OP_SOFTMAX: { const gp_softmax_params a = d.u.softmax; softmax_tile<T>(a, t); break; }
        case OP_LAYERNORM: {
            const gp_layernorm_params a = d.u.ln;
            if (d.sub == 2) layernorm_tile<T, 2>(a, t);
            else if (d.sub == 8) layernorm_tile<T, 8>(a, t);
            else layernorm_tile<T, 16>(a, t);
            break;
        }
        case OP_EMBED: { const gp_embed_params a = d.u.embed; embed_tile<T>(a, t); break; }
        case OP_COPY: { const CopyArgs a = d.u.copy; copy_tile(a, t); break; }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void program_kernel(ProgArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    T *lds = reinterpret_cast<T *>(lds_raw);
    __shared__ int mailbox[2][2];
    const bool leader = threadIdx.x == 0;
    int layer = 0;
    if (leader) layer = __hip_atomic_load(p.cursor, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int acquired = -1;
    for (int it = 0;; ++it) {
        if (leader) {
            int claim = -1;
            int L = layer;
            for (;;) {
                if (L >= p.n_layers) { claim = -2; break; }  // the model is finished
                if (__hip_atomic_load(p.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != -1) { claim = -1; break; }
                const int total = p.layers[L].total;
                int c = atomicAdd(&p.executed[L], 1);
                if (c >= total) { ++L; continue; }
                claim = c;
                if (L == p.inject_layer && c == p.inject_claim && p.flag)
                    __hip_atomic_store(p.flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                if ((c & p.poll_mask) == 0 && p.flag && __hip_atomic_load(p.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0)
                    atomicCAS(p.stop_index, -1, L);
                // the claimed tile is owed from here on, whatever the flag says
                if (L > 0) {
                    const int need = p.layers[L - 1].total;
                    unsigned spins = 0;
                    while (__hip_atomic_load(&p.done[L - 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < need) {
                        __builtin_amdgcn_s_sleep(1);
                        if (++spins > p.spin_limit) {  // never expected; bounded so that no wave can spin for ever
                            __hip_atomic_store(p.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            claim = -3;
                            break;
                        }
                    }
                    if (claim >= 0) atomicMax(p.cursor, L);
                }
                break;
            }
            layer = L;
            mailbox[it & 1][0] = L;
            mailbox[it & 1][1] = claim;
        }
        __syncthreads();
        const int L = __builtin_amdgcn_readfirstlane(mailbox[it & 1][0]);
        const int claim = __builtin_amdgcn_readfirstlane(mailbox[it & 1][1]);
        if (claim < 0) return;
        if (L != acquired) {
            // first tile of this layer for this workgroup: drop cached lines that may predate
            // the previous layer's writes
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            acquired = L;
        }
        const LayerDesc &d = p.layers[L];
        run_layer<T>(d, decode_tile(claim, d.sx, d.sy), lds);
        // publish the tile: every wave's stores reach device scope, then one count
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        __syncthreads();
        if (leader) __hip_atomic_fetch_add(&p.done[L], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace gp

using namespace gp;

struct gp_program_s {
    int dtype = GP_F32;
    std::vector<LayerDesc> layers;
    LayerDesc *d_layers = nullptr;
    int *d_state = nullptr;  // executed[n] | done[n] | cursor | error | internal stop word | pad
    size_t lds_bytes = 0;
    int max_tiles = 0;
    int resident = 0;        // workgroups the device holds at once for this program
    bool finalized = false;
    int n() const { return (int)layers.size(); }
    int *executed() const { return d_state; }
    int *done() const { return d_state + n(); }
    int *cursor() const { return d_state + 2 * n(); }
    int *error() const { return d_state + 2 * n() + 1; }
    int *own_stop() const { return d_state + 2 * n() + 2; }
};

static int push_mat(gp_program pr, const MatPlan &pl) {
    GP_REQUIRE(pr && !pr->finalized, "program is null or already finalized");
    GP_REQUIRE(pl.dtype == pr->dtype, "layer dtype %d differs from the program's %d", pl.dtype, pr->dtype);
    const bool ok = pl.b_kn ? (pl.body == MB_STAGED128 || pl.body == MB_STAGED64)
                            : (pl.body == MB_PIPE128 || pl.body == MB_PIPE64 || pl.body == MB_PIPE64_SK || pl.body == MB_PIPE32_SK);
    GP_REQUIRE(ok, "matrix kernel body %d is not available inside a program", pl.body);
    LayerDesc d{};
    d.op = OP_MAT; d.dtype = pl.dtype; d.body = pl.body; d.conv = pl.conv; d.b_kn = pl.b_kn;
    d.sx = pl.sx; d.sy = pl.sy;
    long total = (long)pl.sx * pl.sy * pl.batch;
    GP_REQUIRE(total > 0 && total < (1L << 31), "tile count %ld out of range", total);
    d.total = (int)total;
    d.u.mat = pl.g;
    pr->layers.push_back(d);
    if (pl.lds_bytes > pr->lds_bytes) pr->lds_bytes = pl.lds_bytes;
    if (d.total > pr->max_tiles) pr->max_tiles = d.total;
    return GP_SUCC;
}

static int push_elt(gp_program pr, const EltPlan &pl) {
    GP_REQUIRE(pr && !pr->finalized, "program is null or already finalized");
    GP_REQUIRE(pl.op == OP_COPY || pl.dtype == pr->dtype, "layer dtype %d differs from the program's %d", pl.dtype, pr->dtype);
    LayerDesc d{};
    d.op = pl.op; d.dtype = pl.dtype; d.sub = pl.sub; d.sx = pl.sx; d.sy = pl.sy;
    long total = (long)pl.sx * pl.sy;
    GP_REQUIRE(total > 0 && total < (1L << 31), "tile count %ld out of range", total);
    d.total = (int)total;
    static_assert(sizeof(d.u) >= sizeof(pl.u), "descriptor union too small");
    memcpy(&d.u, &pl.u, sizeof(pl.u));
    pr->layers.push_back(d);
    if (d.total > pr->max_tiles) pr->max_tiles = d.total;
    return GP_SUCC;
}

extern "C" int gp_program_create(int dtype, gp_program *out) {
    GP_REQUIRE(out != nullptr, "null program out");
    GP_REQUIRE(dtype == GP_F32 || dtype == GP_F16 || dtype == GP_BF16, "program dtype %d", dtype);
    gp_program_s *p = new gp_program_s();
    p->dtype = dtype;
    *out = p;
    return GP_SUCC;
}

extern "C" int gp_program_destroy(gp_program p) {
    if (!p) return GP_SUCC;
    if (p->d_layers) hipFree(p->d_layers);
    if (p->d_state) hipFree(p->d_state);
    delete p;
    return GP_SUCC;
}

#define GP_ADD_MAT(PLAN) MatPlan pl; int rc = PLAN; return rc ? rc : push_mat(pr, pl);
#define GP_ADD_ELT(PLAN) EltPlan pl; int rc = PLAN; return rc ? rc : push_elt(pr, pl);
extern "C" int gp_program_add_gemm(gp_program pr, const gp_gemm_params *p) { GP_ADD_MAT(plan_gemm(p, &pl)) }
extern "C" int gp_program_add_conv2d(gp_program pr, const gp_conv_params *p) { GP_ADD_MAT(plan_conv2d(p, &pl)) }
extern "C" int gp_program_add_nchw_to_nhwc(gp_program pr, const gp_layout_params *p) { GP_ADD_ELT(plan_layout(p, &pl)) }
extern "C" int gp_program_add_pool2d(gp_program pr, const gp_pool_params *p) { GP_ADD_ELT(plan_pool2d(p, &pl)) }
extern "C" int gp_program_add_eltwise(gp_program pr, const gp_eltwise_params *p) { GP_ADD_ELT(plan_eltwise(p, &pl)) }
extern "C" int gp_program_add_softmax(gp_program pr, const gp_softmax_params *p) { GP_ADD_ELT(plan_softmax(p, &pl)) }
extern "C" int gp_program_add_layernorm(gp_program pr, const gp_layernorm_params *p) { GP_ADD_ELT(plan_layernorm(p, &pl)) }
extern "C" int gp_program_add_embed(gp_program pr, const gp_embed_params *p) { GP_ADD_ELT(plan_embed(p, &pl)) }
extern "C" int gp_program_add_copy(gp_program pr, const void *src, void *dst, size_t bytes) { GP_ADD_ELT(plan_copy(src, dst, (long)bytes, &pl)) }

template <typename T>
static int finalize_typed(gp_program p) {
    auto kern = program_kernel<T>;
    if (p->lds_bytes > 48 * 1024)
        GP_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)p->lds_bytes));
    int per_cu = 0;
    GP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, p->lds_bytes));
    if (per_cu < 1) per_cu = 1;
    p->resident = per_cu * device_cus();
    return GP_SUCC;
}

extern "C" int gp_program_finalize(gp_program p) {
    GP_REQUIRE(p && !p->finalized, "program is null or already finalized");
    GP_REQUIRE(!p->layers.empty(), "empty program");
    const int n = p->n();
    GP_HIP(hipMalloc(&p->d_layers, sizeof(LayerDesc) * n));
    GP_HIP(hipMemcpy(p->d_layers, p->layers.data(), sizeof(LayerDesc) * n, hipMemcpyHostToDevice));
    GP_HIP(hipMalloc(&p->d_state, sizeof(int) * (2 * n + 4)));
    std::vector<int> init(2 * n + 4, 0);
    init[2 * n + 2] = -1;
    GP_HIP(hipMemcpy(p->d_state, init.data(), sizeof(int) * init.size(), hipMemcpyHostToDevice));
    int rc = GP_OUTOFRANGE;
    switch (p->dtype) {
        case GP_F32: rc = finalize_typed<float>(p); break;
        case GP_F16: rc = finalize_typed<_Float16>(p); break;
        case GP_BF16: rc = finalize_typed<__bf16>(p); break;
    }
    if (rc) return rc;
    p->finalized = true;
    return GP_SUCC;
}

extern "C" int gp_program_launch(gp_program p, const gp_preempt_ctx *ctx, int reset, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->finalized, "program is null or not finalized");
    const int n = p->n();
    if (reset) {
        int rc = gp_fill32_async(p->d_state, 0, 2 * n + 2, s);  // executed, done, cursor, error
        if (rc) return rc;
    }
    ProgArgs a{};
    a.layers = p->d_layers; a.n_layers = n;
    a.executed = p->executed(); a.done = p->done(); a.cursor = p->cursor(); a.error = p->error();
    a.spin_limit = 1u << 24;  // tens of seconds: only a broken dependency chain gets there
    long grid = p->max_tiles < p->resident ? p->max_tiles : p->resident;
    if (ctx) {
        GP_REQUIRE(ctx->stop_index != nullptr, "preempt context needs stop_index");
        a.flag = ctx->flag; a.stop_index = ctx->stop_index;
        a.inject_layer = ctx->inject_at >= 0 ? ctx->kernel_id : -1;
        a.inject_claim = ctx->inject_at;
        int pe = ctx->poll_every > 0 ? ctx->poll_every : 8;
        GP_REQUIRE((pe & (pe - 1)) == 0, "poll_every must be a power of two");
        a.poll_mask = pe - 1;
        if (ctx->max_workgroups > 0 && grid > ctx->max_workgroups) grid = ctx->max_workgroups;
    } else {
        a.flag = nullptr; a.stop_index = p->own_stop(); a.inject_layer = -1; a.inject_claim = -1; a.poll_mask = 0;
    }
    if (info) { info->total_tiles = 0; for (auto &l : p->layers) info->total_tiles += l.total; info->shape[0] = n; info->shape[1] = 1; info->shape[2] = 1; info->grid = (int)grid; info->block = 256; }
    switch (p->dtype) {
        case GP_F32: hipLaunchKernelGGL(program_kernel<float>, dim3((unsigned)grid), dim3(256), p->lds_bytes, native(s), a); break;
        case GP_F16: hipLaunchKernelGGL(program_kernel<_Float16>, dim3((unsigned)grid), dim3(256), p->lds_bytes, native(s), a); break;
        case GP_BF16: hipLaunchKernelGGL(program_kernel<__bf16>, dim3((unsigned)grid), dim3(256), p->lds_bytes, native(s), a); break;
    }
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

extern "C" int gp_program_layers(gp_program p, int *n_layers) {
    GP_REQUIRE(p && n_layers, "null program");
    *n_layers = p->n();
    return GP_SUCC;
}

// Blocking read-back of the per-layer counters and the error word (for tests and diagnostics).
extern "C" int gp_program_read_state(gp_program p, int *executed, int *done, int *cursor, int *error) {
    GP_REQUIRE(p && p->finalized, "program is null or not finalized");
    const int n = p->n();
    std::vector<int> st(2 * n + 2);
    GP_HIP(hipMemcpy(st.data(), p->d_state, sizeof(int) * st.size(), hipMemcpyDeviceToHost));
    if (executed) memcpy(executed, st.data(), sizeof(int) * n);
    if (done) memcpy(done, st.data() + n, sizeof(int) * n);
    if (cursor) *cursor = st[2 * n];
    if (error) *error = st[2 * n + 1];
    return GP_SUCC;
}
