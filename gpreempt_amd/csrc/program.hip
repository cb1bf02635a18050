// Whole-model program: every layer of a model runs inside ONE persistent kernel.
//
// Why: with one launch (or graph node) per layer, a preempted model still has to push every
// remaining node through the queue, each leaving at its first flag check; at 4-9 us per node
// that drain, not the kernels, sets the preemption latency (hundreds of microseconds for a
// 160-layer network), and a small high-priority model is launch-bound for the same reason.
// Here the layer list lives in device memory and the resident workgroups walk it themselves:
//
//   * a workgroup claims the next tile of the current layer with one atomic on that layer's
//     claim counter (the per-kernel counters executed[l] of the reference; split over counter
//     groups, see program_kernel) and moves to layer l+1 when the counter is exhausted;
//   * a tile of layer l may be claimed only when done[l-1] == total[l-1], i.e. when every tile
//     of the previous layer has been written (layer-granular dependency); a workgroup checks
//     that BEFORE it takes the ticket, so it never owes a tile it cannot run;
//   * it polls the preempt flag exactly as the per-kernel dispatcher does (tile_loop.hpp); when
//     the flag is up it records the layer in *stop_index and leaves.  Everything it had claimed
//     is finished first, so afterwards every claim made is a finished tile and a relaunch
//     continues at the first unclaimed tile of each layer: nothing is redone or skipped, and a tile
//     is still computed by one workgroup in a fixed K order, so the result stays bit-exact.
//
// This is the in-kernel form of the reference's host protocol: executed[] are the counters of
// src/model.cpp:366-396, *stop_index is pStopIndex of scripts/compile/convert_to_blp.py:56-58,
// execute/resume of src/executor.cpp:211-232,280-298 become "reset state + launch" and "launch".
//
// Memory ordering across the 8 XCDs (each has its own L2): the tile bodies store their outputs
// with agent-scope stores (out_store.hpp), a workgroup waits for its stores to complete before
// it increments done[l], and a workgroup that has seen done[l-1] complete issues an agent-scope
// acquire fence (cache invalidate) before it reads layer l-1's output.
// every output store of the tile bodies becomes an agent-scope store in this translation unit
#ifndef GP_EXP_PLAIN_STORES
#define GP_COHERENT_STORES 1
#endif
#include "gemm_pipe.hpp"
#include "gemm_tile.hpp"
#include "plans.hpp"

#include <vector>

namespace gp {

struct LayerDesc {
    int op, dtype, body, sub, conv, b_kn;
    int total, sx, sy;
    int groups;  // counter groups that own a non-empty slice of this layer
    union {
        MatArgs mat;
        LayoutArgs layout;
        PoolArgs pool;
        EltwiseArgs elt;
        gp_softmax_params softmax;
        gp_layernorm_params ln;
        gp_embed_params embed;
        CopyArgs copy;
        AttnArgs attn;
    } u;
};

struct ProgArgs {
    const LayerDesc *layers;
    int n_layers;
    int n_groups;      // counter groups (power of two, <= workgroups launched)
    int poll_groups;   // groups whose claims read the host flag
    int *claimed;      // [n_layers][n_groups] claim counters, one per 64-byte line
    int *done;         // [n_layers][n_groups] finished-tile counters, one per 64-byte line
    int *ldone;        // [n_layers] groups whose slice is finished, one per 64-byte line
    int *error;        // set to 1 when a dependency wait exceeded spin_limit
    int *flag;         // host flag, may be null
    int *stop_index;   // never null (an internal word when the caller passes no context)
    int inject_layer, inject_claim;
    int poll_mask;
    unsigned spin_limit;
    int *exited;       // device counter of workgroups that have left this launch
    int *left_host;    // optional host-visible word: set to `launch_tag` by the last workgroup to leave
    int launch_tag;
    unsigned long long *prof;  // optional: 4 cycle counters per workgroup (claim, acquire, body, publish)
    unsigned long long *stamps;  // optional: time stamps of the preemption (tile_loop.hpp, "time stamps")
};

template <typename T>
__device__ __forceinline__ void run_mat(const LayerDesc &d, TileIdx t, T *lds) {
    // Copy the argument block out of the descriptor first: the loads are wave-uniform, and the
    // tile bodies then index registers instead of memory inside their K loops.
    const MatArgs g = d.u.mat;
    constexpr int SBK = sizeof(T) == 4 ? 16 : 32;
    if (d.conv) {
        switch (d.body) {
            case MB_PIPE128: PipeKernel<T, 128, 128, 2, true, false>::run(g, t, lds); break;
            case MB_PIPE64: PipeKernel<T, 64, 64, 4, true, false>::run(g, t, lds); break;
            case MB_PIPE64_SK: PipeKernel<T, 64, 64, 4, true, true>::run(g, t, lds); break;
            case MB_PIPE32_SK: PipeKernel<T, 32, 32, 4, true, true>::run(g, t, lds); break;
        }
    } else if (d.b_kn) {
        switch (d.body) {
            case MB_STAGED64: TileKernel<T, 64, 64, SBK, 2, 2, false, true>::run(g, t, lds); break;
        }
    } else {
        switch (d.body) {
            case MB_PIPE128: PipeKernel<T, 128, 128, 2, false, false>::run(g, t, lds); break;
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
            if (d.sub == (2 | kLnTwoRows)) layernorm_tile<T, 2, 2>(a, t);
            else if (d.sub == 2) layernorm_tile<T, 2>(a, t);
            else if (d.sub == 8) layernorm_tile<T, 8>(a, t);
            else layernorm_tile<T, 16>(a, t);
            break;
        }
        case OP_EMBED: { const gp_embed_params a = d.u.embed; embed_tile<T>(a, t); break; }
        case OP_COPY: { const CopyArgs a = d.u.copy; copy_tile(a, t); break; }
        case OP_ATTENTION:
            if constexpr (sizeof(T) == 2) { const AttnArgs a = d.u.attn; attention_tile_split<T, 4>(a, t, lds); }  // seq <= 128 only; the same body as the stand-alone kernel, so that both paths give the same bits
            break;
    }
}

// Counters are spread over NG "groups" (workgroup w belongs to group w % NG): device-scope
// atomics on ONE address complete at about one per 40 ns on MI355X, so a single claim counter
// (and a single completion counter) shared by ~500 resident workgroups would cost 20-40 us per
// layer.  Each layer's tiles are split into NG contiguous slices; group g claims from its own
// counter claimed[l][g] and counts finished tiles in its own done[l][g].  A layer is complete
// when every group's done count has reached its slice size.
constexpr int CTR_STRIDE = 16;  // ints: one counter per 64-byte line

__device__ __forceinline__ int slice_begin(int total, int g, int ng) { return (int)((long)total * g / ng); }

#ifndef GP_EXP_WGS
#define GP_EXP_WGS 2
#endif
template <typename T>
__global__ __launch_bounds__(256, GP_EXP_WGS) void program_kernel(ProgArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    T *lds = reinterpret_cast<T *>(lds_raw);
    __shared__ int mailbox[2][2];
    const int lane = threadIdx.x;  // only wave 0 uses it as a lane index
    const bool wave0 = threadIdx.x < 64;
    const bool leader = threadIdx.x == 0;
    const int ng = p.n_groups;
    const int grp = blockIdx.x % ng;
    int layer = 0;
    int acquired = -1;
    int ready_upto = 0;   // wave 0: every layer below this one is known to be complete
    int stop_word = -1;   // wave 0: the stop word, read while the previous tile runs
    if (wave0) {
        stop_word = __hip_atomic_load(p.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // A relaunch after a stop: skip the layers whose slice this group has already handed out,
        // 64 layers per look.
        for (int base = 0; base < p.n_layers; base += 64) {
            int l = base + lane;
            bool open = false;
            if (l < p.n_layers) {
                const int total = p.layers[l].total;
                const int size = slice_begin(total, grp + 1, ng) - slice_begin(total, grp, ng);
                open = size > 0 && __hip_atomic_load(p.claimed + ((long)l * ng + grp) * CTR_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < size;
            }
            unsigned long long m = __builtin_amdgcn_ballot_w64(open);
            if (m) { layer = base + __builtin_ctzll(m); break; }
            layer = p.n_layers;
        }
    }
    unsigned long long t_claim = 0, t_acq = 0, t_body = 0, t_pub = 0, t0 = 0;
    for (int it = 0;; ++it) {
        if (p.prof) t0 = wall_clock64();
        if (wave0) {  // the whole first wave takes part so that the NG completion counters are read in one go
            // A tile of layer L is claimed only once layer L-1 is known to be complete, so a
            // workgroup never owes a tile it cannot run: when a stop is requested, workgroups
            // that are waiting for a layer to complete simply leave.
            int claim = -1, L = layer;
            unsigned spins = 0;
            for (;;) {
                if (stop_word != -1) {
                    if (leader) record_stop(p.stop_index, L < p.n_layers ? L : p.n_layers - 1, p.stamps);
                    claim = -1;
                    break;
                }
                if (L >= p.n_layers) { claim = -2; break; }  // this group's share of the model is finished
                const int total = p.layers[L].total;
                const int begin = slice_begin(total, grp, ng), size = slice_begin(total, grp + 1, ng) - begin;
                if (size == 0) { ++L; continue; }
                if (L > ready_upto) {
                    // one word per layer says how many groups have finished their slice
                    const int have = __hip_atomic_load(p.ldone + (long)(L - 1) * CTR_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (have < p.layers[L - 1].groups) {
                        // not yet: nothing is owed, so look again (and notice a stop request)
                        __builtin_amdgcn_s_sleep(8);
                        if (++spins > p.spin_limit) {  // never expected; bounded so that no wave can spin for ever
                            if (leader) __hip_atomic_store(p.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            claim = -3;
                            break;
                        }
                        stop_word = __hip_atomic_load(p.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        // a few workgroups use their idle time to watch the host flag, so a stop is
                        // noticed within microseconds even between the claims that normally read it
                        if (blockIdx.x < 4 && p.flag && stop_word == -1) {
                            int f = 0;
                            if (leader) f = __hip_atomic_load(p.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                            if (__builtin_amdgcn_readfirstlane(f) != 0) {
                                if (leader) record_stop(p.stop_index, L, p.stamps);
                                stop_word = L;
                            }
                        }
                        continue;
                    }
                    ready_upto = L;  // completion is monotone: layers 0..L-1 stay complete
                }
                int c = 0;
                if (leader) c = atomicAdd(p.claimed + ((long)L * ng + grp) * CTR_STRIDE, 1);
                c = __builtin_amdgcn_readfirstlane(c);
                if (c >= size) { ++L; continue; }  // this group's slice of the layer is handed out
                claim = begin + c;                 // tile index within the layer; owed and runnable from here on
                if (leader) {
                    if (L == p.inject_layer && claim == p.inject_claim && p.flag)
                        __hip_atomic_store(p.flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    if (grp < p.poll_groups && (c & p.poll_mask) == 0 && p.flag &&
                        __hip_atomic_load(p.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0)
                        record_stop(p.stop_index, L, p.stamps);
                    stamp_first_claim(p.stamps);
                }
                break;
            }
            layer = L;
            if (leader) {
                mailbox[it & 1][0] = L;
                mailbox[it & 1][1] = claim;
            }
        }
        __syncthreads();
        const int L = __builtin_amdgcn_readfirstlane(mailbox[it & 1][0]);
        const int claim = __builtin_amdgcn_readfirstlane(mailbox[it & 1][1]);
        if (p.prof) { unsigned long long t1 = wall_clock64(); t_claim += t1 - t0; t0 = t1; }
        if (claim < 0) {
            if (leader && p.stamps) stamp_exit_leader(p.stamps);
            if (leader && p.left_host) {
                // every workgroup of this launch has stopped touching the model's buffers once the
                // count is complete: tell the host without waiting for the queue to report it
                if (atomicAdd(p.exited, 1) == (int)gridDim.x - 1)
                    __hip_atomic_store(p.left_host, p.launch_tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            if (p.prof && leader) { p.prof[blockIdx.x * 4 + 0] = t_claim; p.prof[blockIdx.x * 4 + 1] = t_acq; p.prof[blockIdx.x * 4 + 2] = t_body; p.prof[blockIdx.x * 4 + 3] = t_pub; }
            return;
        }
        if (L != acquired) {
            // first tile of this layer for this workgroup: drop cached lines that may predate
            // the previous layer's writes
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            acquired = L;
        }
        if (p.prof) { unsigned long long t1 = wall_clock64(); t_acq += t1 - t0; t0 = t1; }
        // issue the read for the next claim now; it is consumed after the tile
        if (wave0) stop_word = __hip_atomic_load(p.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const LayerDesc &d = p.layers[L];
        run_layer<T>(d, decode_tile(claim, d.sx, d.sy), lds);
        if (p.prof) { unsigned long long t1 = wall_clock64(); t_body += t1 - t0; t0 = t1; }
        // publish the tile: every wave's (agent-scope) stores have completed, then one count
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (leader) {
            const int total = p.layers[L].total;
            const int size = slice_begin(total, grp + 1, ng) - slice_begin(total, grp, ng);
            int before = __hip_atomic_fetch_add(p.done + ((long)L * ng + grp) * CTR_STRIDE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before == size - 1)  // last tile of this group's slice: one more group is finished with the layer
                __hip_atomic_fetch_add(p.ldone + (long)L * CTR_STRIDE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (p.prof) { unsigned long long t1 = wall_clock64(); t_pub += t1 - t0; t0 = t1; }
    }
}

}  // namespace gp

using namespace gp;

struct gp_program_s {
    int dtype = GP_F32;
    std::vector<LayerDesc> layers;
    LayerDesc *d_layers = nullptr;
    int launches = 0;
    int *d_state = nullptr;  // error | internal stop word | exited | pad.. (16 ints) | claimed[n][NG] | done[n][NG] | ldone[n], one counter per line
    unsigned long long *d_prof = nullptr;
    int n_groups = 1;
    size_t lds_bytes = 0;
    int max_tiles = 0;
    int resident = 0;        // workgroups the device holds at once for this program
    bool finalized = false;
    int n() const { return (int)layers.size(); }
    int *error() const { return d_state; }
    int *own_stop() const { return d_state + 1; }
    int *exited() const { return d_state + 2; }
    int *claimed() const { return d_state + 16; }
    int *done() const { return d_state + 16 + (size_t)n() * n_groups * 16; }
    int *ldone() const { return d_state + 16 + (size_t)2 * n() * n_groups * 16; }
    size_t counter_ints() const { return ((size_t)2 * n() * n_groups + n()) * 16; }
};

static int push_mat(gp_program pr, const MatPlan &pl) {
    GP_REQUIRE(pr && !pr->finalized, "program is null or already finalized");
    GP_REQUIRE(pl.dtype == pr->dtype, "layer dtype %d differs from the program's %d", pl.dtype, pr->dtype);
    const bool ok = pl.b_kn ? (pl.body == MB_STAGED64)
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
    // inside the program the 128x128 kernel runs with two stages (64 KB) so that two workgroups fit a compute unit
    size_t lds = pl.body == MB_PIPE128 ? (size_t)2 * (128 + 128) * 128 : pl.lds_bytes;
    if (lds > pr->lds_bytes) pr->lds_bytes = lds;
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
    if (pl.lds_bytes > pr->lds_bytes) pr->lds_bytes = pl.lds_bytes;
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
    if (p->d_prof) hipFree(p->d_prof);
    delete p;
    return GP_SUCC;
}

#define GP_ADD_MAT(PLAN) MatPlan pl; int rc = PLAN; return rc ? rc : push_mat(pr, pl);
// the 256x256 body needs 128 KB of LDS and is not part of the program kernel: fall back to 128x128
template <class P, class PlanFn>
static int add_mat_layer(gp_program pr, const P *p, PlanFn plan) {
    MatPlan pl;
    int rc = plan(p, &pl);
    if (rc) return rc;
    if (pl.body == MB_PIPE256) {
        P q = *p;
        q.tile_m = q.tile_n = 128;
        rc = plan(&q, &pl);
        if (rc) return rc;
    }
    if (is_wide_body(pl.body)) {
        // 8 or 16 wavefronts per tile do not fit the program's 256-thread workgroups: the
        // four-wavefront split-K bodies stand in (the same summation, hence the same bits)
        P q = *p;
        q.variant = GP_MAT_PIPE_SPLITK;
        q.tile_m = q.tile_n = 0;
        rc = plan(&q, &pl);
        if (rc) return rc;
    }
    return push_mat(pr, pl);
}
#define GP_ADD_ELT(PLAN) EltPlan pl; int rc = PLAN; return rc ? rc : push_elt(pr, pl);
extern "C" int gp_program_add_gemm(gp_program pr, const gp_gemm_params *p) { GP_REQUIRE(p, "null params"); return add_mat_layer(pr, p, plan_gemm); }
extern "C" int gp_program_add_conv2d(gp_program pr, const gp_conv_params *p) { GP_REQUIRE(p, "null params"); return add_mat_layer(pr, p, plan_conv2d); }
extern "C" int gp_program_add_nchw_to_nhwc(gp_program pr, const gp_layout_params *p) { GP_ADD_ELT(plan_layout(p, &pl)) }
extern "C" int gp_program_add_pool2d(gp_program pr, const gp_pool_params *p) { GP_ADD_ELT(plan_pool2d(p, &pl)) }
extern "C" int gp_program_add_eltwise(gp_program pr, const gp_eltwise_params *p) { GP_ADD_ELT(plan_eltwise(p, &pl)) }
extern "C" int gp_program_add_softmax(gp_program pr, const gp_softmax_params *p) { GP_ADD_ELT(plan_softmax(p, &pl)) }
extern "C" int gp_program_add_layernorm(gp_program pr, const gp_layernorm_params *p) { GP_ADD_ELT(plan_layernorm(p, &pl)) }
extern "C" int gp_program_add_embed(gp_program pr, const gp_embed_params *p) { GP_ADD_ELT(plan_embed(p, &pl)) }
extern "C" int gp_program_add_attention(gp_program pr, const gp_attention_params *p) {
    // the program kernel carries the 128-key body only: the longer classes keep up to 256 score
    // registers per lane, which would push every layer of the program into scratch memory
    GP_REQUIRE(p && p->seq <= 128, "program attention: seq must be <= 128 (use unfused layers beyond)");
    GP_ADD_ELT(plan_attention(p, &pl))
}
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
    long all = 0;
    for (LayerDesc &l : p->layers) all += l.total;
    GP_REQUIRE(all < (1L << 30), "program has too many tiles (%ld)", all);
    int rc = GP_OUTOFRANGE;
    switch (p->dtype) {
        case GP_F32: rc = finalize_typed<float>(p); break;
        case GP_F16: rc = finalize_typed<_Float16>(p); break;
        case GP_BF16: rc = finalize_typed<__bf16>(p); break;
    }
    if (rc) return rc;
    // counter groups: a power of two, at most 32, never more than the workgroups that will run
    long grid = p->max_tiles < p->resident ? p->max_tiles : p->resident;
    int ng = 1;
    while (ng * 2 <= 32 && ng * 2 <= grid) ng *= 2;
    p->n_groups = ng;
    for (LayerDesc &l : p->layers) l.groups = l.total < ng ? l.total : ng;
    GP_HIP(hipMalloc(&p->d_layers, sizeof(LayerDesc) * n));
    GP_HIP(hipMemcpy(p->d_layers, p->layers.data(), sizeof(LayerDesc) * n, hipMemcpyHostToDevice));
    std::vector<int> init(16 + p->counter_ints(), 0);
    init[1] = -1;
    GP_HIP(hipMalloc(&p->d_state, sizeof(int) * init.size()));
    GP_HIP(hipMemcpy(p->d_state, init.data(), sizeof(int) * init.size(), hipMemcpyHostToDevice));
    if (getenv("GPREEMPT_PROGRAM_PROF")) {
        GP_HIP(hipMalloc(&p->d_prof, sizeof(unsigned long long) * 4 * 4096));
        GP_HIP(hipMemset(p->d_prof, 0, sizeof(unsigned long long) * 4 * 4096));
    }
    p->finalized = true;
    return GP_SUCC;
}

extern "C" int gp_program_launch(gp_program p, const gp_preempt_ctx *ctx, int reset, gp_stream s, gp_launch_info *info) {
    GP_REQUIRE(p && p->finalized, "program is null or not finalized");
    const int n = p->n();
    if (reset) {
        int rc = gp_fill32_async(p->error(), 0, 1, s);
        if (rc) return rc;
        rc = gp_fill32_async(p->claimed(), 0, p->counter_ints(), s);  // claim and completion counters
        if (rc) return rc;
    }
    ProgArgs a{};
    a.layers = p->d_layers; a.n_layers = n;
    a.n_groups = p->n_groups; a.poll_groups = p->n_groups < 4 ? p->n_groups : 4;
    if (ctx && ctx->poll_every == 1) a.poll_groups = p->n_groups;  // the flag is cheap to read: every group looks
    a.claimed = p->claimed(); a.done = p->done(); a.ldone = p->ldone(); a.error = p->error();
    a.spin_limit = 1u << 22;  // seconds: only a broken dependency chain gets there
    a.exited = p->exited();
    a.left_host = ctx ? ctx->left_host : nullptr;
    a.launch_tag = ++p->launches;
    if (a.left_host) { int rc = gp_fill32_async(p->exited(), 0, 1, s); if (rc) return rc; }
    a.prof = p->d_prof;
    a.stamps = ctx ? ctx->stamps : nullptr;
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
    if (grid < p->n_groups) grid = p->n_groups;  // every group needs at least one workgroup to serve its slices
    if (info) { info->total_tiles = 0; for (auto &l : p->layers) info->total_tiles += l.total; info->shape[0] = n; info->shape[1] = a.launch_tag; info->shape[2] = 1; info->grid = (int)grid; info->block = 256; info->fixed_claims = 0; info->front = 0; }
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
    const int n = p->n(), ng = p->n_groups;
    std::vector<int> st(16 + p->counter_ints());
    GP_HIP(hipMemcpy(st.data(), p->d_state, sizeof(int) * st.size(), hipMemcpyDeviceToHost));
    const int *cl = st.data() + 16, *dn = st.data() + 16 + (size_t)n * ng * 16;
    long handed = 0;
    for (int l = 0; l < n; ++l) {
        long ex = 0, dd = 0;
        const int total = p->layers[l].total;
        for (int g = 0; g < ng; ++g) {
            long size = (long)total * (g + 1) / ng - (long)total * g / ng;
            long c = cl[((size_t)l * ng + g) * 16];
            ex += c > size ? size : c;  // the counter overshoots by one per workgroup that found the slice handed out
            dd += dn[((size_t)l * ng + g) * 16];
        }
        if (executed) executed[l] = (int)ex;
        if (done) done[l] = (int)dd;
        handed += ex;
    }
    if (cursor) *cursor = (int)handed;
    if (error) *error = st[0];
    if (p->d_prof) {  // diagnostic: where the workgroups of the last launch spent their time (100 MHz ticks)
        std::vector<unsigned long long> pr(4 * 4096);
        GP_HIP(hipMemcpy(pr.data(), p->d_prof, sizeof(unsigned long long) * pr.size(), hipMemcpyDeviceToHost));
        double sum[4] = {0, 0, 0, 0};
        int wgs = 0;
        for (int w = 0; w < 4096; ++w) if (pr[w * 4] | pr[w * 4 + 2]) { ++wgs; for (int k = 0; k < 4; ++k) sum[k] += (double)pr[w * 4 + k]; }
        if (wgs) fprintf(stderr, "program profile over %d workgroups (us per workgroup): claim %.1f acquire %.1f body %.1f publish %.1f\n",
                         wgs, sum[0] / wgs / 100, sum[1] / wgs / 100, sum[2] / wgs / 100, sum[3] / wgs / 100);
    }
    return GP_SUCC;
}
