// Tile bodies of the graph workloads (connected components, BFS, PageRank, SSSP over a CSR graph
// with 64-bit offsets and 64-bit neighbour ids), the reference's second family of non-DNN
// preemptible kernels (src/workloads/graphcompute.tr.cu: cc_kernel_coalesce :88-127,
// bfs_kernel_coalesce :218-241, pr_initialize :327-335, pr_kernel_coalesce :367-384, pr_update
// :416-425, sssp_kernel_coalesce :540-561, sssp_update :592-603; derived from EMOGI).
//
// Edge-parallel kernels give one vertex to a group of 16, 32 or 64 lanes of a wavefront (the
// caller picks the width nearest the average degree; the reference always uses a 32-lane warp):
// the group walks the vertex's neighbour list from the 128-byte boundary at or below its first
// edge, so every access of a group is a run of whole cache lines.  A tile is 256 threads = 4 to
// 16 vertices.  Vertex-parallel kernels give one vertex to one lane, 256 per tile.
//
// The reference wraps these kernels by hand with a reduced dispatcher (no stop index, no kernel
// id) and a host loop of `goto resume`; here they run under the same dispatcher as every other
// kernel.  PageRank's push (`atomicAdd` into the neighbour's residual) is the non-idempotent one:
// a tile run twice would add its contribution twice.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/gpreempt_hip.h"
#include "tile_loop.hpp"

namespace gp {

constexpr int GR_TILE = 256;
constexpr int GR_WAVES = GR_TILE / 64;
constexpr unsigned long long GR_ALIGN = ~0xfULL;  // 16 neighbour ids = 128 bytes
constexpr unsigned int GR_INF = 0xFFFFFFFFu;

__host__ __device__ inline bool graph_kernel_is_edge_parallel(int k) {
    return k == GP_GRAPH_BFS_STEP || k == GP_GRAPH_CC_STEP || k == GP_GRAPH_PR_PUSH || k == GP_GRAPH_SSSP_RELAX;
}
__host__ __device__ inline int graph_lanes(int lanes_per_vertex) { return lanes_per_vertex == 16 || lanes_per_vertex == 32 ? lanes_per_vertex : 64; }
__host__ __device__ inline long graph_kernel_tiles(int k, unsigned long long vertex_count, int lanes) {
    const unsigned long long per_tile = graph_kernel_is_edge_parallel(k) ? GR_TILE / lanes : GR_TILE;
    return (long)((vertex_count + per_tile - 1) / per_tile);
}

template <int KIND, int LANES>
__device__ __forceinline__ void graph_tile(const gp_graph_params &p, TileIdx t) {
    typedef unsigned long long u64;
    if constexpr (KIND == GP_GRAPH_PR_INIT || KIND == GP_GRAPH_PR_UPDATE || KIND == GP_GRAPH_SSSP_UPDATE || KIND == GP_GRAPH_CC_INIT) {
        const u64 v = (u64)t.x * GR_TILE + threadIdx.x;
        if (v >= p.vertex_count) return;
        if constexpr (KIND == GP_GRAPH_CC_INIT) {  // CC::compute's upload of 0..n-1 and its two memsets (graphcompute.tr.cu:143-148)
            p.comp[v] = v;
            p.active[v] = 1;
            p.next_active[v] = 0;
        } else if constexpr (KIND == GP_GRAPH_PR_INIT) {
            const u64 deg = p.vertex_list[v + 1] - p.vertex_list[v];
            p.value[v] = 1.0f - p.alpha;
            p.delta[v] = deg ? (1.0f - p.alpha) * p.alpha / (float)deg : 0.f;  // a sink has nobody to push to
            p.residual[v] = 0.0f;
            p.active[v] = 1;
        } else if constexpr (KIND == GP_GRAPH_PR_UPDATE) {
            const float r = p.residual[v];
            if (r > p.tolerance) {
                const u64 deg = p.vertex_list[v + 1] - p.vertex_list[v];
                p.value[v] += r;
                p.delta[v] = deg ? r * p.alpha / (float)deg : 0.f;
                p.residual[v] = 0.0f;
                p.active[v] = 1;
                *p.changed = 1;
            }
        } else {
            const unsigned int nc = p.new_cost[v];
            if (nc < p.cost[v]) {
                p.cost[v] = nc;
                p.active[v] = 1;
                *p.changed = 1;
            }
        }
    } else {
        const u64 v = (u64)t.x * (GR_TILE / LANES) + threadIdx.x / LANES;
        const unsigned lane = threadIdx.x % LANES;
        if (v >= p.vertex_count) return;
        if constexpr (KIND == GP_GRAPH_BFS_STEP) {
            if (p.label[v] != p.level) return;
        } else {
            if (!p.active[v]) return;
        }
        const u64 start = p.vertex_list[v], end = p.vertex_list[v + 1];
        const u64 from = start & GR_ALIGN;
        if constexpr (KIND == GP_GRAPH_BFS_STEP) {
            for (u64 i = from + lane; i < end; i += LANES) {
                if (i < start) continue;
                const u64 next = p.edge_list[i];
                if (p.label[next] == GR_INF) {
                    p.label[next] = p.level + 1;
                    *p.changed = 1;
                }
            }
        } else if constexpr (KIND == GP_GRAPH_CC_STEP) {
            for (u64 i = from + lane; i < end; i += LANES) {
                if (i < start) continue;
                const u64 comp_src = p.comp[v];
                const u64 next = p.edge_list[i];
                const u64 comp_next = p.comp[next];
                if (comp_next != comp_src) {
                    // the smaller label wins on whichever end of the edge holds the larger one
                    const bool fwd = comp_src < comp_next;
                    const u64 target = fwd ? next : v;
                    atomicMin(&p.comp[target], fwd ? comp_src : comp_next);
                    p.next_active[target] = 1;
                    *p.changed = 1;
                }
            }
        } else if constexpr (KIND == GP_GRAPH_PR_PUSH) {
            const float d = p.delta[v];
            for (u64 i = from + lane; i < end; i += LANES) {
                if (i < start) continue;
                atomicAdd(&p.residual[p.edge_list[i]], d);
            }
            if (lane == 0) p.active[v] = 0;
        } else {  // GP_GRAPH_SSSP_RELAX
            const unsigned int c = p.new_cost[v];
            for (u64 i = from + lane; i < end; i += LANES) {
                if (i < start) continue;
                const u64 next = p.edge_list[i];
                const unsigned int via = c + p.weight_list[i];
                if (p.new_cost[next] > via) atomicMin(&p.new_cost[next], via);
            }
            if (lane == 0) p.active[v] = 0;
        }
    }
}

template <int KIND, int LANES, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(GR_TILE) void graph_kernel(gp_graph_params p, BlpArgs blp) {
    tiles<LOOP>(blp, [&](TileIdx t) { graph_tile<KIND, LANES>(p, t); });
}

}  // namespace gp
