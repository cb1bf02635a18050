// Shared host-side helpers of the device layer: error capture, handle types, dtype helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include "../../include/gpreempt_hip.h"
#include "tile_loop.hpp"

struct gp_stream_s { hipStream_t s; int priority; };
struct gp_event_s { hipEvent_t e; };
struct gp_graph_s { hipGraph_t g; hipGraphExec_t x; };

namespace gp {

void set_error(const char *fmt, ...);
int device_cus();

#define GP_HIP(call)                                                                           \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess) {                                                                \
            gp::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            return GP_FAIL;                                                                    \
        }                                                                                      \
    } while (0)

#define GP_REQUIRE(cond, ...)                                                                  \
    do {                                                                                       \
        if (!(cond)) {                                                                         \
            gp::set_error(__VA_ARGS__);                                                        \
            return GP_OUTOFRANGE;                                                              \
        }                                                                                      \
    } while (0)

inline hipStream_t native(gp_stream s) { return s ? s->s : nullptr; }

inline size_t dtype_size(int dt) {
    switch (dt) {
        case GP_F32: return 4; case GP_F16: return 2; case GP_BF16: return 2;
        case GP_I32: return 4; case GP_I64: return 8; default: return 0;
    }
}

// Where claims go through several counters, counters 0..3 read the flag; the others need the lengths of
// those four slices to tell when to take over (reads_flag in tile_loop.hpp).  The slices depend on the
// grid, so a launcher that changes the grid after plan_launch calls this again.
inline void set_poll_slices(BlpArgs *blp, int grid) {
    const int ng = blp->groups;
    for (int g = 0; g < 4; ++g)
        blp->poll_n[g] = ng > 1 && g < ng ? group_slice_begin(blp->total, g + 1, ng, grid) - group_slice_begin(blp->total, g, ng, grid) : 0;
}

// Resolves the launch geometry of one preemptible kernel, as Model::add_block_preemption_param
// does in the reference (src/model.cpp:366-396): total_block = sx*sy*sz; persistent grid =
// min(total_block, resident workgroups the device can hold); a NULL context keeps one
// workgroup per tile.
template <class Kernel>
int plan_launch(Kernel kernel, int block, size_t lds_bytes, int sx, int sy, int sz,
                const gp_preempt_ctx *ctx, BlpArgs *blp, int *grid, gp_launch_info *info, int batch = 1, int waves = 1, bool long_tiles = false) {
    long tiles = (long)sx * sy * sz;
    GP_REQUIRE(tiles > 0 && tiles < (1L << 31), "tile count %ld out of range", tiles);
    if (batch < 1) batch = 1;
    long total = (tiles + batch - 1) / batch;  // claims
    blp->total = (int)total; blp->sx = sx; blp->sy = sy; blp->order = 0; blp->ckpt = nullptr;
    blp->batch = batch; blp->tiles = (int)tiles;
    if (ctx) {
        GP_REQUIRE(ctx->executed != nullptr && ctx->stop_index != nullptr, "preempt context needs executed and stop_index");
        blp->flag = ctx->flag; blp->stop_index = ctx->stop_index; blp->executed = ctx->executed;
        blp->kernel_id = ctx->kernel_id; blp->inject_at = ctx->inject_at; blp->stamps = ctx->stamps;
        blp->started = ctx->started_host; blp->started_seq = ctx->started_seq;
        GP_REQUIRE(ctx->fresh >= 0 && ctx->fresh <= 2, "fresh is 0, 1 or 2");
        blp->fresh = ctx->fresh;
        int pe = ctx->poll_every > 0 ? ctx->poll_every : 8;
        GP_REQUIRE((pe & (pe - 1)) == 0, "poll_every must be a power of two");
        blp->poll_mask = pe - 1;
        int ng = ctx->counter_groups > 1 ? ctx->counter_groups : 1;
        GP_REQUIRE((ng & (ng - 1)) == 0 && ng <= 64, "counter_groups must be a power of two <= 64");
        blp->groups = ng;
        int per_cu = 0;
        GP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block, lds_bytes));
        if (per_cu < 1) per_cu = 1;
        long resident = (long)per_cu * device_cus();
        if (ctx->max_workgroups > 0 && resident > ctx->max_workgroups) resident = ctx->max_workgroups;
        *grid = (int)(total < resident ? total : resident);
        // Up to `waves` times the resident workgroups, a workgroup per claim (fixed claims, started
        // by the hardware as others retire) beats a persistent grid that claims through the
        // counters: 4 % on ResNet-152 b8.  The caller allows it where tiles are short; with
        // VGG-16 b16's 128 x 128 tiles it lengthened the drain (p99 130 -> 178 us).
        // Long tiles that can be given up (see below) always get a workgroup per claim, up to eight rounds of them: a
        // persistent grid would finish the tiles it is in.  (Not where the front workgroup, which keeps one place until
        // the launch ends, would cost a round of its own: a compute unit holds one workgroup of the kernel and the
        // rounds are full.)
        bool long_ok = long_tiles && ctx->done && ctx->flag && blp->poll_mask != 0 && ng > 1;
        if (long_ok && per_cu < 2 && total > resident && (ctx->max_workgroups != 0 || (total + resident - 2) / (resident - 1) != (total + resident - 1) / resident))
            long_ok = false;
        if (long_ok && waves < 8) waves = 8;
        if (ng > 1 && ctx->max_workgroups == 0 && total > resident && total <= (long)waves * resident && total + 8 <= (long)ng * kFixedClaimBits)
            *grid = (int)total;
        if (*grid < blp->groups) *grid = blp->groups;  // every counter needs a workgroup to serve its slice
        // a launch with fixed claims gets four workgroups more, which only read the flag (tile_loop.hpp)
        blp->spare = 0;
        // (only when the whole grid, the four included, starts at once: the last workgroups of a longer grid start last,
        // and a flag read at the end of a kernel stops nothing; there every eighth workgroup of the
        // first four groups reads it after its claim, as in the general loop)
        if (ctx->flag && blp->poll_mask != 0 && *grid + 4 <= resident && fixed_claims(true, ng, *grid, (int)total) && fixed_claims(true, ng, *grid + 4, (int)total)) {
            blp->spare = 4;
            *grid += 4;
        }
        // An eager start (fresh = 2, tile_fixed_early) makes a kernel queued behind a stop leave one operand
        // fetch later per round of workgroups: kept for launches whose workgroups all start at once, where that
        // is half a microsecond; a launch of several rounds waits for the stop index as before (VGG-16 b16 next
        // to two higher levels: drain 41 / 77 us mean / p99 with the wait, 48 / 94 without).
        if (blp->fresh > 1 && (long)*grid > resident) blp->fresh = 1;
        // A launch with more claims than the device holds workgroups gets eight workgroups in front of its workers, the
        // first of which reads the flag for as long as claims are still being made (front_workgroup in tile_loop.hpp);
        // the workers then leave the flag alone.  (Kept out of the slices' arithmetic: the workers are counted without them.)
        // (Not where a compute unit holds a single workgroup of this kernel: the one that stays would cost a whole
        // compute unit, a fifth round of tiles for 8192^3 on 256 x 256 tiles.)
        blp->front = 0; blp->done = nullptr; blp->done_target = 0;
#ifndef GP_NO_FRONT
        if (ctx->flag && blp->poll_mask != 0 && blp->spare == 0 && ng > 1 && per_cu >= 2 && total > resident &&
            (!fixed_claims(true, ng, *grid, (int)total) || fixed_claims(true, ng, *grid + 8, (int)total)))
            blp->front = 8;
#endif
        // Long tiles with fixed claims: the front workgroup stays until the workers have left (they count themselves
        // in ctx->done), whatever the number of rounds, and takes the place of the spare ones; the tile bodies look at
        // the stop index every few K-stages and give their tile up when a stop is recorded (tile_fixed_early).
        const int workers = *grid - blp->spare;
        if (long_ok && fixed_claims(true, ng, workers, (int)total) && fixed_claims(true, ng, workers + 8, (int)total)) {
            *grid = workers;
            blp->spare = 0; blp->front = 8;
            blp->done = ctx->done;
            // (the front workgroup leaves when half of the last round of workers has counted itself, which a worker does at
            // the top of the last K-step of its tile: the microsecond or two in which the front workgroup notices and
            // gets its last read of the flag back would otherwise come on top of every launch, 2.5 us on each of
            // ResNet-50's fp32 kernels)
            const int last_round = (int)(workers < resident ? workers : resident);
            blp->done_target = ctx->done_launches * workers + workers - last_round / 2;
        }
        set_poll_slices(blp, *grid);
        *grid += blp->front;
    } else {
        blp->flag = nullptr; blp->stop_index = nullptr; blp->executed = nullptr;
        blp->kernel_id = 0; blp->inject_at = -1; blp->poll_mask = 0; blp->groups = 1; blp->fresh = 0; blp->spare = 0; blp->stamps = nullptr; blp->front = 0; blp->done = nullptr; blp->done_target = 0;
        blp->started = nullptr; blp->started_seq = 0;
        for (int g = 0; g < 4; ++g) blp->poll_n[g] = 0;
        *grid = (int)total;
    }
    if (info) {
        info->total_tiles = (int)total; info->shape[0] = sx; info->shape[1] = sy; info->shape[2] = sz;
        info->grid = *grid; info->block = block;
        info->front = blp->front;
        info->fixed_claims = fixed_claims(ctx != nullptr, blp->groups, *grid - blp->front, (int)total);
    }
    return GP_SUCC;
}

}  // namespace gp
