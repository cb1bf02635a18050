// Block-level-preemption dispatcher for gfx950 kernels.
//
// Restates the persistent-block wrapper that the reference generates around every kernel
// (scripts/compile/convert_to_blp.py:40-69): a workgroup repeatedly (1) reads the preempt
// flag, (2) claims the next tile index from the kernel's atomic counter, (3) decodes the
// index into the original grid coordinates, (4) runs the kernel body on that tile.  When the
// flag is up it records the kernel id in *stop_index (first writer wins) and leaves; the
// counter then holds exactly the number of tiles already owed to completed claims, so a
// relaunch continues with the next unclaimed tile: no tile is redone or skipped.
//
// Differences from the generated wrapper, all deliberate:
//  * the flag lives in fine-grained pinned host memory and is read with a system-scope load
//    (the reference polls a GDRCopy-mapped device int, src/cuda-clients/blpclient.cpp:45-76);
//  * the claimed index is handed to the other waves through a two-slot LDS mailbox indexed by
//    iteration parity, which removes the reference's reuse race on its single __shared__ slot
//    with one barrier per tile;
//  * *stop_index is claimed with a compare-and-swap instead of a test followed by a store, and a
//    workgroup also leaves when *stop_index is already set (see "Sticky" below);
//  * with executed == nullptr the same kernel runs non-preemptibly, one workgroup per tile
//    (the reference builds a second, untransformed module for that: mod.cubin vs mod.tr.cubin);
//  * a launch that has a workgroup for every claim does not hand claims out through the counter
//    at all (see "fixed claims" below): the counter keeps counting, a bit per workgroup says
//    which claims were made.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/util/slice_map.h"

namespace gp {

// Optional timestamps of the dispatcher's steps in the first workgroups (compile with
// -DGP_TILE_PROF; gp_debug_tile_prof returns them after the bodies' own slots).
#ifdef GP_TILE_PROF
static __device__ unsigned long long g_disp_prof[256 * 8];
#define GP_DISP_PROBE(p)                                                             \
    do {                                                                             \
        if (threadIdx.x == 0 && blockIdx.x < 256) g_disp_prof[blockIdx.x * 8 + (p)] = __builtin_amdgcn_s_memtime(); \
    } while (0)
#else
#define GP_DISP_PROBE(p) do { } while (0)
#endif

struct BlpArgs {
    int *flag;        // nullptr: never preempted
    int *stop_index;
    int *executed;    // nullptr: static mapping, tile = blockIdx.x
    int total;        // total_block
    int sx, sy;       // shape.x, shape.y (shape.z = total / (sx*sy))
    int kernel_id;
    int inject_at;    // -1 = off
    int poll_mask;    // the claim numbered c reads the host flag when (c & poll_mask) == 0
    int groups;       // claim counters per kernel (>= 1); counter g sits at executed + g * COUNTER_STRIDE
    int order;        // tile order: 0 = x fastest (the reference's), 1 = y fastest, G >= 2 = bands of G tile rows (decode_tile)
    void *ckpt;       // checkpoint workspace of kernels that can leave a tile half-way, or nullptr
    int batch;        // tiles per claim (>= 1): a claim of index u stands for tiles [u*batch, (u+1)*batch)
    int tiles;        // number of tiles (total = ceil(tiles / batch) claims)
    int fresh;        // nonzero: the host vouches that no claim of this kernel has been made since its counters were cleared; 2: eager start (tile_fixed_early)
    int spare;        // fixed claims only: the last `spare` workgroups of the grid have no claim and read the flag
    int poll_n[4];    // several counters, claims through them: the number of claims in the slices of counters 0..3
    unsigned long long *stamps;  // nullptr (the default) or device time stamps of the preemption (see "time stamps" below)
    int front;        // the first `front` workgroups of the grid own no claim; the very first reads the flag until every
                      // claim of the launch has been made (front_workgroup); the workers are numbered from `front` on
    int *done;        // nullptr, or counters like `executed` (one per group, COUNTER_STRIDE apart) in which every worker of
                      // every launch of this kernel counts itself when it leaves.  Set for launches of long tiles: the
                      // front workgroup then reads the flag until the counters sum to done_target (most workers of
                      // THIS launch have left: plan_launch), and the bodies look at the stop index
                      // every few K-stages and give a tile up (the claim is withdrawn, the relaunch redoes it)
    int done_target;
    int *started;     // nullptr, or a word in host memory in which the first workgroup stores started_seq when it starts
    int started_seq;  // (gp_preempt_ctx::started_host: the host's flow control when it submits kernel by kernel)
};

// The first workgroup tells the host that this launch has reached the GPU, i.e. that everything submitted before it on
// the stream has left (a store to host memory: nobody waits for it).
__device__ __forceinline__ void announce_start(const BlpArgs &b, bool leader) {
    if (b.started && blockIdx.x == 0 && leader) __hip_atomic_store(b.started, b.started_seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// a worker's number among the workers of the launch, and how many there are
__device__ __forceinline__ int wg_id(const BlpArgs &b) { return (int)blockIdx.x - b.front; }
__device__ __forceinline__ int wg_count(const BlpArgs &b) { return (int)gridDim.x - b.front; }

// Device-scope atomics on ONE address complete at about one per 40 ns on MI355X: a kernel of a
// few hundred tiles claimed from a single counter spends 10-20 us on claims alone.  A caller may
// therefore give a kernel `groups` counters, one per 64-byte line; util/slice_map.h says which
// counter a workgroup claims from and which contiguous slice of the tile order that counter owns.
// groups == 1 is the reference's layout (one int per kernel).
constexpr int COUNTER_STRIDE = 16;  // ints

struct TileIdx { int x, y, z; };

__device__ __forceinline__ TileIdx decode_tile(int idx, int sx, int sy, int order = 0) {
    // x = idx % sx; y = (idx / sx) % sy; z = idx / (sx*sy)   (convert_to_blp.py:52-54);
    // order 1 swaps the roles of x and y, so that consecutive indices share a tile column
    // order G >= 2: bands of G tile rows, y fastest inside a band, so that consecutive indices
    // form G-row blocks: the workgroups an XCD runs side by side then share G row panels and a few
    // column panels instead of one row panel and every column panel (large GEMMs, whose panels
    // do not fit the XCD's L2)
    TileIdx t;
    if (order >= 2) {
        const int per = sx * sy;
        t.z = idx / per;
        const int i = idx - t.z * per;
        const int band = i / (order * sx), first_y = band * order;
        const int rows = sy - first_y < order ? sy - first_y : order;
        const int local = i - band * order * sx;
        t.x = local / rows;
        t.y = first_y + (local - t.x * rows);
    } else if (order == 0) {
        int q = idx / sx;
        t.x = idx - q * sx;
        t.z = q / sy;
        t.y = q - t.z * sy;
    } else {
        int q = idx / sy;
        t.y = idx - q * sy;
        t.z = q / sx;
        t.x = q - t.z * sx;
    }
    return t;
}

// ---- time stamps ----------------------------------------------------------------------------------
// A measurement mode (BlpArgs::stamps != nullptr), off by default.  The reference measures a preemption
// from the host (src/cuda-clients/blpclient.cpp:185-195: flag store, then a spin on the best-effort
// tenant's counter); what the host sees includes its own polling and the PCIe round trips.  With a stamp
// buffer the kernels write the device's constant-rate clock (wall_clock64) at the three moments that
// bound a preemption on the GPU:
//   word 0                 the workgroup whose compare-and-swap recorded the stop (flag seen on the device)
//   word 1                 the first claim made while the word was zero (the host clears it before a resume)
//   words 8 .. 8 + 1023    workgroup b, when it leaves, writes word 8 + (b mod 1024): the largest of them is
//                          the moment the last workgroup of the tenant's latest kernel left the GPU (a stop
//                          is often honoured without being recorded: the few kernels in flight simply end)
// Plain stores to distinct words: no atomic is added to the leaving path (an atomic on one word from every
// leaving workgroup serialises the exit of a large grid).
constexpr int STAMP_STOP = 0, STAMP_FIRST_CLAIM = 1, STAMP_EXIT0 = 8, STAMP_EXIT_SLOTS = 1024;
constexpr int STAMP_WORDS = STAMP_EXIT0 + STAMP_EXIT_SLOTS;

// records the stop (first writer wins) and, in the measurement mode, when
__device__ __forceinline__ void record_stop(int *stop_index, int kernel_id, unsigned long long *stamps) {
    if (atomicCAS(stop_index, -1, kernel_id) == -1 && stamps) stamps[STAMP_STOP] = wall_clock64();
}
__device__ __forceinline__ void stamp_first_claim(unsigned long long *stamps) {
    if (stamps && __hip_atomic_load(stamps + STAMP_FIRST_CLAIM, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
        atomicCAS(stamps + STAMP_FIRST_CLAIM, 0ull, (unsigned long long)wall_clock64());
}
// the leader of a leaving workgroup, once all its threads are done
__device__ __forceinline__ void stamp_exit_leader(unsigned long long *stamps) {
    stamps[STAMP_EXIT0 + ((int)blockIdx.x & (STAMP_EXIT_SLOTS - 1))] = wall_clock64();
}

// One claim by the workgroup's leader: -1 when the workgroup has to leave (stop requested or the
// slice is handed out).
//
// The stop index (device memory) doubles as the device-side mirror of the flag: every claim
// checks it, but only the workgroup about to make a claim whose number is a multiple of
// poll_every reads the flag itself from host memory.  Reads of fine-grained host memory are
// served one at a time (about 90 ns each on MI355X), so a poll per tile from every workgroup
// would dominate short kernels.
// The stop index is also sticky: once a kernel of this executor has been stopped, every later
// kernel of the same submission leaves too until the host re-arms it, even if the flag has been
// lowered in between; otherwise a kernel queued behind a stopped one could run to completion on
// incomplete inputs.
//
// Who reads the flag: with several counters, the first four groups do, for everybody.  Their slices
// end when everybody's do, give or take the skew between XCDs (all four are served by XCD 0), and a
// relaunch may find them handed out while other slices are not.  So a group beyond the four reads
// the flag at the same cadence once the counter of its counterpart among them (grp & 3) has passed
// the end of that group's slice (BlpArgs::poll_n, from the host: the slice arithmetic is too much
// code for every kernel to carry); until then it pays one more read of device memory on those claims.
__device__ __forceinline__ bool reads_flag(const BlpArgs &b, int grp) {
    if (grp < 4 || b.poll_mask == 0) return true;   // (poll_mask == 0: the flag is cheap device memory)
    const int g = grp & 3;
    return __hip_atomic_load(b.executed + g * COUNTER_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= b.poll_n[g];
}

__device__ __forceinline__ int claim_tile(const BlpArgs &b, int grp, int slice_lo, int slice_n) {
    int claim = -1;
    int stop = __hip_atomic_load(b.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != -1;
    if (!stop) {
        const int c = atomicAdd(b.executed + grp * COUNTER_STRIDE, 1);
        if (c < slice_n) {
            claim = slice_lo + c;
#ifndef GP_NO_INJECT  // (build switch for measuring what the test hook costs: nothing measurable)
            if (claim == b.inject_at && b.flag)
                __hip_atomic_store(b.flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#endif
            if (b.front == 0 && (c & b.poll_mask) == 0 && b.flag && reads_flag(b, grp) &&
                __hip_atomic_load(b.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0)
                record_stop(b.stop_index, b.kernel_id, b.stamps);
            // the polling workgroup still owes the tile it has just claimed
            stamp_first_claim(b.stamps);
        }
    }
    // (a workgroup that finds the stop index set has nothing to record: the first writer won.
    // An atomic on that one word from every leaving workgroup would serialise the exit of a
    // 2000-workgroup grid into 80 us.)
    return claim;
}

// ---- one claim per workgroup: fixed claims ------------------------------------------------------
// When a launch has at least as many workgroups as claims, nobody needs to be told which claim is
// next: workgroup b takes claim xcd_contiguous(b, total), the mapping of launches without
// counters.  What a relaunch has to know is which of these were made before, so words 1..15 of
// the 64-byte line of the workgroup's counter hold a bit per workgroup of that group, and word 0
// keeps counting claims for the host.  On a kernel's first launch after its counters were cleared
// (BlpArgs::fresh) every bit is known to be clear: the bit is set and the count raised without
// waiting for the old values.  No slice boundaries are needed either; computing them cost more
// than the claim itself (2 us of scalar arithmetic and instruction fetch in front of the first
// operand load of every launch).
static_assert(kFixedClaimBits == (COUNTER_STRIDE - 1) * 32, "a bit per workgroup in ints 1..15 of the counter's line");

template <bool LOOK = true>
__device__ __forceinline__ int claim_fixed(const BlpArgs &b, int grp) {
    if (wg_id(b) >= b.total) return -1;
    if (LOOK && __hip_atomic_load(b.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != -1) return -1;
    const int j = wg_id(b) >> log2_pow2(b.groups);  // this workgroup's rank among those of its group
    int *line = b.executed + grp * COUNTER_STRIDE;
    const int bit = 1 << (j & 31);
    if (b.fresh) {
        __hip_atomic_fetch_or(line + 1 + (j >> 5), bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if (__hip_atomic_fetch_or(line + 1 + (j >> 5), bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & bit) {
        return -1;  // made in an earlier launch
    }
    __hip_atomic_fetch_add(line, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int claim = xcd_contiguous(wg_id(b), b.total);
#ifndef GP_NO_INJECT
    if (claim == b.inject_at && b.flag)
        __hip_atomic_store(b.flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#endif
    // (with spare workgroups the flag is theirs to read: nobody's tile waits for host memory)
    // (... and so it is with a workgroup in front that does nothing else)
    if (b.spare == 0 && b.front == 0 && (grp < 4 || b.poll_mask == 0) && (j & b.poll_mask) == 0 && b.flag &&
        __hip_atomic_load(b.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0)
        record_stop(b.stop_index, b.kernel_id, b.stamps);
    stamp_first_claim(b.stamps);
    return claim;
}

// A spare workgroup of a launch with fixed claims: reads the flag once on behalf of the launch and
// leaves.  The read of host memory (1-2 us) then delays nobody's tile, where a poll after the
// first claims made four workgroups, and with them the kernel, finish that much later.
__device__ __forceinline__ bool spare_workgroup(const BlpArgs &b, bool fixed, bool leader) {
    if (!fixed || b.spare == 0 || (int)blockIdx.x < (int)gridDim.x - b.spare) return false;
    if (leader && b.flag && __hip_atomic_load(b.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0 &&
        __hip_atomic_load(b.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == -1)
        record_stop(b.stop_index, b.kernel_id, b.stamps);
    if (leader && b.stamps) stamp_exit_leader(b.stamps);
    return true;
}

// A launch of several rounds of workgroups with fixed claims (the hardware starts the later ones as earlier ones
// retire) looks at the flag only when a workgroup starts, and those start in bursts, a tile's length apart: with
// 40 us tiles (VGG-16's 512-channel 3 x 3 layers at batch 16) a stop took up to 43 us to be so much as recorded.
// Such a launch gets `front` workgroups ahead of its workers (a multiple of 8, so that the workers keep their XCDs).
// The first one stays: one lane reads the flag about every microsecond and records the stop, until a stop is
// recorded, or every claim of the launch has been made (from then on no workgroup starts that a stop could hold
// back), or its bounded number of looks is used up.  The others leave at once.  Returns true in a front workgroup.
__device__ __forceinline__ bool front_workgroup(const BlpArgs &b, bool leader) {
    announce_start(b, leader);  // (here because every dispatcher loop comes through here first)
    if (b.front == 0 || (int)blockIdx.x >= b.front) return false;
    const int tid = (int)(threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z));
    if (blockIdx.x != 0 || !b.flag) return true;
    // Two wavefronts look.  The first reads the flag: a trip to host memory, 1-2 us, and a wavefront cannot end before
    // its read has come back.  The second reads what lives in the device's memory, every lane one of the counters (at
    // most 64 of them) and the stop index, a few times per microsecond, so that the end of the launch is noticed soon:
    // the launch lasts until this workgroup has left, and with one wavefront that read the counters between two reads
    // of the flag, it left 2-3 us after the point it waits for, which a kernel of 10 us with 3 us tiles feels
    // (ResNet-152 b8: 3 % of a pass).  They tell each other through a word of LDS that it is time to go.
    __shared__ int front_leave;
    const int threads = (int)(blockDim.x * blockDim.y * blockDim.z);
    const bool two = threads >= 128;  // (a smaller workgroup: one wavefront does both, one after the other)
    if (tid == 0) front_leave = 0;
    __syncthreads();
    auto told = [&] { return __hip_atomic_load(&front_leave, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0; };
    auto tell = [&] { __hip_atomic_store(&front_leave, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); };
    // (with fixed claims word 0 of a line counts the claims made; handed out through the counters, a counter
    // runs past its slice by one per workgroup that found it empty: either way the sum reaches the total
    // no later than the last claim is made.  Long tiles: until most workers of this launch have left; they
    // count themselves in leave_stamped)
    const int *counters = b.done ? b.done : b.executed;
    const int target = b.done ? b.done_target : b.total;
    const int lanes = threads < 64 ? threads : 64;
    auto device_look = [&](int lane) {  // true: a stop is recorded, or the launch is about to end
        const int stop = __hip_atomic_load(b.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int n = 0;  // (ds_bpermute reads 0 from a lane that is off)
        for (int g = lane; g < b.groups; g += lanes) n += __hip_atomic_load(counters + g * COUNTER_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) n += __shfl_xor(n, d);
        return __builtin_amdgcn_readfirstlane(stop) != -1 || __builtin_amdgcn_readfirstlane(n) >= target;
    };
    if (tid < 64) {
        for (int look = 0; look < (1 << 17); ++look) {  // 1-2 us per look: at most about a quarter of a second
            int flag = 0;
            if (tid == 0) flag = __hip_atomic_load(b.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            if (__builtin_amdgcn_readfirstlane(flag) != 0) {
                if (tid == 0) record_stop(b.stop_index, b.kernel_id, b.stamps);
                break;
            }
            if (two ? told() : device_look(tid)) break;
            __builtin_amdgcn_s_sleep(4);
        }
        if (tid == 0) tell();
    } else if (two && tid < 128) {
        for (int look = 0; look < (1 << 19); ++look) {  // about half a microsecond per look
            if (device_look(tid - 64) || told()) break;
            __builtin_amdgcn_s_sleep(4);
        }
        if (tid == 64) tell();
    }
    return true;
}

// the counter of `done` in which this worker counts itself
__device__ __forceinline__ int *done_counter(const BlpArgs &b) { return b.done + wg_group(wg_id(b), b.groups) * COUNTER_STRIDE; }

// A worker of a preemptible launch leaves (every thread calls this).  Launches of long tiles count the leavers, for
// the front workgroup; the measurement mode stamps the moment.
__device__ __forceinline__ void leave_stamped(const BlpArgs &b, bool count = true) {
    if (!b.executed || (!b.stamps && !b.done)) return;
    if (wg_id(b) < 0 || (int)blockIdx.x >= (int)gridDim.x - b.spare) return;  // front and spare workgroups are no workers
    const bool leader = (threadIdx.x == 0) & (threadIdx.y == 0) & (threadIdx.z == 0);
    if (b.stamps) {
        __syncthreads();
        if (leader) stamp_exit_leader(b.stamps);
    }
    // (no value comes back: the atomic costs the leaver nothing; one line per group keeps them from queueing up on one address)
    // (count == false: the body has counted the workgroup already, at the top of the last K-step of its tile)
    if (b.done && count && leader) __hip_atomic_fetch_add(done_counter(b), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Runs body(TileIdx) for every tile this workgroup obtains.  All threads of the workgroup must
// call it; the body may use barriers freely.
template <class Body>
__device__ __forceinline__ void tile_loop(const BlpArgs &b, Body &&body) {
    __shared__ int mailbox[2];
    const bool dynamic = b.executed != nullptr;
    const bool leader = (threadIdx.x == 0) & (threadIdx.y == 0) & (threadIdx.z == 0);
    // As many workgroups as claims: a counter's slice is as long as the number of workgroups that
    // serve it (util/slice_map.h), so nobody can get a second claim, on a first launch or on a
    // relaunch, and the claim that would only report "nothing left" (an atomic and a barrier at
    // the tail of every small kernel) is skipped.
    GP_DISP_PROBE(0);
    if (front_workgroup(b, leader)) return;
    const bool single = wg_count(b) >= b.total;
    const bool fixed = fixed_claims(dynamic, b.groups, wg_count(b), b.total);
    // which counter this workgroup serves and the slice of the tile order that counter owns
    const int grp = wg_group(wg_id(b), b.groups);
    int slice_lo = 0, slice_n = b.total;
    if (b.groups > 1 && !fixed) {
        slice_lo = group_slice_begin(b.total, grp, b.groups, wg_count(b));
        slice_n = group_slice_begin(b.total, grp + 1, b.groups, wg_count(b)) - slice_lo;
    }
    if (spare_workgroup(b, fixed, leader)) return;
    // One loop and one call site for both modes, so that the body is inlined into the kernel and
    // the kernel arguments stay in scalar registers.
    for (int it = 0;; ++it) {
        int idx;
        if (!dynamic) {
            idx = (it == 0 && wg_id(b) < b.total) ? xcd_contiguous(wg_id(b), b.total) : -1;
        } else {
            if (it == 0) GP_DISP_PROBE(1);
            if (leader) mailbox[it & 1] = fixed ? claim_fixed(b, grp) : claim_tile(b, grp, slice_lo, slice_n);
            if (it == 0) GP_DISP_PROBE(2);
            __syncthreads();
            idx = __builtin_amdgcn_readfirstlane(mailbox[it & 1]);  // wave-uniform: tile coordinates stay scalar
        }
        if (it == 0) GP_DISP_PROBE(3);
        if (idx < 0) { leave_stamped(b); return; }
        // Streaming kernels have tiles of a few KB; handing them out several at a time keeps the
        // claim (an atomic and a barrier, 1-2 us) off their critical path.
        const int first = idx * b.batch, last = first + b.batch < b.tiles ? first + b.batch : b.tiles;
        for (int tile = first; tile < last; ++tile) body(decode_tile(tile, b.sx, b.sy, b.order));
        if (single) { leave_stamped(b); return; }
    }
}

// ---- the two common cases as loops of their own --------------------------------------------------
// tile_loop serves every kind of launch, and a kernel built on it carries all of that code in
// front of its body: slice arithmetic, both ways of claiming, the mailbox loop.  Measured on the
// convolution kernels, a launch WITHOUT counters takes 2 us longer through that kernel than
// through one that holds nothing but the body (12.4 against 10.3 us per launch, averaged over
// ResNet-152's layers): instruction fetch from a cold cache along a path full of taken branches.
// And any loop around the body, even one of a single trip, lets the compiler move the body's
// loop-invariant work (output addressing, bias loads) in front of it, i.e. in front of the first
// operand fetch: 1.5 us of the 2.
// So kernels are also instantiated around the two forms below, which call the body once, for
// launches of one tile per claim (BlpArgs::batch == 1), and the launcher picks: tile_plain for a
// launch without counters, tile_fixed for one whose claims are fixed (see above), tile_loop for
// the rest (more claims than workgroups, one counter per kernel, several tiles per claim).
template <class Body>
__device__ __forceinline__ void tile_plain(const BlpArgs &b, Body &&body) {
    if ((int)blockIdx.x >= b.total) return;
    body(decode_tile(xcd_contiguous((int)blockIdx.x, b.total), b.sx, b.sy, b.order));
}

// the claim of a workgroup of a launch with fixed claims, for all its threads; -1: leave
__device__ __forceinline__ int fixed_claim_of_workgroup(const BlpArgs &b) {
    __shared__ int mailbox;
    const bool leader = (threadIdx.x == 0) & (threadIdx.y == 0) & (threadIdx.z == 0);
    if (front_workgroup(b, leader)) return -1;
    if (spare_workgroup(b, true, leader)) return -1;
    if (leader) mailbox = claim_fixed(b, wg_group(wg_id(b), b.groups));
    __syncthreads();
    return __builtin_amdgcn_readfirstlane(mailbox);
}

// Fixed claims with a second look: body(TileIdx, stop word or nullptr) returns true when it found a
// stop recorded shortly after the claim and did not run the tile; the claim is then withdrawn
// (bit cleared, count lowered), so that the relaunch runs it.  The word is handed over only when
// the launch has spare workgroups reading the flag: that read is what the second look waits for.
__device__ __forceinline__ void unclaim_fixed(const BlpArgs &b) {
    const int grp = wg_group(wg_id(b), b.groups);
    const int j = wg_id(b) >> log2_pow2(b.groups);
    int *line = b.executed + grp * COUNTER_STRIDE;
    __hip_atomic_fetch_and(line + 1 + (j >> 5), ~(1 << (j & 31)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_fetch_add(line, -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
//
// Eager start (BlpArgs::fresh == 2).  On a kernel's first launch after its counters were cleared
// nothing has to come back from memory before the tile starts: the claim is known from the
// workgroup's number, its bit cannot be set yet, and the body's look at the stop word, which travels
// with the first operands, stands in for the look in front of the claim.  The bit and the count go
// out without waiting for their old values and are withdrawn like any claim if the body finds the
// stop recorded.  A launch saves the wait for the stop index that way (0.2 us of a 10 us
// convolution); a kernel queued behind a stop leaves a first operand fetch later than it would
// have, which adds 4 us to the drain of a chunk of launches.  That trade is the caller's.
// Everything the body is handed is computed from kernel arguments and the workgroup's number alone:
// a stop word that reaches the body in a vector register (a value merged from two branches does)
// makes the compiler treat the body's control flow as divergent, and the body, whose barriers and
// hand-placed waits assume uniform flow, then computes garbage for K of one step.
// ANNOUNCES: a body that was handed a stop word counts its workgroup in b.done itself at the top of the last K-step of a
// tile that it finishes, a microsecond or two before it leaves (so that the front workgroup is gone by the time the
// workers are: the launch lasts until the last workgroup has left, and the front one needs a microsecond or two to notice
// and to get its read of the flag back).
template <bool ANNOUNCES = false, class Body>
__device__ __forceinline__ void tile_fixed_early(const BlpArgs &b, Body &&body) {
    const bool eager = b.fresh > 1;
    int idx;
    if (eager) {
        const bool leader = threadIdx.x == 0;
        if (front_workgroup(b, leader)) return;
        if (spare_workgroup(b, true, leader)) return;
        if (wg_id(b) >= b.total) { leave_stamped(b); return; }
        if (leader) claim_fixed<false>(b, wg_group(wg_id(b), b.groups));
        idx = xcd_contiguous(wg_id(b), b.total);
    } else {
        idx = fixed_claim_of_workgroup(b);
    }
    if (idx < 0) { leave_stamped(b); return; }
    int *word = (eager || b.spare || b.front) ? b.stop_index : nullptr;
    const bool left = body(decode_tile(idx, b.sx, b.sy, b.order), word);
    if (left && threadIdx.x == 0) unclaim_fixed(b);
    leave_stamped(b, !(ANNOUNCES && word != nullptr && !left));
}

template <class Body>
__device__ __forceinline__ void tile_fixed(const BlpArgs &b, Body &&body) {
    const int idx = fixed_claim_of_workgroup(b);
    if (idx < 0) { leave_stamped(b); return; }
    body(decode_tile(idx, b.sx, b.sy, b.order));
    leave_stamped(b);
}

// body(first_tile, last_tile) forms, for kernels built on tile_loop_span
template <class Body>
__device__ __forceinline__ void span_plain(const BlpArgs &b, Body &&body) {
    if ((int)blockIdx.x >= b.total) return;
    const int first = xcd_contiguous((int)blockIdx.x, b.total);
    body(first, first + 1);
}

template <class Body>
__device__ __forceinline__ void span_fixed(const BlpArgs &b, Body &&body) {
    const int idx = fixed_claim_of_workgroup(b);
    if (idx < 0) { leave_stamped(b); return; }
    body(idx, idx + 1);
    leave_stamped(b);
}

// which of the loops a kernel instantiation is built around
enum { LOOP_ANY = 0, LOOP_PLAIN = 1, LOOP_FIXED = 2 };
template <int LOOP, class Body>
__device__ __forceinline__ void tiles(const BlpArgs &b, Body &&body) {
    if constexpr (LOOP == LOOP_PLAIN) tile_plain(b, body);
    else if constexpr (LOOP == LOOP_FIXED) tile_fixed(b, body);
    else tile_loop(b, body);
}
template <int LOOP, class Body>
__device__ __forceinline__ void spans(const BlpArgs &b, Body &&body);

// The same dispatcher for one-dimensional streaming kernels that want a claim's tiles all at once
// (to keep the loads of several tiles in flight together): body(first_tile, last_tile) is called
// once per claim with the half-open range of tile numbers the claim stands for.
template <class Body>
__device__ __forceinline__ void tile_loop_span(const BlpArgs &b, Body &&body) {
    __shared__ int mailbox[2];
    const bool dynamic = b.executed != nullptr;
    const bool leader = (threadIdx.x == 0) & (threadIdx.y == 0) & (threadIdx.z == 0);
    if (front_workgroup(b, leader)) return;
    const int grp = wg_group(wg_id(b), b.groups);
    const bool fixed = fixed_claims(dynamic, b.groups, wg_count(b), b.total);
    int slice_lo = 0, slice_n = b.total;
    if (b.groups > 1 && !fixed) {
        slice_lo = group_slice_begin(b.total, grp, b.groups, wg_count(b));
        slice_n = group_slice_begin(b.total, grp + 1, b.groups, wg_count(b)) - slice_lo;
    }
    if (spare_workgroup(b, fixed, leader)) return;
    for (int it = 0;; ++it) {
        int idx;
        if (!dynamic) {
            idx = (it == 0 && wg_id(b) < b.total) ? xcd_contiguous(wg_id(b), b.total) : -1;
        } else {
            if (leader) mailbox[it & 1] = fixed ? claim_fixed(b, grp) : claim_tile(b, grp, slice_lo, slice_n);
            __syncthreads();
            idx = __builtin_amdgcn_readfirstlane(mailbox[it & 1]);
        }
        if (idx < 0) { leave_stamped(b); return; }
        const int first = idx * b.batch;
        body(first, first + b.batch < b.tiles ? first + b.batch : b.tiles);
        if (wg_count(b) >= b.total) { leave_stamped(b); return; }  // one claim per workgroup at most (see tile_loop)
    }
}

template <int LOOP, class Body>
__device__ __forceinline__ void spans(const BlpArgs &b, Body &&body) {
    if constexpr (LOOP == LOOP_PLAIN) span_plain(b, body);
    else if constexpr (LOOP == LOOP_FIXED) span_fixed(b, body);
    else tile_loop_span(b, body);
}

// ---- tiles that can be left half-way ------------------------------------------------------------
// A tile whose K loop runs for hundreds of microseconds (a 256 x 256 tile over K = 8192 takes
// about 200 us) makes "finish the tile you owe" too slow a way to leave.  Kernels built on
// tile_loop_ckpt poll for the stop request inside the tile, and a workgroup that is asked to
// leave writes its fp32 accumulators and its position in K to its own slot of a checkpoint
// workspace; the relaunch (same grid) finds the slot, reloads the accumulators and continues
// with the next K-step.  The accumulation order is unchanged, so the result stays bit-identical.
//
// Workspace layout (BlpArgs::ckpt): CKPT_MAX_WGS headers of 64 bytes, then one slot of
// `ckpt_slot_bytes` per workgroup.  Header words: [0] valid, [1] kernel id, [2] tile index,
// [3] K-step to continue with.
constexpr int CKPT_MAX_WGS = 1024;
constexpr int CKPT_HEADER_INTS = 16;

// body(TileIdx, tile index, first K-step (0 = fresh tile)) returns true when it has left the tile
// half-way (and written its checkpoint); the workgroup then leaves the kernel.
template <class Body>
__device__ __forceinline__ void tile_loop_ckpt(const BlpArgs &b, Body &&body) {
    __shared__ int mailbox[2][2];
    const bool dynamic = b.executed != nullptr;
    const bool leader = (threadIdx.x == 0) & (threadIdx.y == 0) & (threadIdx.z == 0);
    const int grp = wg_group((int)blockIdx.x, b.groups);
    const int slice_lo = b.groups > 1 ? group_slice_begin(b.total, grp, b.groups, (int)gridDim.x) : 0;
    const int slice_n = (b.groups > 1 ? group_slice_begin(b.total, grp + 1, b.groups, (int)gridDim.x) : b.total) - slice_lo;
    announce_start(b, leader);
    for (int it = 0;; ++it) {
        int idx, kt0 = 0;
        if (!dynamic) {
            idx = (it == 0 && (int)blockIdx.x < b.total) ? xcd_contiguous((int)blockIdx.x, b.total) : -1;
        } else {
            if (leader) {
                int claim = -1, first = 0;
                int *hdr = b.ckpt ? (int *)b.ckpt + (size_t)blockIdx.x * CKPT_HEADER_INTS : nullptr;
                if (it == 0 && hdr && hdr[0] == 1 && hdr[1] == b.kernel_id) {
                    // a tile this workgroup left half-way in an earlier launch comes first; it was
                    // counted when it was claimed
                    // (the flag as well, by everybody: a launch that resumes stopped tiles may find the next request
                    // already there, and reloading 256 KB of accumulators only to store them again is 30 us of a
                    // preemption; the read costs a resumption one trip to host memory)
                    bool stopped = __hip_atomic_load(b.stop_index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != -1;
                    if (!stopped && b.flag && __hip_atomic_load(b.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0) {
                        record_stop(b.stop_index, b.kernel_id, b.stamps);
                        stopped = true;
                    }
                    if (!stopped) {
                        claim = hdr[2];
                        first = hdr[3];
                        hdr[0] = 0;
                    }
                } else {
                    claim = claim_tile(b, grp, slice_lo, slice_n);
                }
                mailbox[it & 1][0] = claim;
                mailbox[it & 1][1] = first;
            }
            __syncthreads();
            idx = __builtin_amdgcn_readfirstlane(mailbox[it & 1][0]);  // wave-uniform: tile coordinates and
            kt0 = __builtin_amdgcn_readfirstlane(mailbox[it & 1][1]);  // K position stay scalar
        }
        if (idx < 0) { leave_stamped(b); return; }
        if (body(decode_tile(idx, b.sx, b.sy, b.order), idx, kt0)) { leave_stamped(b); return; }
        // one claim per workgroup at most (see tile_loop); a relaunch may continue a stored tile and
        // then still owe its slice a claim, so the shortcut holds on the fresh path only
        if ((int)gridDim.x >= b.total && kt0 == 0 && !(it == 0 && b.ckpt)) { leave_stamped(b); return; }
    }
}

}  // namespace gp
