// Pipelined tile kernel: operands stream global -> LDS directly (global_load_lds_dwordx4, no
// register staging) through a ring of STAGES buffers, so loads for K-step kt+STAGES-1 are in
// flight while the MFMAs consume K-step kt, with one workgroup barrier per K-step.
//
// LDS layout of one stage: A rows then B rows, each row BK elements = 128 bytes = 8 chunks of
// 16 bytes, K-contiguous, chunk c of row r stored at position c ^ ((r >> 1) & 7).  A direct
// load writes lane i's 16 bytes at (wave-uniform base) + 16*i, i.e. one instruction fills 8
// consecutive rows; the swizzle is applied on the global-address side (lane i fetches the chunk
// that belongs at its slot), which keeps the later 16-byte MFMA-operand reads spread over the
// banks.  Rows outside M/N, K-chunks past K and convolution taps outside the image are fetched
// from a zero page instead of being predicated.
//
// SPLITK = false: the 4 waves tile the BM x BN block 2 x 2.
// SPLITK = true : every wave computes the whole BM x BN block for one quarter of each K-step
//                 (wave w takes MFMA k-step w of the 4 in a stage); the four partial
//                 accumulators are then summed through LDS in the fixed order w0+w1+w2+w3.
//                 This quarters the length of the serial K loop for small, deep problems
//                 without making the result depend on scheduling.
#pragma once
#include "mma.hpp"
#include "../../include/util/conv_addr.h"

namespace gp {

// one copy per translation unit; only ever read
static __device__ __attribute__((aligned(64))) unsigned int g_zero_page[16] = {0};

// Direct global -> LDS load of 16 bytes per lane: lane i's data lands at lds_byte + 16*i.
// `lds_byte` must be wave-uniform (it travels in M0).  Written as inline assembly because the
// compiler serialises the equivalent builtin (it waits for every earlier LDS-DMA load before
// issuing the next one), which would defeat the multi-stage pipeline; the waits are placed by
// hand with wait_vmcnt() instead.
__device__ __forceinline__ void load_lds16(const void *gptr, unsigned lds_byte) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_byte)
                 : "memory", "m0");
}

// Reads a word that a load-to-LDS has written.  The pointer must carry the LDS address space: through a plain
// `volatile int *` the read is a flat load, which counts as a vector-memory operation as well, and the wait that the
// compiler puts behind it (vmcnt 0) also waits for every operand load the wavefront has in flight.
__device__ __forceinline__ int read_lds_word(const int *p) {
    return *(__attribute__((address_space(3))) volatile int *)(__attribute__((address_space(3))) void *)p;
}
// 4 bytes per lane: lane i's dword lands at lds_byte + 4*i.  Read past the caches (sc0 sc1): the
// word is one that another workgroup or the host changes while this kernel runs.
__device__ __forceinline__ void load_lds4(const void *gptr, unsigned lds_byte) {
    lds_byte = __builtin_amdgcn_readfirstlane(lds_byte);  // (the same for every lane; the compiler may hold it in a vector register)
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off sc0 sc1"
                 :
                 : "v"(gptr), "s"(lds_byte)
                 : "memory", "m0");
}

#ifndef GP_LOAD_SPREAD
#define GP_LOAD_SPREAD 0  // MFMAs between two loads of a stage; 0: chosen from the tile shape
#endif

// Optional phase timestamps of the first workgroups (compile with -DGP_TILE_PROF; read back with
// gp_debug_tile_prof).  Slot p of workgroup b is g_tile_prof[b * 8 + p], in shader-clock ticks.
#ifdef GP_TILE_PROF
static __device__ unsigned long long g_tile_prof[256 * 8];
#define GP_PROBE(p)                                                                  \
    do {                                                                             \
        if (threadIdx.x == 0 && blockIdx.x < 256) g_tile_prof[blockIdx.x * 8 + (p)] = __builtin_amdgcn_s_memtime(); \
    } while (0)
#else
#define GP_PROBE(p) do { } while (0)
#endif

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// four consecutive output elements
template <typename T> struct __attribute__((aligned(4 * sizeof(T)))) Vec4 { T v[4]; };
template <typename T> __device__ __forceinline__ void st_vec4(T *p, Vec4<T> o) {
    if constexpr (sizeof(T) == 4) st_out128(p, __builtin_bit_cast(out_u32x4, o));
    else st_out64(p, __builtin_bit_cast(unsigned long long, o));
}

// CKPT = true (bodies with the waves tiled 2 x 2): the tile can be left between two K-steps; see
// tile_loop_ckpt in tile_loop.hpp.  The stop index is read with the same direct-to-LDS loads as
// the operands, one extra load per stage: it lands in an LDS word in order with the stage it
// travels with, is covered by the same hand-placed vmcnt wait and barrier, and every wave then
// reads the same word, so the decision to leave is uniform and nothing ever waits for the poll.
// Eight workgroups take turns fetching the host flag the same way (each once in 8 polls: that
// read takes about as long as a K-step) and pass it on through the stop index.
struct CkptCtx {       // what a checkpointing body needs from the dispatcher, passed by value
    int *stop_index;   // nullptr: never leave a tile
    int *flag;
    void *ckpt;
    int kernel_id;
    unsigned long long *stamps = nullptr;  // BlpArgs::stamps (the measurement mode of tile_loop.hpp)
    int *announce = nullptr;               // run<true> with a stop word: the counter in which the workgroup counts itself at the
                                           // top of the last K-step of a tile that it finishes
};

// NWAVES: wavefronts per workgroup.  With eight (two per SIMD, 128 accumulator registers each) the
// second wavefront of a SIMD covers the first one's barrier, vmcnt and LDS waits, and each wavefront
// issues half of a stage's loads: measured 5-8 % faster than four on the 256 x 256 tile.
template <typename T, int BM, int BN, int STAGES, bool CONV, bool SPLITK, bool CKPT = false, int NWAVES = 4>
struct PipeKernel {
    using elem = T;
    static constexpr int bm = BM, bn = BN;
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int WAVES = NWAVES, NT = WAVES * 64;
    static constexpr int RB = 128;                        // row bytes in LDS
    static constexpr int BK = RB / (int)sizeof(T);        // 64 (16-bit) or 32 (fp32) elements
    static constexpr int KSTEPS = 4;                      // mma() calls per stage along K (2 chunks each)
    static constexpr int A_BYTES = BM * RB, B_BYTES = BN * RB, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int A_PW = BM / 8 / WAVES, B_PW = BN / 8 / WAVES;  // load instructions per wave per stage
    static constexpr int LPS = A_PW + B_PW;
    static constexpr int NLOADS = LPS + (CKPT ? 1 : 0);   // + the stop-word load of a checkpointing body
    static constexpr int WGM = SPLITK ? 1 : 2, WGN = SPLITK ? 1 : WAVES / 2;  // 2 x 2 or 2 x 4 wavefronts over the tile
    static constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / 32, NI = WN / 32;
    static constexpr size_t RED_BYTES = (size_t)WAVES * (SPLITK ? MI : 1) * NI * 16 * 64 * 4;  // epilogue staging
    static constexpr size_t RING_BYTES = (size_t)STAGES * STAGE_BYTES > RED_BYTES ? (size_t)STAGES * STAGE_BYTES : RED_BYTES;
    static constexpr size_t POLL_BYTES = CKPT ? (size_t)STAGES * WAVES * 256 : 0;  // a 256-byte landing slot per wave and stage
    static constexpr size_t LDS_BYTES = RING_BYTES + POLL_BYTES;
    static constexpr size_t CKPT_SLOT_BYTES = (size_t)WAVES * MI * NI * 16 * 64 * 4;  // one workgroup's accumulators
    static constexpr bool ckpt = CKPT;
    static constexpr bool early_stop = !CKPT;  // run() takes an early-stop word (see there)
    static constexpr bool can_look = !CKPT;    // run<true>() looks at it again every few K-steps
    // The stop words are fetched with every stage (so that every wave issues the same number of
    // loads) but looked at every POLL_EVERY-th K-step: about every 2.5 us for either tile size.
    static constexpr int POLL_EVERY = BM >= 256 ? 2 : 4;
    static_assert(!CKPT || !SPLITK, "checkpointing is built for the bodies without split K");
    static_assert(WAVES == 4 || (WAVES == 8 && !SPLITK), "4 wavefronts, or 8 without split K");
    static_assert(BM % 32 == 0 && BN % 32 == 0 && A_PW >= 1 && B_PW >= 1, "tile shape");
    static_assert(STAGES >= 2 && (STAGES - 2) * NLOADS < 64, "pipeline depth");

    // Returns true when the tile was left half-way (CKPT only); kt0 > 0 continues such a tile.
    //
    // Bodies without checkpoints take cc.stop_index as an "early stop" word (nullptr: none): it is
    // fetched once, with the first stage's operands, and looked at when that stage has landed,
    // about 2 us into the tile.  If a stop has been recorded by then the tile is not run and the
    // function returns true: the caller withdraws the claim.  This is for launches whose workgroups
    // all claim at once while a few spare workgroups read the host flag (tile_loop.hpp): the flag
    // read takes 1-2 us, so without the second look a kernel launched just after the flag went up
    // would still run to its end.
    template <bool LOOKS = false>
    static __device__ __forceinline__ bool run(const MatArgs &g, TileIdx t, T *lds_t, CkptCtx cc = CkptCtx{nullptr, nullptr, nullptr, 0},
                                               int tile_index = 0, int kt0 = 0) {
        GP_PROBE(0);
        __shared__ int early_slot[LOOKS ? 192 : 64];  // landing places of the stop word (lane 0's dword of each 64): the early look's, then two that the later looks take in turn
        // (made wave-uniform by force: handed over in a vector register, the word would make the compiler treat every branch
        // that depends on it as divergent, and the barriers and hand-placed waits below assume uniform control flow)
        const bool early = !CKPT && __builtin_amdgcn_readfirstlane((int)(cc.stop_index != nullptr)) != 0;
        // Long tiles look again every LOOK_EVERY K-steps (a K-step is 64 elements, a quarter to half a microsecond): the
        // word is fetched by wavefront 0 in front of a run of LOOK_EVERY K-steps and read by everybody behind the run
        // (the main loop below).  A tile that finds a stop recorded is given up (the caller withdraws the claim; the
        // relaunch computes it from the start).
        constexpr int LOOK_EVERY = 8;
        static_assert(LOOK_EVERY >= STAGES, "the waits of a run's K-steps cover the fetch in front of it");
        // (an instantiation of its own, LOOKS: as a run-time switch the looks cost the short tiles 3 % of a ResNet-152 pass)
        const bool looking = LOOKS && early;
        const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) void *)lds_t;
        const char *lds_c = (const char *)lds_t;
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: kept in a scalar register
        const int l32 = lane & 31, half = lane >> 5;
        const int m0 = t.y * BM, n0 = t.x * BN;
        long offa, offb, offc;
        if (g.batch_inner > 0) {
            int zo = t.z / g.batch_inner, zi = t.z - zo * g.batch_inner;
            offa = zo * g.stride_a_outer + zi * g.stride_a;
            offb = zo * g.stride_b_outer + zi * g.stride_b;
            offc = zo * g.stride_c_outer + zi * g.stride_c;
        } else {
            offa = t.z * g.stride_a; offb = t.z * g.stride_b; offc = t.z * g.stride_c;
        }
        const T *A = (const T *)g.A + offa, *B = (const T *)g.B + offb;
        const T *zero = (const T *)g_zero_page;
        const bool can_ckpt = CKPT && cc.stop_index != nullptr && cc.ckpt != nullptr;

        // ---- loader slots -------------------------------------------------------------------
        // Slot j of a wave covers rows (wave*PW + j)*8 .. +7 of the operand block; lane -> (row in
        // the group, chunk slot).  Only the wave's first row pointer is kept in registers: the
        // other slots are a uniform number of rows further on, and the swizzled chunk depends on
        // the slot's parity only ((row >> 1) & 7 = 4*(slot & 1) + (rig >> 1)).
        const int rig = lane >> 3, cpos = lane & 7;
        const int c_base = cpos ^ (rig >> 1);
        auto chunk_of = [&](int slot) { return c_base ^ ((slot & 1) << 2); };
        const int a_row0 = m0 + wave * A_PW * 8 + rig, b_row0 = n0 + wave * B_PW * 8 + rig;
        // Pointers with the lane's chunk already added, one per parity of the slot number j: a
        // load's address is then this plus a wave-uniform offset.
        const T *a_par[2] = {nullptr, nullptr};  // GEMM: row a_row0 of A
        const T *a_org[CONV ? A_PW : 1];         // CONV: the slot's window origin (may lie outside the image)
        int a_h0[CONV ? A_PW : 1], a_w0[CONV ? A_PW : 1];
        if (CONV) {
            const int hw = g.Ho * g.Wo;
            const bool small = g.M < kSmallDivLimit;
            const float rcp_hw = 1.0f / (float)hw, rcp_wo = 1.0f / (float)g.Wo;
#pragma unroll
            for (int j = 0; j < A_PW; ++j) {
                int m = a_row0 + j * 8;
                int mm = m < g.M ? m : 0;
                int n = small ? small_div(mm, hw, rcp_hw) : mm / hw, rem = mm - n * hw;
                int ho = small ? small_div(rem, g.Wo, rcp_wo) : rem / g.Wo, wo = rem - ho * g.Wo;
                a_h0[j] = ho * g.sh - g.ph; a_w0[j] = wo * g.sw - g.pw;
                a_org[j] = A + ((long)n * g.H * g.W + (long)a_h0[j] * g.W + a_w0[j]) * g.lda;
            }
        } else {
            a_par[0] = A + (long)a_row0 * g.lda + chunk_of(wave * A_PW) * VEC;
            a_par[1] = A + (long)a_row0 * g.lda + chunk_of(wave * A_PW + 1) * VEC;
        }
        const T *b_par[2] = {B + (long)b_row0 * g.ldb + chunk_of(wave * B_PW) * VEC,
                             B + (long)b_row0 * g.ldb + chunk_of(wave * B_PW + 1) * VEC};
        const bool conv_fast = CONV && (g.Cin % BK == 0);  // a K-step never straddles a filter tap
        const bool k_full = g.K % BK == 0;                 // no K-chunk of any stage lies past K
        // Running source pointers.  Within one filter tap (conv) or along K (weights, GEMM rows) a
        // slot's address only advances by BK elements per stage, so it is kept and bumped instead
        // of rebuilt: a wave has one instruction stream, and twenty address instructions per load
        // were more issue time than the MFMAs they feed.  `inc` is 0 for a slot parked on the zero
        // page.  (Only bodies with few slots keep them for the B / GEMM-A side: registers.)
        constexpr bool INCR = A_PW + B_PW <= 8;
        const T *a_cur[A_PW], *b_cur[B_PW];
        int a_inc[A_PW], b_inc[B_PW];
#pragma unroll
        for (int j = 0; j < A_PW; ++j) { a_cur[j] = zero; a_inc[j] = 0; }
#pragma unroll
        for (int j = 0; j < B_PW; ++j) { b_cur[j] = zero; b_inc[j] = 0; }

        // Loads of one stage: slot l < A_PW is an A slot, the rest are B slots.  `StageAddr` holds
        // the wave-uniform part, computed once per stage.
        struct StageAddr { unsigned sbase, sbase_poll; int k0, r_u, s_u, tap_off; bool new_tap, first; };
        // Stages are fetched in increasing order, so the filter tap (r, s) and channel offset of
        // the next stage advance incrementally instead of being divided out of k every time.
        int nx_r = 0, nx_s = 0, nx_ci = 0;
        if (CKPT && CONV && kt0 > 0 && conv_fast) {  // a tile that is continued starts at K-step kt0
            const int k = kt0 * BK, rs = k / g.Cin;
            nx_ci = k - rs * g.Cin;
            nx_r = rs / g.S;
            nx_s = rs - nx_r * g.S;
        }
        auto stage_addr = [&](int kt) {
            StageAddr sa;
            sa.sbase = lds0 + ((unsigned)kt % STAGES) * STAGE_BYTES;
            sa.sbase_poll = lds0 + (unsigned)RING_BYTES + ((unsigned)kt % STAGES) * WAVES * 256;
            sa.k0 = kt * BK;
            sa.r_u = nx_r; sa.s_u = nx_s;
            sa.tap_off = (nx_r * g.W + nx_s) * (int)g.lda + nx_ci;  // elements from the window origin
            sa.first = kt == kt0;                  // first stage fetched for this tile (or its continuation)
            sa.new_tap = sa.first || nx_ci == 0;   // the running conv pointers have to be rebuilt
            if (conv_fast) {
                nx_ci += BK;
                if (nx_ci >= g.Cin) {
                    nx_ci = 0;
                    if (++nx_s == g.S) { nx_s = 0; ++nx_r; }
                }
            }
            return sa;
        };
        auto issue_one = [&](const StageAddr &sa, int l) {  // l is a compile-time constant at every call
            if (CKPT && l == LPS) {
                // wave 0 fetches the stop index, wave 1 (when it is this workgroup's turn) the host
                // flag, the others a zero: every wave issues the same number of loads per stage
                const void *src = zero;
                if (can_ckpt) {
                    if (wave == 0) src = cc.stop_index;
                    // Whose turn it is goes by the clock, not by the K position: workgroups that continue tiles left
                    // at different depths are at different K positions, and turns taken by position then bunch up
                    // (a stop took up to 44 us to be recorded).  A turn is 5.12 us (two looks of this workgroup at
                    // least fall into it), eight turns a cycle.
                    else if (wave == 1 && blockIdx.x < 8 && cc.flag && ((sa.k0 / BK) & (POLL_EVERY - 1)) == 0 &&
                             (int)((wall_clock64() >> 9) & 7) == (int)blockIdx.x) src = cc.flag;
                }
                load_lds4(src, sa.sbase_poll + (unsigned)wave * 256);
            } else if (l < A_PW) {
                const int j = l;
                const int kc = chunk_of(wave * A_PW + j) * VEC;
                const T *src;
                if (CONV) {
                    const int jj = CONV ? j : 0;
                    if (conv_fast) {
                        if (sa.new_tap) {  // (uniform) rebuild: bounds of the tap, pointer or zero page
                            const bool ok = (a_row0 + j * 8 < g.M) & ((unsigned)(a_h0[jj] + sa.r_u) < (unsigned)g.H) &
                                            ((unsigned)(a_w0[jj] + sa.s_u) < (unsigned)g.W);
                            a_cur[j] = ok ? a_org[jj] + (sa.tap_off + kc) : zero;
                            a_inc[j] = ok ? BK : 0;
                        } else {
                            a_cur[j] += a_inc[j];
                        }
                        src = a_cur[j];
                    } else {
                        const int k = sa.k0 + kc, rs = k / g.Cin, ci = k - rs * g.Cin;
                        const int r = rs / g.S, s2 = rs - r * g.S;
                        const int off = (r * g.W + s2) * (int)g.lda + ci;
                        // selects, not branches: every lane computes an address and picks it or the zero page
                        const bool ok = (a_row0 + j * 8 < g.M) & (k < g.K) & ((unsigned)(a_h0[jj] + r) < (unsigned)g.H) &
                                        ((unsigned)(a_w0[jj] + s2) < (unsigned)g.W);
                        src = ok ? a_org[jj] + off : zero;
                    }
                } else if (INCR && k_full) {
                    if (sa.first) {
                        const bool ok = a_row0 + j * 8 < g.M;
                        a_cur[j] = ok ? a_par[j & 1] + ((long)(j * 8) * g.lda + sa.k0) : zero;
                        a_inc[j] = ok ? BK : 0;
                    } else {
                        a_cur[j] += a_inc[j];
                    }
                    src = a_cur[j];
                } else {
                    const bool ok = (a_row0 + j * 8 < g.M) & (k_full | (sa.k0 + kc < g.K));
                    src = ok ? a_par[j & 1] + ((long)(j * 8) * g.lda + sa.k0) : zero;
                }
                load_lds16(src, sa.sbase + (unsigned)((wave * A_PW + j) * 8 * RB));
            } else {
                const int j = l - A_PW;
                const int kc = chunk_of(wave * B_PW + j) * VEC;
                const T *src;
                if (INCR && k_full) {
                    if (sa.first) {
                        const bool ok = b_row0 + j * 8 < g.N;
                        b_cur[j] = ok ? b_par[j & 1] + ((long)(j * 8) * g.ldb + sa.k0) : zero;
                        b_inc[j] = ok ? BK : 0;
                    } else {
                        b_cur[j] += b_inc[j];
                    }
                    src = b_cur[j];
                } else {
                    const bool ok = (b_row0 + j * 8 < g.N) & (k_full | (sa.k0 + kc < g.K));
                    src = ok ? b_par[j & 1] + ((long)(j * 8) * g.ldb + sa.k0) : zero;
                }
                load_lds16(src, sa.sbase + (unsigned)(A_BYTES + (wave * B_PW + j) * 8 * RB));
            }
        };
        auto issue = [&](int kt) {
            const StageAddr sa = stage_addr(kt);
#pragma unroll
            for (int l = 0; l < NLOADS; ++l) issue_one(sa, l);
        };

        f32x16 acc[MI][NI];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        // checkpointing state
        f32x4 *slot = nullptr;       // this wave's part of the workgroup's checkpoint slot
        // landing slots of the stop-word loads, behind the ring: [stage][wave][64 dwords]
        typedef __attribute__((address_space(3))) volatile int lds_vint;
        lds_vint *pollw = (lds_vint *)(__attribute__((address_space(3))) void *)lds_t + RING_BYTES / 4;
        if (CKPT && can_ckpt) {
            slot = (f32x4 *)((char *)cc.ckpt + (size_t)CKPT_MAX_WGS * CKPT_HEADER_INTS * 4 + (size_t)blockIdx.x * CKPT_SLOT_BYTES) +
                   (size_t)wave * MI * NI * 4 * 64;
            if (kt0 > 0) {
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            f32x4 v = slot[((i * NI + j) * 4 + q) * 64 + lane];
                            // (reading the value here makes the compiler wait for the load now: left
                            // pending, it would put vmcnt waits in front of the MFMAs of every K-step)
                            asm volatile("" : "+v"(v));
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[i][j][q * 4 + e] = v[e];
                        }
            }
        }

        const int wm = SPLITK ? 0 : wave / WGN, wn = SPLITK ? 0 : wave % WGN;
        auto frag = [&](int stage, int region_bytes, int row, int chunk) -> u32x4 {
            int phys = chunk ^ ((row >> 1) & 7);
            return *(const u32x4 *)(lds_c + (size_t)stage * STAGE_BYTES + region_bytes + row * RB + phys * 16);
        };
        // Operand fragments are double-buffered in registers: while the MFMAs of k-step ks run, the
        // LDS reads of k-step ks+1 are in flight.  The last k-step of a stage is multiplied after
        // the next stage's barrier, so that the first fragment read of that stage is hidden too.
        u32x4 fa[2][MI], fb[2][NI];
        auto read_frags = [&](int buf, int stage, int ks) {
#pragma unroll
            for (int i = 0; i < MI; ++i) fa[buf][i] = frag(stage, 0, wm * WM + i * 32 + l32, ks * 2 + half);
#pragma unroll
            for (int j = 0; j < NI; ++j) fb[buf][j] = frag(stage, A_BYTES, wn * WN + j * 32 + l32, ks * 2 + half);
        };
        auto mma_all = [&](int buf) {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) Elem<T>::mma(fa[buf][i], fb[buf][j], acc[i][j]);
        };

        // One MFMA phase = the MI*NI products of one k-step; a k-tile has KSTEPS phases, i.e.
        // KSTEPS*MI*NI MFMA slots.  When `ISSUE`, the loads of the stage being fetched follow every
        // SPREAD-th MFMA, so that their address arithmetic issues while the matrix pipe is busy
        // instead of in front of it, and the requests reach the memory system as a steady stream.
        constexpr int NM = MI * NI;
        // (the spacing is that of the operand loads alone: the stop-word load of a checkpointing body goes with
        // the first of them, so that it has the whole stage to come back.  Counted with the others it halved
        // the spacing of the 128 x 128 body, 2 -> 1, which bunched its eight operand loads at the start of the
        // stage: 21 % of a VGG-16 layer)
        constexpr int EVEN = KSTEPS * NM / LPS > 0 ? KSTEPS * NM / LPS : 1;
        // measured: slightly front-loaded beats even for the 256x256 tile; with eight wavefronts (each issues
        // half the loads) every second slot is better still: the last load of a stage then leaves 40 % into
        // the stage instead of 70 %, and the stage's end waits less for it (8192^3: 3-7 % of the launch)
        constexpr int SPREAD = GP_LOAD_SPREAD > 0 ? GP_LOAD_SPREAD : (BM == 256 && WAVES == 8 && EVEN >= 4) ? 2 : (EVEN >= 4 ? EVEN - 1 : EVEN);
        static_assert(SPLITK || LPS <= KSTEPS * NM, "every operand load of a stage needs an MFMA slot");
        auto phase = [&](int buf, auto issue_c, const StageAddr &sa, auto p_c) {
            constexpr bool ISSUE = decltype(issue_c)::value != 0;
            constexpr int P = decltype(p_c)::value;
            static_for<0, NM>([&](auto qc) {
                constexpr int q = decltype(qc)::value, slot = P * NM + q;
                Elem<T>::mma(fa[buf][q / NI], fb[buf][q % NI], acc[q / NI][q % NI]);
                if constexpr (ISSUE && slot % SPREAD == 0 && slot / SPREAD < LPS) issue_one(sa, slot / SPREAD);
                if constexpr (ISSUE && slot == 0) static_for<LPS, NLOADS>([&](auto lc) { issue_one(sa, decltype(lc)::value); });
                // the slots cannot hold every load at this spacing: the rest follow the last MFMA
                if constexpr (ISSUE && slot == KSTEPS * NM - 1 && slot / SPREAD + 1 < LPS)
                    static_for<slot / SPREAD + 1, LPS>([&](auto lc) { issue_one(sa, decltype(lc)::value); });
                if constexpr (ISSUE) __builtin_amdgcn_sched_barrier(0);
            });
        };
        const int KT = (g.K + BK - 1) / BK;
        // A tile that is being finished counts its workgroup in cc.announce at the top of its last K-step, behind that step's
        // wait for its operands: nothing the wavefront issues later is waited for before the epilogue.  (Counted at the last
        // look instead, several K-steps from the end, the atomic stood in wavefront 0's queue in front of operand loads: the
        // counts that the waits of the next K-steps rely on go down in the order of issue, so the whole workgroup waited for
        // the atomic to be acknowledged, 6 us a tile with 512 workgroups resident.)
        auto announce = [&]() {
            if constexpr (LOOKS)
                if (cc.announce && tid == 0) __hip_atomic_fetch_add(cc.announce, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        // k-tile kt: wait for its stage, start fetching stage kt+STAGES-1 (ISSUE) and multiply.
        auto ktile = [&](int kt, bool tail, auto issue_c, auto plain_c) -> int {
            constexpr bool ISSUE = decltype(issue_c)::value != 0;
            constexpr bool PLAIN = decltype(plain_c)::value != 0;  // a K-step that cannot be the first of its tile and looks at nothing
            // stage kt has landed once at most the loads of the younger in-flight stages remain
            if (!tail) wait_vmcnt<(STAGES - 2) * NLOADS>();
            else wait_vmcnt<0>();
            int stop_word = -1, flag_word = 0;
            __syncthreads();  // everyone's part of stage kt is visible; stage kt-1's buffer is free
            if (kt == 0) GP_PROBE(2);
            if constexpr (LOOKS && !ISSUE)
                if (looking && kt == KT - 1 && kt > kt0) announce();
            const int stage = (int)((unsigned)kt % STAGES);
            StageAddr sa = {};
            if constexpr (ISSUE) sa = stage_addr(kt + STAGES - 1);
            if constexpr (SPLITK) {
                read_frags(0, stage, wave);  // the address arithmetic of the loads overlaps the LDS latency
                if constexpr (ISSUE) static_for<0, NLOADS>([&](auto lc) { issue_one(sa, decltype(lc)::value); });
                mma_all(0);
            } else {
                constexpr int LAST = (KSTEPS - 1) & 1;
                read_frags(0, stage, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (PLAIN || kt > kt0) {
                    phase(LAST, issue_c, sa, IntC<0>{});  // last k-step of stage kt-1 (in registers)
                } else if constexpr (ISSUE) {
                    static_for<0, NM>([&](auto qc) {  // first k-tile: phase 0 has loads but no MFMAs
                        constexpr int slot = decltype(qc)::value;
                        if constexpr (slot % SPREAD == 0 && slot / SPREAD < LPS) issue_one(sa, slot / SPREAD);
                        if constexpr (slot == 0) static_for<LPS, NLOADS>([&](auto lc) { issue_one(sa, decltype(lc)::value); });
                    });
                }
                static_for<0, KSTEPS - 1>([&](auto kc) {
                    constexpr int ks = decltype(kc)::value;
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (CKPT && ks == KSTEPS - 2) {
                        // the words that travelled with stage kt: the same two for every wave, looked at after the
                        // last phase, whose MFMAs cover the LDS latency (read at the top of the k-tile they cost
                        // 12 % of a VGG-16 layer: the wait for them came in front of the first fragment reads)
                        if (can_ckpt && (kt & (POLL_EVERY - 1)) == 0) {
                            stop_word = pollw[(((unsigned)kt % STAGES) * WAVES + 0) * 64];
                            flag_word = pollw[(((unsigned)kt % STAGES) * WAVES + 1) * 64];
                        }
                    }
                    read_frags((ks + 1) & 1, stage, ks + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    phase(ks & 1, issue_c, sa, IntC<ks + 1>{});
                });
                __builtin_amdgcn_sched_barrier(0);
            }
            int stop_now = 0;
            if constexpr (!CKPT && !PLAIN) {
                if (early && kt == kt0) stop_now = __builtin_amdgcn_readfirstlane(read_lds_word(early_slot)) != -1;
            }
            if constexpr (CKPT) {
                const int sw = __builtin_amdgcn_readfirstlane(stop_word), fw = __builtin_amdgcn_readfirstlane(flag_word);
                if (fw != 0 && tid == 0) record_stop(cc.stop_index, cc.kernel_id, cc.stamps);  // pass the host flag on
                stop_now = (sw != -1) | (fw != 0);
            }
            return stop_now;
        };

        // ---- output addressing; the lane's bias values are fetched before the main loop ---------
        T *C = (T *)g.C + offc;
        const T *R = g.residual ? (const T *)g.residual + offc : nullptr;
        const T *bias = (const T *)g.bias;
        const bool vec_ok = (g.N % 4 == 0) && (g.ldc % 4 == 0) && (offc % 4 == 0) && ((size_t)g.C % 16 == 0) &&
                            (!R || (g.ldr % 4 == 0 && (size_t)g.residual % 16 == 0)) && (!bias || (size_t)bias % 16 == 0);
        constexpr int EPI_L4 = SPLITK ? BN / 4 : 8 * NI;  // lanes per output row (4 columns each)
        const int epi_c4 = (SPLITK ? tid : lane) % EPI_L4;
        const int epi_n = n0 + wn * WN + (epi_c4 >> 3) * 32 + (epi_c4 & 7) * 4;
        // A lane's four columns are the same in every pass, so its bias values are read once; they
        // stay unconverted until the epilogue so that nothing waits for them before the main loop.
        Vec4<T> bias_raw;
#pragma unroll
        for (int q = 0; q < 4; ++q) bias_raw.v[q] = Elem<T>::from_f(0.f);
        if (bias && vec_ok && epi_n < g.N) bias_raw = *(const Vec4<T> *)(bias + epi_n);

        // ---- main loop ------------------------------------------------------------------------
        GP_PROBE(1);
        __syncthreads();  // the previous tile of this workgroup may still be reading LDS
#pragma unroll
        for (int s = 0; s < STAGES - 1; ++s) {
            if (kt0 + s < KT) issue(kt0 + s);
            // (older than every later stage's loads, so the wait for the first stage covers it; the
            // other waves issue nothing extra: each wave counts its own loads)
            if (!CKPT && s == 0 && early && wave == 0)
                load_lds4(cc.stop_index, (unsigned)(size_t)(__attribute__((address_space(3))) void *)early_slot);
        }
        int kt = kt0, stopped = 0;
        // Later looks: after the first K-step the tile goes on in runs of LOOK_EVERY K-steps, as many as fit in front
        // of the last STAGES-1 K-steps.  Wavefront 0 fetches the word in front of a run, everybody reads it behind
        // the run (the waits and barriers of the K-steps between have made it land and be seen), and the runs take two
        // landing places in turn, so that the fetch for the next run cannot overwrite a word that a slower wavefront
        // has still to read.  A run has no way out in the middle and tests nothing: its K-steps are the plain ones of the
        // steady state.
        const int runs = looking ? max(KT - (kt0 + 1) - (STAGES - 1), 0) / LOOK_EVERY : 0;
        for (; kt + STAGES - 1 < KT; ++kt) {
            stopped = ktile(kt, false, IntC<1>{}, IntC<0>{});
            if (stopped) break;  // (CKPT: leave the tile here; otherwise only the looks can say so)
            if constexpr (LOOKS) {
                if (looking && kt == kt0) {
                    for (int r = 0; r < runs; ++r) {
                        int *slot = early_slot + 64 + 64 * (r & 1);
                        if (wave == 0) load_lds4(cc.stop_index, (unsigned)(size_t)(__attribute__((address_space(3))) void *)slot);
#pragma nounroll
                        for (int i = 0; i < LOOK_EVERY; ++i) ktile(++kt, false, IntC<1>{}, IntC<1>{});
                        if (__builtin_amdgcn_readfirstlane(read_lds_word(slot)) != -1) { stopped = 1; break; }
                    }
                    if (stopped) break;
                }
            }
        }
        if (!stopped)
            for (; kt < KT; ++kt) {
                const int st = ktile(kt, KT - kt - 1 < STAGES - 2, IntC<0>{}, IntC<0>{});
                if (!CKPT && st) { stopped = 1; break; }  // (a checkpointing body finishes a tile whose last stages are in flight)
                if constexpr (LOOKS)
                    if (looking && kt == kt0 && kt == KT - 1) announce();  // (a tile of one K-step: its early look has just said go on)
            }
        if (!CKPT && stopped) {
            wait_vmcnt<0>();  // operand loads still landing in LDS must not outlive the workgroup
            return true;
        }
        if (!SPLITK && KT > kt0) mma_all((KSTEPS - 1) & 1);
        GP_PROBE(3);
        // When `stopped` (CKPT only), K-steps kt0..kt are in the accumulators and the "epilogue" below
        // writes them to the checkpoint slot instead of finishing the tile.  The loads of step kt+1
        // are still landing in LDS and must be waited for before the workgroup may go away.
        if (CKPT && stopped) wait_vmcnt<0>();

        // ---- epilogue -------------------------------------------------------------------------
        // Accumulators go through LDS once so that each lane finishes four consecutive columns of
        // one row: bias and residual are read, and the result written, as 8- or 16-byte vectors in
        // full rows instead of one element per lane.  Slice s = (block j, register v) of a wave's
        // accumulators is stored as 64 consecutive floats (one per lane), which is exactly
        // "row 8*(v/4) + 4*(lane/32) + v%4, columns 32*j + lane%32".
        // Finishes G rows (m_first, m_first + m_step, ...) of columns n..n+3: the residual reads of
        // the whole group are issued before the first result is needed.
        auto finish_group = [&](auto g_c, int n, const float (&bq)[4], int m_first, int m_step, const f32x4 *a) {
            constexpr int G = decltype(g_c)::value;
            if (n >= g.N) return;
            if (vec_ok) {
                Vec4<T> rv[G];
                if (R) {
#pragma unroll
                    for (int gi = 0; gi < G; ++gi) {
                        int m = m_first + gi * m_step;
                        if (m < g.M) rv[gi] = *(const Vec4<T> *)(R + (long)m * g.ldr + n);
                    }
                }
#pragma unroll
                for (int gi = 0; gi < G; ++gi) {
                    int m = m_first + gi * m_step;
                    if (m >= g.M) continue;
                    Vec4<T> o;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float x = a[gi][q] * g.alpha + bq[q];
                        if (R) x += Elem<T>::to_f(rv[gi].v[q]);
                        o.v[q] = Elem<T>::from_f(apply_act(x, g.act));
                    }
                    st_vec4<T>(&C[(long)m * g.ldc + n], o);
                }
            } else {
#pragma unroll
                for (int gi = 0; gi < G; ++gi) {
                    int m = m_first + gi * m_step;
                    if (m >= g.M) continue;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (n + q >= g.N) break;
                        float x = a[gi][q] * g.alpha + bq[q];
                        if (R) x += Elem<T>::to_f(R[(long)m * g.ldr + n + q]);
                        st_elem<T>(&C[(long)m * g.ldc + n + q], Elem<T>::from_f(apply_act(x, g.act)));
                    }
                }
            }
        };
        float *red = (float *)lds_t;
        // Every epilogue index is derived from these two laundered values: left to itself the compiler
        // computes the output addresses before the main loop and keeps them in registers across it.
        int lane_e = lane, tid_e = tid;
        asm volatile("" : "+v"(lane_e), "+v"(tid_e));
        // (the empty asm pins the conversion here: hoisted next to the load it would wait for it)
        {
            typedef unsigned int raw_t __attribute__((ext_vector_type(sizeof(Vec4<T>) / 4)));
            raw_t raw = __builtin_bit_cast(raw_t, bias_raw);
#pragma unroll
            for (int w = 0; w < (int)(sizeof(Vec4<T>) / 4); ++w) {
                unsigned int x = raw[w];
                asm volatile("" : "+v"(x));
                raw[w] = x;
            }
            bias_raw = __builtin_bit_cast(Vec4<T>, raw);
        }
        float bq[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) bq[q] = Elem<T>::to_f(bias_raw.v[q]);
        if (bias && !vec_ok) {  // unaligned or ragged output: element-wise
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (epi_n + q < g.N) bq[q] = Elem<T>::to_f(bias[epi_n + q]);
        }
        if (!SPLITK) {
            // each wave transposes its own 32-row strips through a private NI x 4 KB region
            float *mine = red + (size_t)wave * NI * 16 * 64;
            constexpr int L4 = 8 * NI;       // lanes per output row (4 columns each)
            constexpr int RPP = 64 / L4;     // rows per pass of the wave
            constexpr int PASSES = 32 / RPP;
            constexpr int G = PASSES < 4 ? PASSES : 4;
            const int c4 = lane_e % L4, r_in = lane_e / L4;
            const int j = c4 >> 3, col = (c4 & 7) * 4;
            const int n = n0 + wn * WN + j * 32 + col;
            __syncthreads();  // all waves are done reading the stage buffers
            static_for<0, MI>([&](auto ic) {
                constexpr int i = ic;
                if (CKPT && stopped) {  // (uniform) checkpoint: this strip's accumulators go to the slot as they are
#pragma unroll
                    for (int jj = 0; jj < NI; ++jj)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            f32x4 v = {acc[i][jj][q * 4], acc[i][jj][q * 4 + 1], acc[i][jj][q * 4 + 2], acc[i][jj][q * 4 + 3]};
                            slot[((i * NI + jj) * 4 + q) * 64 + lane_e] = v;
                        }
                    return;
                }
#pragma unroll
                for (int jj = 0; jj < NI; ++jj)
#pragma unroll
                    for (int v = 0; v < 16; ++v) mine[(jj * 16 + v) * 64 + lane_e] = acc[i][jj][v];
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // same wave reads other lanes' values next
#pragma unroll 1
                for (int p = 0; p < PASSES; p += G) {
                    f32x4 a[G];
#pragma unroll
                    for (int gi = 0; gi < G; ++gi) {
                        int r = (p + gi) * RPP + r_in;
                        int v = 4 * (r >> 3) + (r & 3), hf = (r >> 2) & 1;
                        a[gi] = *(const f32x4 *)(mine + (j * 16 + v) * 64 + hf * 32 + col);
                    }
                    finish_group(IntC<G>{}, n, bq, m0 + wm * WM + i * 32 + p * RPP + r_in, RPP, a);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // strip i+1 overwrites the region
            });
        } else {
            // partial sums -> LDS as [wave][slice][lane], slice = (i*NI + j)*16 + v; the BM x BN
            // block is then finished by all 256 threads, 4 columns each, summing the four partials
            // in the fixed order w0 + w1 + w2 + w3
            constexpr int SLICES = MI * NI * 16;
            constexpr int L4 = BN / 4;
            constexpr int RPP = NT / L4;     // rows per pass of the workgroup
            constexpr int PASSES = BM / RPP;
            constexpr int G = PASSES < 4 ? PASSES : 4;
            const int c4 = tid_e % L4, r_in = tid_e / L4;
            const int j = c4 >> 3, col = (c4 & 7) * 4;
            const int n = n0 + j * 32 + col;
            __syncthreads();  // all waves are done reading the stage buffers
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int jj = 0; jj < NI; ++jj)
#pragma unroll
                    for (int v = 0; v < 16; ++v) red[((size_t)wave * SLICES + (i * NI + jj) * 16 + v) * 64 + lane_e] = acc[i][jj][v];
            __syncthreads();
#pragma unroll 1
            for (int p = 0; p < PASSES; p += G) {
                f32x4 a[G];
#pragma unroll
                for (int gi = 0; gi < G; ++gi) {
                    int row = (p + gi) * RPP + r_in;
                    int i = row >> 5, r = row & 31;
                    int v = 4 * (r >> 3) + (r & 3), hf = (r >> 2) & 1;
                    size_t o = ((size_t)(i * NI + j) * 16 + v) * 64 + hf * 32 + col;
                    a[gi] = *(const f32x4 *)(red + o);
                    a[gi] += *(const f32x4 *)(red + (size_t)1 * SLICES * 64 + o);
                    a[gi] += *(const f32x4 *)(red + (size_t)2 * SLICES * 64 + o);
                    a[gi] += *(const f32x4 *)(red + (size_t)3 * SLICES * 64 + o);
                }
                finish_group(IntC<G>{}, n, bq, m0 + p * RPP + r_in, RPP, a);
            }
        }
#ifdef GP_TILE_PROF
        GP_PROBE(4);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        GP_PROBE(5);
#endif
        if constexpr (CKPT) {
            if (stopped) {
                if (tid == 0) {
                    int *hdr = (int *)cc.ckpt + (size_t)blockIdx.x * CKPT_HEADER_INTS;
                    hdr[1] = cc.kernel_id; hdr[2] = tile_index; hdr[3] = kt + 1; hdr[0] = 1;
                }
                return true;
            }
        }
        return false;
    }
};

}  // namespace gp
