// Wide split-K GEMM tile kernel for small, deep problems (few output tiles, long K): 8 or 16 wavefronts
// share ONE output tile and split every K-stage between them.
//
// Why: on MI355X one wavefront's operand fetches (direct global -> LDS loads as well as register
// loads of 16 bytes per lane) complete at about 30-35 GB/s from an L2-resident source, however many
// loads it keeps in flight (about 60 cycles per 1 KB instruction), and the rate of a compute unit
// grows with the number of wavefronts that issue loads (about 120-140 GB/s with 4 wavefronts,
// 260-440 with 16).  A layer with fewer tiles than the GPU has compute units therefore streams its
// operands two to three times faster when sixteen wavefronts fetch for a tile than when four do,
// and for these layers the operand stream is what the main loop waits for (a 32 x 32 tile of a
// K = 3072 layer does 6 MFLOP on 384 KB of operands: 3 us at 130 GB/s).
//
// Structure: a stage holds KB = WAVES / 4 consecutive K-blocks of BK elements (one 128-byte row
// chunk per tile row, the layout and swizzle of gemm_pipe.hpp); wavefront w belongs to block group
// kb = w / 4 and fetches a quarter of the rows of that group's block.  One barrier per stage.  The
// arithmetic stays with wavefronts 0..3 (there is little of it: these layers wait for operands):
// wavefront w multiplies MFMA k-step w of every block, block after block, for the whole BM x BN
// tile (the code lets G groups of four share the output blocks between them; G = 1, see there), and at the end
// the four partial tiles are summed through LDS in the order 0, 1, 2, 3.  That
// is exactly the summation of the four-wavefront split-K bodies of gemm_pipe.hpp, so the result
// has the same bits as theirs (the whole-model program, whose workgroups have four wavefronts,
// uses those) and does not depend on scheduling: a preempted-then-resumed run stays bit-identical.
//
// Measured (fp16, launch to launch): 128 x 768 x 3072 (BERT's second FFN layer) 10.2 -> 8.2 us,
// 384 x 768 x 3072 11.9 -> 10.4 us; level with the four-wavefront bodies at K <= 1024, where the
// longer wait for the first, larger stage costs what the faster stream saves.
//
// CONV = true: the A operand is gathered (implicit GEMM over NHWC pixels): row m is output pixel
// (n, ho, wo), K element k is filter tap k / Cin, channel k % Cin.  Needs Cin to be a multiple of
// BK (a block never straddles two taps) and at most 32 taps: which taps of a pixel's window lie
// inside the image is worked out once per tile, as one bit per tap, so that a stage's loads cost a
// shift, a select and an add per lane; the tap and channel of a wavefront group's next block
// advance incrementally.
#pragma once
#include "gemm_pipe.hpp"

namespace gp {

// 1: ask for all STAGES buffers of the ring before the main loop instead of STAGES - 1 (every buffer is free
// at the start of a tile).  Measured, launch to launch: 128 x 768 x 3072 8.04 -> 7.80 us, but 128 x 2304 x 768
// 5.74 -> 5.85 and 128 x 768 x 768 4.84 -> 4.90: off.
#ifndef GP_WIDE_PREFILL
#define GP_WIDE_PREFILL 0
#endif
// waits until at most `stages` stages of LPW loads each are still in flight (stages = 0..3)
template <int LPW> __device__ __forceinline__ void wait_stages(int stages) {
    if (stages >= 3) wait_vmcnt<3 * LPW>();
    else if (stages == 2) wait_vmcnt<2 * LPW>();
    else if (stages == 1) wait_vmcnt<LPW>();
    else wait_vmcnt<0>();
}

// The end of a tile of the wide bodies: the partial tiles of wavefronts 0..3 are summed through LDS in
// wavefront order and the epilogue (alpha, bias, residual, activation) is applied on the way out.
template <typename T, int BM, int BN, int NT, int G>
__device__ __forceinline__ void wide_reduce_store(const MatArgs &g, float *red, const f32x16 (&acc)[(BM / 32) * (BN / 32) / G], int m0, int n0, long offc,
                                                  int tid, int wv, int lane, int kb) {
    constexpr int MI = BM / 32, NI = BN / 32, SLICES = MI * NI * 16, BPW = MI * NI / G;
    // ---- reduction and epilogue -------------------------------------------------------------
    // partial tiles of wavefronts 0..3 -> LDS as [wavefront][slice][lane], slice = (i*NI + j)*16 + v,
    // which is row 8*(v/4) + 4*(lane/32) + v%4, column 32*j + lane%32 of 32 x 32 block (i, j).
    // The first BM*BN/4 threads then finish four consecutive columns of one row each, adding the
    // partials in wavefront order.
    T *C = (T *)g.C + offc;
    const T *R = g.residual ? (const T *)g.residual + offc : nullptr;
    const T *bias = (const T *)g.bias;
    const bool vec_ok = (g.N % 4 == 0) && (g.ldc % 4 == 0) && (offc % 4 == 0) && ((size_t)g.C % 16 == 0) &&
                        (!R || (g.ldr % 4 == 0 && (size_t)g.residual % 16 == 0)) && (!bias || (size_t)bias % 16 == 0);
    __syncthreads();  // all wavefronts are done reading the stage buffers
    if (kb < G) {  // wavefront (kb, wv) holds k-step wv of the 32 x 32 blocks kb, kb + G, ...
#pragma unroll
        for (int q = 0; q < BPW; ++q)
#pragma unroll
            for (int v = 0; v < 16; ++v) red[((size_t)wv * SLICES + (kb + q * G) * 16 + v) * 64 + lane] = acc[q][v];
    }
    __syncthreads();
    GP_PROBE(4);
    constexpr int L4 = BN / 4;                        // threads per output row
    constexpr int FIN = BM * L4 < NT ? BM * L4 : NT;  // threads that finish
    constexpr int RPP = FIN / L4, PASSES = BM / RPP;
    if (tid < FIN) {
        const int c4 = tid % L4, r_in = tid / L4;
        const int j = c4 >> 3, col = (c4 & 7) * 4;
        const int n = n0 + j * 32 + col;
        float bq[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias && n < g.N) {
            if (vec_ok) {
                const Vec4<T> b = *(const Vec4<T> *)(bias + n);
#pragma unroll
                for (int q = 0; q < 4; ++q) bq[q] = Elem<T>::to_f(b.v[q]);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (n + q < g.N) bq[q] = Elem<T>::to_f(bias[n + q]);
            }
        }
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int row = p * RPP + r_in, m = m0 + row;
            const int i = row >> 5, r = row & 31;
            const int v = 4 * (r >> 3) + (r & 3), hf = (r >> 2) & 1;
            const size_t o = ((size_t)(i * NI + j) * 16 + v) * 64 + hf * 32 + col;
            f32x4 a = *(const f32x4 *)(red + o);
#pragma unroll
            for (int w = 1; w < 4; ++w) a += *(const f32x4 *)(red + (size_t)w * SLICES * 64 + o);
            if (m >= g.M || n >= g.N) continue;
            if (vec_ok) {
                Vec4<T> rv;
                if (R) rv = *(const Vec4<T> *)(R + (long)m * g.ldr + n);
                Vec4<T> out;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float x = a[q] * g.alpha + bq[q];
                    if (R) x += Elem<T>::to_f(rv.v[q]);
                    out.v[q] = Elem<T>::from_f(apply_act(x, g.act));
                }
                st_vec4<T>(&C[(long)m * g.ldc + n], out);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (n + q >= g.N) break;
                    float x = a[q] * g.alpha + bq[q];
                    if (R) x += Elem<T>::to_f(R[(long)m * g.ldr + n + q]);
                    st_elem<T>(&C[(long)m * g.ldc + n + q], Elem<T>::from_f(apply_act(x, g.act)));
                }
            }
        }
    }
}

template <typename T, int BM, int BN, int WAVES, int STAGES, bool CONV = false>
struct WideKernel {
    using elem = T;
    static constexpr int bm = BM, bn = BN;
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int NT = WAVES * 64;
    static constexpr int RB = 128;                         // row bytes of a block in LDS
    static constexpr int BK = RB / (int)sizeof(T);         // K elements per block: 64 (16-bit) or 32 (fp32)
    static constexpr int KB = WAVES / 4;                   // blocks per stage
    static constexpr int GROUPS = (BM + BN) / 8;           // 8-row load groups per block (A rows, then B rows)
    static constexpr int LPW_A = BM / 8 / 4, LPW_B = BN / 8 / 4;  // of a wavefront's loads per stage, the first LPW_A fetch A rows
    static constexpr int LPW = LPW_A + LPW_B;              // load instructions per wavefront per stage
    static constexpr int A_BYTES = BM * RB, BLK_BYTES = (BM + BN) * RB, STAGE_BYTES = KB * BLK_BYTES;
    static constexpr int MI = BM / 32, NI = BN / 32;
    // Which wavefronts multiply: group kb < G takes the 32 x 32 output blocks kb, kb + G, ... (k-step wv of every
    // K-block: whose registers a partial sum lives in does not change what is added to what).  G = 1 here:
    // two multiplying groups (one per output block of a 64 x 32 tile) were measured and changed nothing or
    // cost a little (1568 x 256 x 2304: 8.50 -> 8.54 us, 128 x 2304 x 768: 5.16 -> 5.43; each group re-reads
    // the fragments it shares with the other); the layer-norm prologue body, whose A operand stays in LDS,
    // gains from two (gemm_ln.hpp).
    static constexpr int G = 1;
    static constexpr int BPW = MI * NI / G;
    static_assert(MI * NI % G == 0, "output blocks divide among the multiplying groups");
    static constexpr int SLICES = MI * NI * 16;            // 64-float slices of one k-step's partial tile
    static constexpr size_t RED_BYTES = (size_t)4 * SLICES * 64 * 4;   // the partial tiles of wavefronts 0..3
    static constexpr size_t RING_BYTES = (size_t)STAGES * STAGE_BYTES;
    static constexpr size_t LDS_BYTES = RING_BYTES > RED_BYTES ? RING_BYTES : RED_BYTES;
    static constexpr size_t CKPT_SLOT_BYTES = 0;
    static constexpr bool ckpt = false;
    static constexpr bool early_stop = true;  // as PipeKernel::run: a second look at the stop index when the first stage has landed
    static constexpr bool can_look = true;
    static constexpr int PRE = GP_WIDE_PREFILL ? STAGES : STAGES - 1;  // stages asked for before the main loop
    static_assert(WAVES % 4 == 0 && WAVES >= 4 && WAVES <= 16, "4, 8, 12 or 16 wavefronts");
    static_assert(BM % 32 == 0 && BN % 32 == 0 && GROUPS % 4 == 0, "tile shape");
    // slot j of wavefront wv (of its block group): row group wv*LPW_A + j of A, or wv*LPW_B + (j - LPW_A) of B
    static __device__ __forceinline__ constexpr int group_of(int wv, int j) { return j < LPW_A ? wv * LPW_A + j : BM / 8 + wv * LPW_B + (j - LPW_A); }
    static_assert(STAGES >= 2 && STAGES <= 4 && (STAGES - 1) * LPW < 64, "pipeline depth");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");

    // Returns true when the early look found a stop recorded: the tile was not run.
    template <bool LOOKS = false>
    static __device__ __forceinline__ bool run(const MatArgs &g, TileIdx t, T *lds_t, CkptCtx cc = CkptCtx{nullptr, nullptr, nullptr, 0}) {
        GP_PROBE(0);
        __shared__ int early_slot[64];
        const bool early = __builtin_amdgcn_readfirstlane((int)(cc.stop_index != nullptr)) != 0;
        // Long tiles look again every LOOK_EVERY stages (a stage is KB blocks of 64 K-elements: about a microsecond of a
        // 32 x 32 x 25088 tile): the word is fetched by wavefront 0 in front of the loads of the stage it travels
        // with, so that the wait for that stage covers it, and read by everybody behind that stage's barrier.  One
        // landing slot is enough: the next fetch is issued LOOK_EVERY - (STAGES - 1) stages after this one was read.
        constexpr int LOOK_EVERY = 4;
        static_assert(LOOK_EVERY >= STAGES, "a look is read before the next one is fetched");
        const bool looking = LOOKS && early;  // (an instantiation of its own, as in PipeKernel)
        const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) void *)lds_t;
        const char *lds_c = (const char *)lds_t;
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int kb = wave >> 2, wv = wave & 3;
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

        // ---- loader slots: every wavefront fetches LPW_A row groups of A and LPW_B of B of its block (which
        // kind a slot is is known at compile time: no branches in the stage's load sequence) ------
        // lane -> (row in the group, chunk position); the swizzle is applied on the source side:
        // the lane at position cpos of row r fetches chunk cpos ^ ((r >> 1) & 7) of that row
        const int rig = lane >> 3, cpos = lane & 7;
        const int hw = CONV ? g.Ho * g.Wo : 1, ntap_rows = CONV ? g.K / (g.Cin * g.S) : 0;
        const bool small = g.M < kSmallDivLimit;
        const float rcp_hw = 1.0f / (float)hw, rcp_wo = CONV ? 1.0f / (float)g.Wo : 1.0f;
        const T *base[LPW];    // the lane's row and chunk at k = 0 (CONV, A rows: its window's origin, which may lie outside the image)
        bool row_ok[LPW];
        int kc[LPW];           // the lane's chunk offset in elements
        unsigned taps[CONV ? LPW : 1];  // CONV, A rows: bit t set = tap t of the row's window is inside the image
#pragma unroll
        for (int j = 0; j < LPW; ++j) {
            const int gi = group_of(wv, j);           // group index in the block
            const bool is_a = j < LPW_A;
            const int r = (is_a ? gi : gi - BM / 8) * 8 + rig;   // row in its region
            kc[j] = (cpos ^ ((r >> 1) & 7)) * VEC;
            if (is_a && CONV) {
                const int m = m0 + r;
                row_ok[j] = m < g.M;
                const int mm = row_ok[j] ? m : 0;
                const int n = small ? small_div(mm, hw, rcp_hw) : mm / hw, rem = mm - n * hw;
                const int ho = small ? small_div(rem, g.Wo, rcp_wo) : rem / g.Wo, wo = rem - ho * g.Wo;
                const int h0 = ho * g.sh - g.ph, w0 = wo * g.sw - g.pw;
                base[j] = A + (long)((n * g.H + h0) * g.W + w0) * g.lda + kc[j];  // (pixel indices fit an int: checked by the planner)
                const unsigned mask = row_ok[j] ? window_tap_mask(h0, w0, g.H, g.W, ntap_rows, g.S) : 0u;
                taps[CONV ? j : 0] = mask;
            } else if (is_a) {
                const int m = m0 + r;
                row_ok[j] = m < g.M;
                base[j] = A + (long)m * g.lda + kc[j];
            } else {
                const int n = n0 + r;
                row_ok[j] = n < g.N;
                base[j] = B + (long)n * g.ldb + kc[j];
            }
        }
        const int KT = (g.K + BK - 1) / BK;             // blocks along K
        const int NS = (KT + KB - 1) / KB;              // stages
        // CONV: tap and channel of the block this wavefront group fetches next (stages are issued in order)
        int nx_tap = 0, nx_r = 0, nx_s = 0, nx_ci = 0;
        if (CONV) {
            nx_tap = kb * BK / g.Cin;
            nx_ci = kb * BK - nx_tap * g.Cin;
            nx_r = nx_tap / g.S;
            nx_s = nx_tap - nx_r * g.S;
        }
        auto issue = [&](int s) {
            const int k0 = (s * KB + kb) * BK;          // first K element of this wavefront group's block
            const unsigned sbase = lds0 + ((unsigned)s % STAGES) * STAGE_BYTES + (unsigned)kb * BLK_BYTES;
            const unsigned tap_bit = (k0 < g.K && nx_tap < 32) ? 1u << nx_tap : 0u;  // blocks past K have no tap
            const int tap_off = (nx_r * g.W + nx_s) * (int)g.lda + nx_ci;  // elements from the window's origin
#pragma unroll
            for (int j = 0; j < LPW; ++j) {
                const int gi = group_of(wv, j);
                if (CONV && j < LPW_A) {
                    // taps outside the image, rows outside the problem and blocks past K come from the zero page
                    const bool ok = (taps[CONV ? j : 0] & tap_bit) != 0;
                    load_lds16(ok ? base[j] + tap_off : zero, sbase + (unsigned)(gi * 8 * RB));
                } else {
                    // rows outside the problem and K-chunks past K (also whole blocks past the last one,
                    // when the stage is not full) come from the zero page
                    const bool ok = row_ok[j] & (k0 + kc[j] < g.K);
                    load_lds16(ok ? base[j] + k0 : zero, sbase + (unsigned)(gi * 8 * RB));
                }
            }
            if (CONV) {
                nx_ci += KB * BK;
                while (nx_ci >= g.Cin) {
                    nx_ci -= g.Cin;
                    ++nx_tap;
                    if (++nx_s == g.S) { nx_s = 0; ++nx_r; }
                }
            }
        };

        f32x16 acc[BPW];
#pragma unroll
        for (int q = 0; q < BPW; ++q)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[q][v] = 0.f;
        auto frag = [&](int stage, int blk, int region_bytes, int row, int chunk) -> u32x4 {
            const int phys = chunk ^ ((row >> 1) & 7);
            return *(const u32x4 *)(lds_c + (size_t)stage * STAGE_BYTES + (size_t)blk * BLK_BYTES + region_bytes + row * RB + phys * 16);
        };

        // ---- main loop ------------------------------------------------------------------------
        GP_PROBE(1);
        __syncthreads();  // the previous tile of this workgroup may still be reading LDS
#pragma unroll
        for (int s = 0; s < PRE; ++s) {
            if (s < NS) issue(s);
            if (s == 0 && early && wave == 0) load_lds4(cc.stop_index, (unsigned)(size_t)(__attribute__((address_space(3))) void *)early_slot);
        }
        for (int s = 0; s < NS; ++s) {
            // stage s has landed once at most the loads of the younger stages in flight remain
            if (s == 0) wait_stages<LPW>((NS < PRE ? NS : PRE) - 1);
            else if (s + STAGES - 2 < NS) wait_vmcnt<(STAGES - 2) * LPW>();
            else wait_vmcnt<0>();
            __syncthreads();  // everyone's part of stage s is visible; the buffer of stage s-1 is free
            if (s == 0) GP_PROBE(2);
            if (((s == 0 && early) || (looking && s > 0 && (s & (LOOK_EVERY - 1)) == 0)) && __builtin_amdgcn_readfirstlane(read_lds_word(early_slot)) != -1) {
                wait_vmcnt<0>();  // loads still landing in LDS must not outlive the workgroup
                return true;      // the tile is given up: the caller withdraws the claim
            }
            if constexpr (LOOKS) {
                // the last stage: the workgroup counts itself (tile_fixed_early).  Not earlier: an atomic in front of operand
                // loads is waited for with them (the waits count in the order of issue), and its acknowledgement takes
                // microseconds when every resident workgroup sends one.
                if (looking && cc.announce && s == NS - 1 && tid == 0)
                    __hip_atomic_fetch_add(cc.announce, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (s >= PRE - (STAGES - 1) && s + STAGES - 1 < NS) {
                if (looking && wave == 0 && ((s + STAGES - 1) & (LOOK_EVERY - 1)) == 0)
                    load_lds4(cc.stop_index, (unsigned)(size_t)(__attribute__((address_space(3))) void *)early_slot);
                issue(s + STAGES - 1);
            }
            if (kb >= G) continue;  // (uniform) the other wavefronts only fetch
            const int stage = (int)((unsigned)s % STAGES);
#pragma unroll
            for (int b = 0; b < KB; ++b) {
                // a block past the last one holds zeros; it is skipped, not multiplied, so that the sum
                // has the bits of a K loop that ends at the last block
                if (s * KB + b >= KT) break;
#pragma unroll
                for (int q = 0; q < BPW; ++q) {
                    const int blk = kb + q * G, i = blk / NI, j = blk % NI;
                    const u32x4 fa = frag(stage, b, 0, i * 32 + l32, wv * 2 + half);
                    const u32x4 fb = frag(stage, b, A_BYTES, j * 32 + l32, wv * 2 + half);
                    Elem<T>::mma(fa, fb, acc[q]);
                }
            }
        }

        GP_PROBE(3);
        wide_reduce_store<T, BM, BN, NT, G>(g, (float *)lds_t, acc, m0, n0, offc, tid, wv, lane, kb);
#ifdef GP_TILE_PROF
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        GP_PROBE(5);
#endif
        return false;
    }
};

}  // namespace gp
