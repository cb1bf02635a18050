// Layer-norm + GEMM in one kernel, for small deep-learning shapes where a launch costs more than the
// arithmetic: C = act(LN(A) * B^T + bias [+ residual]), with LN(A) also written out once.
//
// Why: in a transformer layer at batch 1 the layer-norm kernel in front of the QKV and the first FFN
// projection moves 0.4 MB and takes as long as any dependent launch takes on this GPU (about 5 us),
// a fifth of the request.  The projection's workgroups read their rows of A anyway, and a row is
// short (K elements), so every workgroup normalises its own BM rows before it multiplies them:
// the rows go from global memory through registers into LDS, where they stay for the whole tile
// (BM x K elements: 48 KB for 32 rows of 768 halves), and only B streams through the ring of
// gemm_wide.hpp.  The workgroups of tile column 0 also store the normalised rows, for the later
// kernels that read them (the residual additions).
//
// Same bits as the two-kernel form: a row is normalised by one wavefront through ln_rows_math, the
// function the stand-alone layer-norm kernel uses, with the same lane-to-chunk assignment, and
// rounded to the storage type before it is multiplied, as it would be on its way through memory;
// the main loop and the reduction are those of WideKernel (wavefront w multiplies MFMA k-step w of
// every K-block, partial tiles summed in wavefront order).
#pragma once
#include "elementwise_bodies.hpp"
#include "gemm_wide.hpp"

namespace gp {

template <typename T, int BM, int BN, int WAVES, int STAGES>
struct LnWideKernel {
    using elem = T;
    static constexpr int bm = BM, bn = BN;
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int NT = WAVES * 64;
    static constexpr int RB = 128;                         // row bytes of a block in LDS
    static constexpr int BK = RB / (int)sizeof(T);         // K elements per block
    static constexpr int KB = WAVES / 4;                   // blocks per stage
    static constexpr int LPW = BN / 8 / 4;                 // B row groups a wavefront fetches per stage
    static constexpr int MAXK = 832;                       // longest row: BM x MAXK elements stay resident (104 KB of the 160)
    static constexpr int MAXC = 2;                         // 16-byte chunks of a row per lane (ln_rows_math): K <= 128 * VEC
    static constexpr int A_BLK_BYTES = BM * RB;            // one K-block of the resident rows
    static constexpr int B_BLK_BYTES = BN * RB, STAGE_BYTES = KB * B_BLK_BYTES;
    static constexpr int MI = BM / 32, NI = BN / 32;
    // wavefront group kb < G multiplies for the output blocks kb, kb + G, ... (WideKernel keeps G = 1; here two
    // groups, one per 32 x 32 block of the 32 x 64 tile, took 0.25-0.3 us off a launch: 7.87 -> 7.62, 8.43 -> 8.13)
    static constexpr int G = MI * NI < KB ? MI * NI : KB, BPW = MI * NI / G;
    static_assert(MI * NI % G == 0, "output blocks divide among the multiplying groups");
    static constexpr int SLICES = MI * NI * 16;
    static constexpr size_t RED_BYTES = (size_t)4 * SLICES * 64 * 4;
    static constexpr size_t RING_BYTES = (size_t)STAGES * STAGE_BYTES;
    static constexpr size_t A_RES_BYTES = (size_t)BM * MAXK * sizeof(T);
    // the reduction buffer reuses the ring, which lies in front of the resident rows
    static constexpr size_t RING_REGION = RING_BYTES > RED_BYTES ? RING_BYTES : RED_BYTES;
    static constexpr size_t LDS_BYTES = RING_REGION + A_RES_BYTES;
    static constexpr size_t CKPT_SLOT_BYTES = 0;
    static constexpr bool ckpt = false;
    static constexpr bool early_stop = true;
    static constexpr bool can_look = false;
    static constexpr int PRE = GP_WIDE_PREFILL ? STAGES : STAGES - 1;
    static_assert(sizeof(T) == 2, "16-bit element types");
    static_assert(WAVES == 16 && BM % WAVES == 0 && BN % 32 == 0 && BM % 32 == 0, "tile shape");
    static_assert(STAGES >= 2 && STAGES <= 4 && (STAGES - 1) * LPW < 64, "pipeline depth");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");

    static __device__ __forceinline__ bool run(const MatArgs &g, TileIdx t, T *lds_t, CkptCtx cc = CkptCtx{nullptr, nullptr, nullptr, 0}) {
        GP_PROBE(0);
        __shared__ int early_slot[64];
        const bool early = __builtin_amdgcn_readfirstlane((int)(cc.stop_index != nullptr)) != 0;
        const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) void *)lds_t;
        char *lds_c = (char *)lds_t;
        char *a_res = lds_c + RING_REGION;
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int kb = wave >> 2, wv = wave & 3;
        const int l32 = lane & 31, half = lane >> 5;
        const int m0 = t.y * BM, n0 = t.x * BN;
        const T *A = (const T *)g.A, *B = (const T *)g.B;
        const T *zero = (const T *)g_zero_page;
        const int KT = g.K / BK;                        // blocks along K (K is a multiple of BK: checked by the planner)
        const int NS = (KT + KB - 1) / KB;              // stages of B

        // ---- B loader slots, as in WideKernel ---------------------------------------------------
        const int rig = lane >> 3, cpos = lane & 7;
        const T *base[LPW];
        bool row_ok[LPW];
        int kc[LPW];
#pragma unroll
        for (int j = 0; j < LPW; ++j) {
            const int r = (wv * LPW + j) * 8 + rig;
            kc[j] = (cpos ^ ((r >> 1) & 7)) * VEC;
            row_ok[j] = n0 + r < g.N;
            base[j] = B + (long)(n0 + r) * g.ldb + kc[j];
        }
        auto issue = [&](int s) {
            const int k0 = (s * KB + kb) * BK;
            const unsigned sbase = lds0 + ((unsigned)s % STAGES) * STAGE_BYTES + (unsigned)kb * B_BLK_BYTES;
#pragma unroll
            for (int j = 0; j < LPW; ++j) {
                const bool ok = row_ok[j] & (k0 < g.K);   // whole blocks past the last one, when the stage is not full
                load_lds16(ok ? base[j] + k0 : zero, sbase + (unsigned)((wv * LPW + j) * 8 * RB));
            }
        };

        __syncthreads();  // the previous tile of this workgroup may still be reading LDS

        // ---- the rows of A: normalise, keep in LDS, store once -------------------------------------
        // wavefront w takes rows w, w + WAVES, ...; lane l holds chunks l and l + 64 of a row.  The rows are
        // asked for first and B only once they are here: the wait for them would otherwise also wait for
        // B (the counter of outstanding loads does not tell them apart), and B's way from memory is then
        // covered by the arithmetic on the rows.
        {
            constexpr int RPW = BM / WAVES;
            const int chunks = g.K / VEC;
            out_u32x4 rx[RPW][MAXC];
#pragma unroll
            for (int q = 0; q < RPW; ++q) {
                const int m = m0 + wave + q * WAVES;
                const T *x = A + (long)(m < g.M ? m : g.M - 1) * g.lda;
#pragma unroll
                for (int i = 0; i < MAXC; ++i) {
                    const int ch = lane + i * 64;
                    rx[q][i] = out_u32x4{0, 0, 0, 0};
                    if (ch < chunks) rx[q][i] = *(const out_u32x4 *)(x + ch * VEC);
                }
            }
            // gamma and beta with them: a wait for them later would be a wait for B as well
            out_u32x4 graw[MAXC], braw[MAXC];
#pragma unroll
            for (int i = 0; i < MAXC; ++i) {
                const int ch = lane + i * 64;
                graw[i] = braw[i] = out_u32x4{0, 0, 0, 0};
                if (ch < chunks) {
                    graw[i] = *(const out_u32x4 *)((const T *)g.ln_gamma + ch * VEC);
                    braw[i] = *(const out_u32x4 *)((const T *)g.ln_beta + ch * VEC);
                }
            }
#pragma unroll
            for (int i = 0; i < MAXC; ++i) {
#pragma unroll
                for (int q = 0; q < RPW; ++q) asm volatile("" : "+v"(rx[q][i]) :: "memory");  // the rows have arrived
                asm volatile("" : "+v"(graw[i]), "+v"(braw[i]) :: "memory");
            }
#pragma unroll
            for (int s = 0; s < PRE; ++s) {
                if (s < NS) issue(s);
                if (s == 0 && early && wave == 0) load_lds4(cc.stop_index, (unsigned)(size_t)(__attribute__((address_space(3))) void *)early_slot);
            }
            float v[RPW][MAXC][VEC];
#pragma unroll
            for (int q = 0; q < RPW; ++q)
#pragma unroll
                for (int i = 0; i < MAXC; ++i) {
                    const int ch = lane + i * 64;
                    if (ch < chunks) VecIO<T>::unpack(rx[q][i], v[q][i]);
                }
            out_u32x4 y[RPW][MAXC];
            ln_rows_math<T, MAXC, RPW, true>(v, chunks, lane, g.K, g.ln_eps, (const T *)g.ln_gamma, (const T *)g.ln_beta, graw, braw, y);
#pragma unroll
            for (int q = 0; q < RPW; ++q) {
                const int r = wave + q * WAVES, m = m0 + r;
#pragma unroll
                for (int i = 0; i < MAXC; ++i) {
                    const int ch = lane + i * 64;
                    if (ch < chunks) {
                        // chunk ch of the row is chunk ch % 8 of K-block ch / 8, at the swizzled position
                        const int blk = ch >> 3, phys = (ch & 7) ^ ((r >> 1) & 7);
                        *(out_u32x4 *)(a_res + (size_t)blk * A_BLK_BYTES + r * RB + phys * 16) = y[q][i];
                    }
                }
            }
        }

        GP_PROBE(1);
        f32x16 acc[BPW];
#pragma unroll
        for (int q = 0; q < BPW; ++q)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[q][v] = 0.f;
        auto frag_a = [&](int blk, int row, int chunk) -> u32x4 {
            const int phys = chunk ^ ((row >> 1) & 7);
            return *(const u32x4 *)(a_res + (size_t)blk * A_BLK_BYTES + row * RB + phys * 16);
        };
        auto frag_b = [&](int stage, int blk, int row, int chunk) -> u32x4 {
            const int phys = chunk ^ ((row >> 1) & 7);
            return *(const u32x4 *)(lds_c + (size_t)stage * STAGE_BYTES + (size_t)blk * B_BLK_BYTES + row * RB + phys * 16);
        };

        // ---- main loop: B streams, A is there ------------------------------------------------------
        for (int s = 0; s < NS; ++s) {
            if (s == 0) wait_stages<LPW>((NS < PRE ? NS : PRE) - 1);
            else if (s + STAGES - 2 < NS) wait_vmcnt<(STAGES - 2) * LPW>();
            else wait_vmcnt<0>();
            __syncthreads();  // stage s of B (and, the first time, the rows of A) visible; the buffer of stage s-1 is free
            if (s == 0) GP_PROBE(2);
            if (s == 0 && early && __builtin_amdgcn_readfirstlane(read_lds_word(early_slot)) != -1) {
                wait_vmcnt<0>();  // loads still landing in LDS must not outlive the workgroup
                return true;
            }
            // The workgroups of tile column 0 store the normalised rows, and only now: a launch that started
            // eagerly behind a stopped kernel normalised rows of an incomplete x, and must leave (above) without
            // having written anything.  Every wavefront stores the rows it normalised, from their copy in LDS.
            if (s == 0 && t.x == 0) {
                const int chunks = g.K / VEC;
#pragma unroll
                for (int q = 0; q < BM / WAVES; ++q) {
                    const int r = wave + q * WAVES, m = m0 + r;
#pragma unroll
                    for (int i = 0; i < MAXC; ++i) {
                        const int ch = lane + i * 64;
                        if (ch < chunks && m < g.M) {
                            const int blk = ch >> 3, phys = (ch & 7) ^ ((r >> 1) & 7);
                            st_out128((T *)g.ln_out + (long)m * g.K + ch * VEC, *(const out_u32x4 *)(a_res + (size_t)blk * A_BLK_BYTES + r * RB + phys * 16));
                        }
                    }
                }
            }
            if (s >= PRE - (STAGES - 1) && s + STAGES - 1 < NS) issue(s + STAGES - 1);
            if (kb >= G) continue;  // (uniform) the other wavefronts only fetch
            const int stage = (int)((unsigned)s % STAGES);
#pragma unroll
            for (int b = 0; b < KB; ++b) {
                if (s * KB + b >= KT) break;
#pragma unroll
                for (int q = 0; q < BPW; ++q) {
                    const int blk = kb + q * G, i = blk / NI, j = blk % NI;
                    const u32x4 fa = frag_a(s * KB + b, i * 32 + l32, wv * 2 + half);
                    const u32x4 fb = frag_b(stage, b, j * 32 + l32, wv * 2 + half);
                    Elem<T>::mma(fa, fb, acc[q]);
                }
            }
        }
        GP_PROBE(3);
        wide_reduce_store<T, BM, BN, NT, G>(g, (float *)lds_t, acc, m0, n0, 0, tid, wv, lane, kb);
#ifdef GP_TILE_PROF
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        GP_PROBE(5);
#endif
        return false;
    }
};

}  // namespace gp
