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

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <typename T, int BM, int BN, int STAGES, bool CONV, bool SPLITK>
struct PipeKernel {
    using elem = T;
    static constexpr int bm = BM, bn = BN;
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int NT = 256, WAVES = 4;
    static constexpr int RB = 128;                        // row bytes in LDS
    static constexpr int BK = RB / (int)sizeof(T);        // 64 (16-bit) or 32 (fp32) elements
    static constexpr int KSTEPS = 4;                      // mma() calls per stage along K (2 chunks each)
    static constexpr int A_BYTES = BM * RB, B_BYTES = BN * RB, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int A_PW = BM / 8 / WAVES, B_PW = BN / 8 / WAVES;  // load instructions per wave per stage
    static constexpr int LPS = A_PW + B_PW;
    static constexpr int WGM = SPLITK ? 1 : 2, WGN = SPLITK ? 1 : 2;
    static constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / 32, NI = WN / 32;
    static constexpr size_t RED_BYTES = SPLITK ? (size_t)WAVES * MI * NI * 16 * 64 * 4 : 0;
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_BYTES > RED_BYTES ? (size_t)STAGES * STAGE_BYTES : RED_BYTES;
    static_assert(BM % 32 == 0 && BN % 32 == 0 && A_PW >= 1 && B_PW >= 1, "tile shape");
    static_assert(STAGES >= 2 && (STAGES - 2) * LPS < 64, "pipeline depth");

    static __device__ __forceinline__ void run(const MatArgs &g, TileIdx t, T *lds_t) {
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

        // ---- loader slots -------------------------------------------------------------------
        const int rig = lane >> 3, cpos = lane & 7;  // row within the 8-row group, chunk slot
        const T *a_row[A_PW];       // GEMM: pointer to the row start; CONV: pointer to image n
        int a_h0[A_PW], a_w0[A_PW]; // CONV: window origin of the output pixel
        int a_c[A_PW];              // logical chunk this lane fetches for that slot
        bool a_ok[A_PW];
#pragma unroll
        for (int j = 0; j < A_PW; ++j) {
            int row = (wave * A_PW + j) * 8 + rig;
            a_c[j] = cpos ^ ((row >> 1) & 7);
            int m = m0 + row;
            a_ok[j] = m < g.M;
            if (CONV) {
                int mm = a_ok[j] ? m : 0;
                int n = mm / (g.Ho * g.Wo), rem = mm - n * (g.Ho * g.Wo);
                int ho = rem / g.Wo, wo = rem - ho * g.Wo;
                a_h0[j] = ho * g.sh - g.ph; a_w0[j] = wo * g.sw - g.pw;
                a_row[j] = A + (long)n * g.H * g.W * g.lda;
            } else {
                a_row[j] = A + (long)(a_ok[j] ? m : 0) * g.lda;
                a_h0[j] = a_w0[j] = 0;
            }
        }
        const T *b_row[B_PW];
        int b_c[B_PW];
        bool b_ok[B_PW];
#pragma unroll
        for (int j = 0; j < B_PW; ++j) {
            int row = (wave * B_PW + j) * 8 + rig;
            b_c[j] = cpos ^ ((row >> 1) & 7);
            int n = n0 + row;
            b_ok[j] = n < g.N;
            b_row[j] = B + (long)(b_ok[j] ? n : 0) * g.ldb;
        }
        const bool conv_fast = CONV && (g.Cin % BK == 0);  // a K-step never straddles a filter tap

        auto issue = [&](int kt) {
            const unsigned sbase = lds0 + (unsigned)(kt % STAGES) * STAGE_BYTES;
            const int k0 = kt * BK;
            int r_u = 0, s_u = 0, ci_u = 0;
            if (conv_fast) {
                int rs = k0 / g.Cin;
                ci_u = k0 - rs * g.Cin;
                r_u = rs / g.S; s_u = rs - r_u * g.S;
            }
#pragma unroll
            for (int j = 0; j < A_PW; ++j) {
                const int k = k0 + a_c[j] * VEC;
                const T *src = zero;
                if (a_ok[j] && k < g.K) {
                    if (CONV) {
                        int r, s, ci;
                        if (conv_fast) { r = r_u; s = s_u; ci = ci_u + a_c[j] * VEC; }
                        else { int rs = k / g.Cin; ci = k - rs * g.Cin; r = rs / g.S; s = rs - r * g.S; }
                        int hi = a_h0[j] + r, wi = a_w0[j] + s;
                        if ((unsigned)hi < (unsigned)g.H && (unsigned)wi < (unsigned)g.W)
                            src = a_row[j] + ((long)hi * g.W + wi) * g.lda + ci;
                    } else {
                        src = a_row[j] + k;
                    }
                }
                load_lds16(src, sbase + (unsigned)((wave * A_PW + j) * 8 * RB));
            }
#pragma unroll
            for (int j = 0; j < B_PW; ++j) {
                const int k = k0 + b_c[j] * VEC;
                const T *src = (b_ok[j] && k < g.K) ? b_row[j] + k : zero;
                load_lds16(src, sbase + (unsigned)(A_BYTES + (wave * B_PW + j) * 8 * RB));
            }
        };

        f32x16 acc[MI][NI];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

        const int wm = SPLITK ? 0 : wave / WGN, wn = SPLITK ? 0 : wave % WGN;
        auto frag = [&](int stage, int region_bytes, int row, int chunk) -> u32x4 {
            int phys = chunk ^ ((row >> 1) & 7);
            return *(const u32x4 *)(lds_c + (size_t)stage * STAGE_BYTES + region_bytes + row * RB + phys * 16);
        };
        auto compute = [&](int stage) {
#pragma unroll
            for (int kq = 0; kq < (SPLITK ? 1 : KSTEPS); ++kq) {
                const int ks = SPLITK ? wave : kq;
                u32x4 fa[MI], fb[NI];
#pragma unroll
                for (int i = 0; i < MI; ++i) fa[i] = frag(stage, 0, wm * WM + i * 32 + l32, ks * 2 + half);
#pragma unroll
                for (int j = 0; j < NI; ++j) fb[j] = frag(stage, A_BYTES, wn * WN + j * 32 + l32, ks * 2 + half);
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j) Elem<T>::mma(fa[i], fb[j], acc[i][j]);
            }
        };

        // ---- main loop ------------------------------------------------------------------------
        const int KT = (g.K + BK - 1) / BK;
        __syncthreads();  // the previous tile of this workgroup may still be reading LDS
#pragma unroll
        for (int s = 0; s < STAGES - 1; ++s)
            if (s < KT) issue(s);
        for (int kt = 0; kt < KT; ++kt) {
            // stage kt has landed once at most the loads of the younger in-flight stages remain
            if (KT - kt - 1 >= STAGES - 2) wait_vmcnt<(STAGES - 2) * LPS>();
            else wait_vmcnt<0>();
            __syncthreads();  // everyone's part of stage kt is visible; stage kt-1's buffer is free
            if (kt + STAGES - 1 < KT) issue(kt + STAGES - 1);
            compute(kt % STAGES);
        }

        // ---- epilogue -------------------------------------------------------------------------
        T *C = (T *)g.C + offc;
        const T *R = g.residual ? (const T *)g.residual + offc : nullptr;
        const T *bias = (const T *)g.bias;
        auto emit = [&](int i, int j, int v, float a) {
            int n = n0 + wn * WN + j * 32 + l32;
            int m = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
            if (n >= g.N || m >= g.M) return;
            float x = a * g.alpha + (bias ? Elem<T>::to_f(bias[n]) : 0.f);
            if (R) x += Elem<T>::to_f(R[(long)m * g.ldr + n]);
            st_elem<T>(&C[(long)m * g.ldc + n], Elem<T>::from_f(apply_act(x, g.act)));
        };
        if (!SPLITK) {
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) emit(i, j, v, acc[i][j][v]);
        } else {
            // partial sums -> LDS as [wave][slice][lane], slice = (i*NI + j)*16 + v
            float *red = (float *)lds_t;
            constexpr int SLICES = MI * NI * 16;
            __syncthreads();  // all waves are done reading the stage buffers
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) red[((size_t)wave * SLICES + (i * NI + j) * 16 + v) * 64 + lane] = acc[i][j][v];
            __syncthreads();
            // wave w finishes slices w, w+4, ...: fixed summation order over the four partials
#pragma unroll
            for (int sidx = 0; sidx < SLICES / WAVES; ++sidx) {
                int sl = sidx * WAVES + wave;
                float a = red[((size_t)0 * SLICES + sl) * 64 + lane];
                a += red[((size_t)1 * SLICES + sl) * 64 + lane];
                a += red[((size_t)2 * SLICES + sl) * 64 + lane];
                a += red[((size_t)3 * SLICES + sl) * 64 + lane];
                int blk = sl / 16, v = sl % 16;
                emit(blk / NI, blk % NI, v, a);
            }
        }
    }
};

}  // namespace gp
