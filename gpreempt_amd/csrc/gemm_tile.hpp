// Register-staged tile kernel: both operands go global -> registers -> LDS with a one-step
// register prefetch.  It handles every layout (including B stored K x N, which is transposed on
// the way into LDS) and is the fallback of the pipelined kernel in gemm_pipe.hpp.
#pragma once
#include "mma.hpp"

namespace gp {

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool CONV, bool B_KN>
struct TileKernel {
    using elem = T;
    static constexpr int bm = BM, bn = BN;
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int NT = WGM * WGN * 64;
    static constexpr int LDK = BK + VEC;           // LDS row stride in elements (16-byte pad)
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int KSTEP = 2 * VEC;          // K consumed per mma() call
    static constexpr int A_CHUNKS = BM * BK / VEC, B_CHUNKS = BN * BK / VEC;
    static constexpr int A_PER = (A_CHUNKS + NT - 1) / NT, B_PER = (B_CHUNKS + NT - 1) / NT;
    static constexpr size_t LDS_BYTES = (size_t)(BM + BN) * LDK * sizeof(T);
    static constexpr bool early_stop = false;
    static constexpr bool can_look = false;
    static_assert(BK % KSTEP == 0 && WM % 32 == 0 && WN % 32 == 0, "tile shape");
    static_assert(A_CHUNKS % NT == 0 && B_CHUNKS % NT == 0, "loader shape");

    static __device__ __forceinline__ void run(const MatArgs &g, TileIdx t, T *lds) {
        T *As = lds, *Bs = lds + BM * LDK;
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int wm = wave / WGN, wn = wave % WGN;
        const int l32 = lane & 31, half = lane >> 5;
        const int m0 = t.y * BM, n0 = t.x * BN;
        long offa = 0, offb = 0, offc = 0;
        if (g.batch_inner > 0) {
            int zo = t.z / g.batch_inner, zi = t.z - zo * g.batch_inner;
            offa = zo * g.stride_a_outer + zi * g.stride_a;
            offb = zo * g.stride_b_outer + zi * g.stride_b;
            offc = zo * g.stride_c_outer + zi * g.stride_c;
        } else {
            offa = t.z * g.stride_a; offb = t.z * g.stride_b; offc = t.z * g.stride_c;
        }
        const T *A = (const T *)g.A + offa, *B = (const T *)g.B + offb;

        // Per-thread loader slots: which (row, k-chunk) of the tile each 16-byte load covers.
        constexpr int KC = BK / VEC;  // chunks per tile row
        int a_row[A_PER], a_kc[A_PER];
        long a_base[A_PER];           // GEMM: element offset of the row; CONV: offset of image n
        int a_h0[A_PER], a_w0[A_PER]; // CONV: top-left input coordinate of the pixel's window
        bool a_ok[A_PER];
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            int c = tid + i * NT;
            a_row[i] = c / KC; a_kc[i] = c % KC;
            int m = m0 + a_row[i];
            a_ok[i] = m < g.M;
            if (CONV) {
                int mm = a_ok[i] ? m : 0;
                int n = mm / (g.Ho * g.Wo), rem = mm - n * (g.Ho * g.Wo);
                int ho = rem / g.Wo, wo = rem - ho * g.Wo;
                a_h0[i] = ho * g.sh - g.ph; a_w0[i] = wo * g.sw - g.pw;
                a_base[i] = (long)n * g.H * g.W * g.lda;
            } else {
                a_base[i] = (long)m * g.lda; a_h0[i] = a_w0[i] = 0;
            }
        }
        int b_row[B_PER], b_kc[B_PER];
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            int c = tid + i * NT;
            if (B_KN) { b_row[i] = c / (BN / VEC); b_kc[i] = c % (BN / VEC); }  // row = k, kc = n-chunk
            else { b_row[i] = c / KC; b_kc[i] = c % KC; }
        }

        u32x4 ra[A_PER], rb[B_PER];
        auto load_global = [&](int kt) {
            const int k0 = kt * BK;
#pragma unroll
            for (int i = 0; i < A_PER; ++i) {
                int k = k0 + a_kc[i] * VEC;
                u32x4 v = {0, 0, 0, 0};
                if (a_ok[i] && k < g.K) {
                    if (CONV) {
                        int rs = k / g.Cin, ci = k - rs * g.Cin;
                        int r = rs / g.S, s = rs - r * g.S;
                        int hi = a_h0[i] + r, wi = a_w0[i] + s;
                        if ((unsigned)hi < (unsigned)g.H && (unsigned)wi < (unsigned)g.W)
                            v = *(const u32x4 *)(A + a_base[i] + ((long)hi * g.W + wi) * g.lda + ci);
                    } else {
                        v = *(const u32x4 *)(A + a_base[i] + k);
                    }
                }
                ra[i] = v;
            }
#pragma unroll
            for (int i = 0; i < B_PER; ++i) {
                u32x4 v = {0, 0, 0, 0};
                if (B_KN) {
                    int k = k0 + b_row[i], n = n0 + b_kc[i] * VEC;
                    if (k < g.K && n < g.N) v = *(const u32x4 *)(B + (long)k * g.ldb + n);
                } else {
                    int k = k0 + b_kc[i] * VEC, n = n0 + b_row[i];
                    if (k < g.K && n < g.N) v = *(const u32x4 *)(B + (long)n * g.ldb + k);
                }
                rb[i] = v;
            }
        };
        auto store_lds = [&]() {
#pragma unroll
            for (int i = 0; i < A_PER; ++i) *(u32x4 *)(As + a_row[i] * LDK + a_kc[i] * VEC) = ra[i];
#pragma unroll
            for (int i = 0; i < B_PER; ++i) {
                if (B_KN) {
                    // transpose on the way in: element j of the chunk is B[k][n + j]
                    T tmp[VEC];
                    *(u32x4 *)tmp = rb[i];
#pragma unroll
                    for (int j = 0; j < VEC; ++j) Bs[(b_kc[i] * VEC + j) * LDK + b_row[i]] = tmp[j];
                } else {
                    *(u32x4 *)(Bs + b_row[i] * LDK + b_kc[i] * VEC) = rb[i];
                }
            }
        };

        f32x16 acc[MI][NI];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

        const int KT = (g.K + BK - 1) / BK;
        load_global(0);
        __syncthreads();  // the previous tile of this workgroup may still be reading LDS
        store_lds();
        __syncthreads();
        for (int kt = 0; kt < KT; ++kt) {
            if (kt + 1 < KT) load_global(kt + 1);
#pragma unroll
            for (int ks = 0; ks < BK / KSTEP; ++ks) {
                u32x4 fa[MI], fb[NI];
#pragma unroll
                for (int i = 0; i < MI; ++i)
                    fa[i] = *(const u32x4 *)(As + (wm * WM + i * 32 + l32) * LDK + ks * KSTEP + half * VEC);
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    fb[j] = *(const u32x4 *)(Bs + (wn * WN + j * 32 + l32) * LDK + ks * KSTEP + half * VEC);
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j) Elem<T>::mma(fa[i], fb[j], acc[i][j]);
            }
            if (kt + 1 < KT) {
                __syncthreads();
                store_lds();
                __syncthreads();
            }
        }

        // Epilogue: lane holds column n = l32 and rows 8*(v/4) + 4*half + v%4 of each 32x32 block.
        T *C = (T *)g.C + offc;
        const T *R = g.residual ? (const T *)g.residual + offc : nullptr;
        const T *bias = (const T *)g.bias;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            int n = n0 + wn * WN + j * 32 + l32;
            if (n >= g.N) continue;
            float bv = bias ? Elem<T>::to_f(bias[n]) : 0.f;
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int m = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                    if (m >= g.M) continue;
                    float x = acc[i][j][v] * g.alpha + bv;
                    if (R) x += Elem<T>::to_f(R[(long)m * g.ldr + n]);
                    st_elem<T>(&C[(long)m * g.ldc + n], Elem<T>::from_f(apply_act(x, g.act)));
                }
            }
        }
    }
};

}  // namespace gp
