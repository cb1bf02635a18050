// Element types, MFMA wrappers and the argument block shared by the matrix kernels.
#pragma once
#include "common.hpp"
#include "out_store.hpp"

namespace gp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// loop whose index is a compile-time constant in the body (register arrays stay registers)
template <int I> struct IntC { static constexpr int value = I; constexpr operator int() const { return I; } };
template <int B, int E, class F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (B < E) {
        f(IntC<B>{});
        static_for<B + 1, E>(f);
    }
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ void mma(u32x4 a, u32x4 b, f32x16 &acc) {
        f32x4 fa = __builtin_bit_cast(f32x4, a), fb = __builtin_bit_cast(f32x4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[i], acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f(float v) { return v; }
    static __device__ __forceinline__ float from_f(float v) { return v; }
};
template <> struct Elem<_Float16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void mma(u32x4 a, u32x4 b, f32x16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f(_Float16 v) { return (float)v; }
    static __device__ __forceinline__ _Float16 from_f(float v) { return (_Float16)v; }
};
template <> struct Elem<__bf16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void mma(u32x4 a, u32x4 b, f32x16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f(__bf16 v) { return (float)v; }
    static __device__ __forceinline__ __bf16 from_f(float v) { return (__bf16)v; }
};

__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == GP_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == GP_ACT_GELU) return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
    return v;
}

struct MatArgs {
    // GEMM view: C[M,N] = A[M,K] * B ; conv fills the conv fields and M = N*Ho*Wo, K = R*S*Cin.
    int M, N, K;
    const void *A; long lda, stride_a, stride_a_outer;
    const void *B; long ldb, stride_b, stride_b_outer;
    void *C; long ldc, stride_c, stride_c_outer;
    const void *bias;
    const void *residual; long ldr;
    float alpha;
    int act;
    int batch_inner;
    // convolution geometry (CONV only)
    int H, W, Cin, S, Ho, Wo, sh, sw, ph, pw;
    // layer-norm prologue (gemm_ln.hpp; ln_gamma == nullptr: none): the rows of A are normalised over
    // their K elements before they are multiplied, and written to ln_out (M x K)
    const void *ln_gamma, *ln_beta;
    void *ln_out;
    float ln_eps;
};

}  // namespace gp
