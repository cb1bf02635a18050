// Output stores of the tile bodies.
//
// Stand-alone kernels store normally: the kernel boundary makes their results visible.  Inside
// the whole-model program a tile's consumer may run on another XCD (each XCD has its own L2)
// within the same kernel, so there every output store is an agent-scope store (written through
// to device-coherent memory) and the producer only has to wait for its stores to complete
// before it counts the tile as done; a cache write-back fence per tile, which costs tens of
// microseconds, is not needed.  program.hip selects that form by defining GP_COHERENT_STORES
// before it includes the bodies; the bodies are always inlined into the including kernel.
#pragma once
#include <hip/hip_runtime.h>

namespace gp {

#ifdef GP_COHERENT_STORES
constexpr bool kCoherentStores = true;
#else
constexpr bool kCoherentStores = false;
#endif

typedef unsigned int out_u32x4 __attribute__((ext_vector_type(4)));

// experiment switch: stand-alone kernels store their outputs with the nontemporal hint
#ifdef GP_NT_STORES
#define GP_PLAIN_STORE(T, p, v) __builtin_nontemporal_store((T)(v), (T *)(p))
#else
#define GP_PLAIN_STORE(T, p, v) (*(T *)(p) = (v))
#endif

__device__ __forceinline__ void st_out16(void *p, unsigned short v) {
    if (kCoherentStores) __hip_atomic_store((unsigned short *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else GP_PLAIN_STORE(unsigned short, p, v);
}
__device__ __forceinline__ void st_out32(void *p, unsigned int v) {
    if (kCoherentStores) __hip_atomic_store((unsigned int *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else GP_PLAIN_STORE(unsigned int, p, v);
}
__device__ __forceinline__ void st_out64(void *p, unsigned long long v) {
    if (kCoherentStores) __hip_atomic_store((unsigned long long *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else GP_PLAIN_STORE(unsigned long long, p, v);
}
__device__ __forceinline__ void st_out128(void *p, out_u32x4 v) {
    if (kCoherentStores) {
        unsigned long long lo = ((unsigned long long)v[1] << 32) | v[0], hi = ((unsigned long long)v[3] << 32) | v[2];
        __hip_atomic_store((unsigned long long *)p, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store((unsigned long long *)p + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        GP_PLAIN_STORE(out_u32x4, p, v);
    }
}
__device__ __forceinline__ void st_out8(void *p, unsigned char v) {
    if (kCoherentStores) __hip_atomic_store((unsigned char *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else GP_PLAIN_STORE(unsigned char, p, v);
}

// typed element store
template <typename T> __device__ __forceinline__ void st_elem(T *p, T v);
template <> __device__ __forceinline__ void st_elem<float>(float *p, float v) { st_out32(p, __builtin_bit_cast(unsigned int, v)); }
template <> __device__ __forceinline__ void st_elem<_Float16>(_Float16 *p, _Float16 v) { st_out16(p, __builtin_bit_cast(unsigned short, v)); }
template <> __device__ __forceinline__ void st_elem<__bf16>(__bf16 *p, __bf16 v) { st_out16(p, __builtin_bit_cast(unsigned short, v)); }

}  // namespace gp
