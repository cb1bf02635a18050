// Fused scaled-dot-product attention; a tile is one (batch, head, 128-query block):
//   O = softmax(Q K^T * scale) V      with head dimension 64, 16-bit operands, fp32 softmax.
//
// It replaces three launches (batched Q K^T, row softmax, batched P V) and the two S x S score
// tensors they pass through memory.  One wavefront owns 32 query rows and computes the transposed
// scores S^T = K Q^T with v_mfma_f32_32x32x16: in the accumulator layout a lane then holds, for
// ITS query (column lane%32), the scores of keys 8*(v/4) + 4*(lane/32) + v%4 of every 32-key
// block, so the row softmax is a reduction over the lane's own registers plus one exchange with
// lane^32, and the probabilities are already laid out as the A operand of the second product:
// an MFMA only needs A and B to agree on which K indices a (lane, register) pair stands for,
// and V^T is staged in LDS so that the B fragments can be gathered in that same key order.
#pragma once
#include "mma.hpp"

namespace gp {

struct AttnArgs {
    gp_attention_params p;
};

constexpr int ATT_D = 64;        // head dimension
constexpr int ATT_QB = 128;      // query rows per tile (32 per wave)
__host__ __device__ inline int attention_key_blocks(int seq) { return (seq + 31) / 32; }
__host__ __device__ inline size_t attention_lds_bytes(int nb) { return (size_t)ATT_D * (nb * 32 + 4) * 2; }

template <typename T, int NB>
__device__ __forceinline__ void attention_tile(const AttnArgs &a, TileIdx t, T *vt) {
    const gp_attention_params &p = a.p;
    // padded row of V^T: consecutive rows (d) start 2 banks apart, so the 8-byte fragment reads of 16
    // lanes cover all 32 banks once
    constexpr int SP = NB * 32 + 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const int S = p.seq;
    const int head = t.y % p.heads, bat = t.y / p.heads;  // tile grid: x = query block, y = batch * heads + head
    const long tok0 = (long)bat * S;
    const T *Q = (const T *)p.q + tok0 * p.ld_qkv + (long)head * ATT_D;
    const T *K = (const T *)p.k + tok0 * p.ld_qkv + (long)head * ATT_D;
    const T *V = (const T *)p.v + tok0 * p.ld_qkv + (long)head * ATT_D;
    T *O = (T *)p.out + tok0 * p.ld_out + (long)head * ATT_D;
    const u32x4 zero4 = {0, 0, 0, 0};

    // ---- operand fetches first: Q and (for short sequences) every K fragment are requested before
    // V is staged, so that their latency overlaps the staging instead of following it ------------
    const int q = t.x * ATT_QB + wave * 32 + l32;  // this lane's query row
    u32x4 bq[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bq[ks] = q < S ? *(const u32x4 *)(Q + (long)q * p.ld_qkv + ks * 16 + half * 8) : zero4;
    constexpr bool PREFETCH_K = NB <= 4;  // 16 registers per key block
    u32x4 ak[PREFETCH_K ? NB : 1][4];
    if constexpr (PREFETCH_K) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int key = nb * 32 + l32;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) ak[nb][ks] = key < S ? *(const u32x4 *)(K + (long)key * p.ld_qkv + ks * 16 + half * 8) : zero4;
        }
    }

    // ---- V^T into LDS: vt[d][key], keys past the sequence zero-filled (their probability is 0,
    // but 0 * garbage could be NaN) -----------------------------------------------------------
    __syncthreads();  // the previous tile of this workgroup may still be reading vt
    for (int idx = tid; idx < NB * 32 * (ATT_D / 8); idx += 256) {
        // a wavefront takes 64 consecutive keys of one 8-wide d chunk: its transposing 2-byte
        // writes are then 128 contiguous bytes per d, free of bank conflicts
        const int key = idx % (NB * 32), dc = idx / (NB * 32);
        u32x4 raw = key < S ? *(const u32x4 *)(V + (long)key * p.ld_qkv + dc * 8) : zero4;
        const unsigned short *e = (const unsigned short *)&raw;
#pragma unroll
        for (int j = 0; j < 8; ++j) ((unsigned short *)vt)[(dc * 8 + j) * SP + key] = e[j];
    }
    __syncthreads();

    // ---- scores (transposed): s[nb][v] = <K[key], Q[query]> ------------------------------------
    f32x16 s[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[nb][v] = 0.f;
        const int key = nb * 32 + l32;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 a_k;
            if constexpr (PREFETCH_K) a_k = ak[nb][ks];
            else a_k = key < S ? *(const u32x4 *)(K + (long)key * p.ld_qkv + ks * 16 + half * 8) : zero4;
            Elem<T>::mma(a_k, bq[ks], s[nb]);
        }
    }
    // ---- softmax over the keys of this lane's query ---------------------------------------------
    float m = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = nb * 32 + 8 * (v / 4) + 4 * half + (v % 4);
            s[nb][v] = key < S ? s[nb][v] * p.scale : -INFINITY;
            m = fmaxf(m, s[nb][v]);
        }
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    float sum = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            s[nb][v] = __expf(s[nb][v] - m);
            sum += s[nb][v];
        }
    sum += __shfl_xor(sum, 32, 64);
    const float inv = 1.f / sum;

    // ---- O = P V: A = probabilities (already per query lane), B gathered from V^T ----------------
    f32x16 o[2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            // registers 8j..8j+7 of block nb are keys nb*32 + 16j + 4*half + {0..3} and + 8 + {0..3}
            typedef T tx8 __attribute__((ext_vector_type(8)));
            tx8 pa;
#pragma unroll
            for (int e = 0; e < 8; ++e) pa[e] = Elem<T>::from_f(s[nb][8 * j + e] * inv);
            const int kbase = nb * 32 + 16 * j + 4 * half;
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                const unsigned short *row = (const unsigned short *)vt + (db * 32 + l32) * SP + kbase;
                const unsigned long long lo = *(const unsigned long long *)row, hi = *(const unsigned long long *)(row + 8);
                u32x4 bv = {(unsigned)lo, (unsigned)(lo >> 32), (unsigned)hi, (unsigned)(hi >> 32)};
                Elem<T>::mma(__builtin_bit_cast(u32x4, pa), bv, o[db]);
            }
        }
    // ---- store: o[db][v] = O[query 8*(v/4) + 4*half + v%4][db*32 + lane%32] ----------------------
    const int q0 = t.x * ATT_QB + wave * 32;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int qr = q0 + 8 * (v / 4) + 4 * half + (v % 4);
            if (qr < S) st_elem<T>(O + (long)qr * p.ld_out + db * 32 + l32, Elem<T>::from_f(o[db][v]));
        }
}

// Key blocks the body is instantiated for: seq <= 128 / 256 / 384 / 512 keys.
__host__ __device__ inline int attention_nb_class(int seq) {
    const int nb = attention_key_blocks(seq);
    return nb <= 4 ? 4 : nb <= 8 ? 8 : nb <= 12 ? 12 : 16;
}

// One kernel per class: the score registers of the longest class (256 per lane) would otherwise set
// the register budget, and the scratch memory, of the short sequences too.
template <typename T, int NB>
__global__ __launch_bounds__(256) void attention_kernel(AttnArgs a, BlpArgs blp) {
    extern __shared__ __attribute__((aligned(16))) unsigned char att_lds[];
    tile_loop(blp, [&](TileIdx t) { attention_tile<T, NB>(a, t, reinterpret_cast<T *>(att_lds)); });
}

}  // namespace gp
