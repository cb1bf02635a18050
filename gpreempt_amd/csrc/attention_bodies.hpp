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

// V^T into LDS: vt[d][key] for NB * 32 keys, keys past the sequence zero-filled.  A thread moves
// NB * 32 * 8 / 256 chunks of eight d values; a wavefront takes 64 consecutive keys of one chunk, so
// its transposing 2-byte writes are 128 contiguous bytes per d, free of bank conflicts.  The chunks
// are fetched up to eight at a time before any is written (as one loop over the chunks, every
// iteration waited for its own load; 384 keys: 12.95 -> 12.3 us per launch).
template <typename T, int NB>
__device__ __forceinline__ void stage_vt(const T *V, long ld, int S, T *vt, int tid) {
    constexpr int SP = NB * 32 + 4;
    constexpr int ITER = NB * 32 * (ATT_D / 8) / 256;   // NB
    constexpr int BATCH = ITER % 8 == 0 ? 8 : ITER % 4 == 0 ? 4 : ITER;
    const u32x4 zero4 = {0, 0, 0, 0};
#pragma unroll
    for (int b0 = 0; b0 < ITER; b0 += BATCH) {
        u32x4 raw[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int idx = tid + (b0 + b) * 256;
            const int key = idx % (NB * 32), dc = idx / (NB * 32);
            raw[b] = key < S ? *(const u32x4 *)(V + (long)key * ld + dc * 8) : zero4;
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int idx = tid + (b0 + b) * 256;
            const int key = idx % (NB * 32), dc = idx / (NB * 32);
            const unsigned short *e = (const unsigned short *)&raw[b];
#pragma unroll
            for (int j = 0; j < 8; ++j) ((unsigned short *)vt)[(dc * 8 + j) * SP + key] = e[j];
        }
    }
}

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

    // ---- V^T into LDS (keys past the sequence zero-filled: their probability is 0, but 0 * garbage
    // could be NaN) ---------------------------------------------------------------------------
    __syncthreads();  // the previous tile of this workgroup may still be reading vt
    stage_vt<T, NB>(V, p.ld_qkv, S, vt, tid);
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

// ---- the stand-alone kernel: 64 queries per tile, the keys split between two wavefronts -----------
// A (batch, head) pair has too few 128-query tiles to fill the GPU and a wavefront too long a chain
// of work (12 heads x 1 tile at 128 keys, x 3 at 384).  Here a tile is 64 queries; waves 0 and
// 1 take the first half of the key blocks for query rows 0-31 and 32-63, waves 2 and 3 the second
// half.  Each wave runs the same S^T / softmax / P V sequence on its keys with its own running
// maximum (probabilities left unnormalised), the second pair parks its partial result in LDS and
// the first pair merges: O = (a1 O1 + a2 O2) / (a1 sum1 + a2 sum2), a_i = exp(m_i - max(m1, m2)).
constexpr int ATT_QB_SPLIT = 64;
__host__ __device__ inline size_t attention_vt_bytes(int nb) { return (attention_lds_bytes(nb) + 15) / 16 * 16; }
__host__ __device__ inline size_t attention_split_lds_bytes(int nb) { return attention_vt_bytes(nb) + 2 * (32 * ATT_D + 64) * sizeof(float); }

template <typename T, int NB>
__device__ __forceinline__ void attention_tile_split(const AttnArgs &a, TileIdx t, T *vt) {
    static_assert(NB % 2 == 0, "key blocks are halved");
    constexpr int NBH = NB / 2;
    const gp_attention_params &p = a.p;
    constexpr int SP = NB * 32 + 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const int qg = wave & 1, kh = wave >> 1;  // query group, key half (wave-uniform)
    const int S = p.seq;
    const int head = t.y % p.heads, bat = t.y / p.heads;
    const long tok0 = (long)bat * S;
    const T *Q = (const T *)p.q + tok0 * p.ld_qkv + (long)head * ATT_D;
    const T *K = (const T *)p.k + tok0 * p.ld_qkv + (long)head * ATT_D;
    const T *V = (const T *)p.v + tok0 * p.ld_qkv + (long)head * ATT_D;
    T *O = (T *)p.out + tok0 * p.ld_out + (long)head * ATT_D;
    const u32x4 zero4 = {0, 0, 0, 0};
    float *merge = (float *)((char *)vt + attention_vt_bytes(NB)) + qg * (32 * ATT_D + 64);  // O2[32][64], m2[32], sum2[32]

    const int q = t.x * ATT_QB_SPLIT + qg * 32 + l32;
    u32x4 bq[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bq[ks] = q < S ? *(const u32x4 *)(Q + (long)q * p.ld_qkv + ks * 16 + half * 8) : zero4;

    __syncthreads();  // the previous tile of this workgroup may still be reading vt or the merge area
    stage_vt<T, NB>(V, p.ld_qkv, S, vt, tid);
    __syncthreads();

    const int nb0 = kh * NBH;
    f32x16 s[NBH];
#pragma unroll
    for (int i = 0; i < NBH; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[i][v] = 0.f;
        const int key = (nb0 + i) * 32 + l32;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const u32x4 a_k = key < S ? *(const u32x4 *)(K + (long)key * p.ld_qkv + ks * 16 + half * 8) : zero4;
            Elem<T>::mma(a_k, bq[ks], s[i]);
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NBH; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = (nb0 + i) * 32 + 8 * (v / 4) + 4 * half + (v % 4);
            s[i][v] = key < S ? s[i][v] * p.scale : -INFINITY;
            m = fmaxf(m, s[i][v]);
        }
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    const float mm = m == -INFINITY ? 0.f : m;  // a half with no valid key contributes nothing (and no NaN)
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NBH; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            s[i][v] = __expf(s[i][v] - mm);
            sum += s[i][v];
        }
    sum += __shfl_xor(sum, 32, 64);

    f32x16 o[2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
#pragma unroll
    for (int i = 0; i < NBH; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            typedef T tx8 __attribute__((ext_vector_type(8)));
            tx8 pa;
#pragma unroll
            for (int e = 0; e < 8; ++e) pa[e] = Elem<T>::from_f(s[i][8 * j + e]);
            const int kbase = (nb0 + i) * 32 + 16 * j + 4 * half;
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                const unsigned short *row = (const unsigned short *)vt + (db * 32 + l32) * SP + kbase;
                const unsigned long long lo = *(const unsigned long long *)row, hi = *(const unsigned long long *)(row + 8);
                u32x4 bv = {(unsigned)lo, (unsigned)(lo >> 32), (unsigned)hi, (unsigned)(hi >> 32)};
                Elem<T>::mma(__builtin_bit_cast(u32x4, pa), bv, o[db]);
            }
        }
    // ---- merge the two key halves ------------------------------------------------------------------
    if (kh == 1) {
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) merge[(8 * (v / 4) + 4 * half + (v % 4)) * ATT_D + db * 32 + l32] = o[db][v];
        if (half == 0) {
            merge[32 * ATT_D + l32] = m;
            merge[32 * ATT_D + 32 + l32] = sum;
        }
    }
    __syncthreads();
    if (kh == 0) {
        const float m2 = merge[32 * ATT_D + l32], sum2 = merge[32 * ATT_D + 32 + l32];
        const float M = fmaxf(mm, m2);
        const float a1 = __expf(mm - M), a2 = m2 == -INFINITY ? 0.f : __expf(m2 - M);
        const float den = a1 * sum + a2 * sum2;
        const float f1 = a1 / den, f2 = a2 / den;  // this lane's query (row l32 of the group)
        const int q0 = t.x * ATT_QB_SPLIT + qg * 32;
        // The accumulator registers of a lane belong to four runs of four consecutive query rows, whose
        // factors sit in other lanes: they go through LDS (the slots of m2 and sum2, read above) and
        // come back as 16-byte reads, one per run.  The wavefront is alone in this part of LDS, and its
        // LDS operations complete in order.
        float *fac = merge + 32 * ATT_D;
        if (half == 0) {
            fac[l32] = f1;
            fac[32 + l32] = f2;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
            const f32x4 g1 = *(const f32x4 *)(fac + 8 * vq + 4 * half), g2 = *(const f32x4 *)(fac + 32 + 8 * vq + 4 * half);
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int v = 4 * vq + e, r = 8 * vq + 4 * half + e;
                    o[db][v] = g1[e] * o[db][v] + g2[e] * merge[r * ATT_D + db * 32 + l32];
                }
        }
        // The 32 x 64 block of results is laid out in LDS (over the partial block, which has been read)
        // and leaves as 16-byte stores, four per lane, instead of sixty-four 2-byte ones.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        T *ob = (T *)merge;
        const bool vec_out = p.ld_out % 8 == 0 && (size_t)p.out % 16 == 0;  // rows of 64 values start on 16-byte boundaries
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) ob[(8 * (v / 4) + 4 * half + (v % 4)) * ATT_D + db * 32 + l32] = Elem<T>::from_f(o[db][v]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int c0 = 0; c0 < 32 * ATT_D / 8; c0 += 64) {
            const int c = c0 + lane, r = c >> 3, d8 = (c & 7) * 8;
            const u32x4 chunk = *(const u32x4 *)(ob + r * ATT_D + d8);
            if (q0 + r >= S) continue;
            T *dst = O + (long)(q0 + r) * p.ld_out + d8;
            if (vec_out) st_out128(dst, __builtin_bit_cast(out_u32x4, chunk));
            else {
                const T *e = (const T *)&chunk;
#pragma unroll
                for (int j = 0; j < 8; ++j) st_elem<T>(dst + j, e[j]);
            }
        }
    }
}

// Key blocks the body is instantiated for: seq <= 128 / 256 / 384 / 512 keys.
__host__ __device__ inline int attention_nb_class(int seq) {
    const int nb = attention_key_blocks(seq);
    return nb <= 4 ? 4 : nb <= 8 ? 8 : nb <= 12 ? 12 : 16;
}

// One kernel per class: the score registers of the longest class (256 per lane) would otherwise set
// the register budget, and the scratch memory, of the short sequences too.
template <typename T, int NB, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(256) void attention_kernel(AttnArgs a, BlpArgs blp) {
    extern __shared__ __attribute__((aligned(16))) unsigned char att_lds[];
    tiles<LOOP>(blp, [&](TileIdx t) {
        if constexpr (NB < 4) attention_tile<T, NB>(a, t, reinterpret_cast<T *>(att_lds));
        else attention_tile_split<T, NB>(a, t, reinterpret_cast<T *>(att_lds));
    });
}
// queries per tile and LDS bytes of the class a sequence length falls into
__host__ __device__ inline int attention_queries_per_tile(int seq) { return attention_nb_class(seq) < 4 ? ATT_QB : ATT_QB_SPLIT; }
__host__ __device__ inline size_t attention_class_lds_bytes(int seq) {
    const int nb = attention_nb_class(seq);
    return nb < 4 ? attention_lds_bytes(nb) : attention_split_lds_bytes(nb);
}

}  // namespace gp
