/*
 * gpreempt_hip.h — C ABI of libgpreempt_hip.so, the MI355X (gfx950) device layer of the
 * preemptible inference executor.
 *
 * This is the drop-in boundary: the C++ host classes (foo::Executor / foo::BLPExecutor /
 * foo::Model, gpreempt.h) reach the GPU only through these entry points.  Each entry point
 * names the interface of the reference (thustorage/GPreempt) that it replaces.
 *
 * Conventions: every function returns 0 on success and a non-zero gp_status otherwise; it never
 * throws and never aborts; gp_last_error() gives the message of the calling thread's last
 * failure.  All pointers are plain device or host addresses; sizes are bytes unless named
 * otherwise.  Callable from any host thread.
 */
#ifndef GPREEMPT_HIP_H
#define GPREEMPT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Mirrors `enum Status` of the reference (include/util/common.h:16-23). */
enum gp_status { GP_SUCC = 0, GP_FAIL = 1, GP_TIMEOUT = 2, GP_NOTFOUND = 3, GP_OUTOFRANGE = 4, GP_FULL = 5 };

enum gp_dtype { GP_F32 = 0, GP_F16 = 1, GP_BF16 = 2, GP_I32 = 3, GP_I64 = 4 };
enum gp_act { GP_ACT_NONE = 0, GP_ACT_RELU = 1, GP_ACT_GELU = 2 };
/* Matrix-kernel variants: register-staged (handles B stored K x N), pipelined direct-to-LDS,
 * pipelined with K split across the four waves of a workgroup, and "wide": 16 (GP_MAT_WIDE) or 8
 * (GP_MAT_WIDE8) waves share one tile and split every K-stage (problems with fewer tiles than the
 * GPU has compute units; tiles 32 x 32, 64 x 32, 64 x 64). */
enum gp_mat_variant { GP_MAT_AUTO = 0, GP_MAT_STAGED = 1, GP_MAT_PIPE = 2, GP_MAT_PIPE_SPLITK = 3, GP_MAT_WIDE = 4, GP_MAT_WIDE8 = 5 };

typedef struct gp_stream_s *gp_stream; /* opaque; wraps one HIP stream */
typedef struct gp_event_s *gp_event;
typedef struct gp_graph_s *gp_graph;

/* ---- device / errors ---------------------------------------------------------------------
 * Replaces foo::util::init_cuda (src/util/gpu_util.cpp:14-25): selects the device for the
 * calling thread.  Safe to call once per thread, as the reference's clients do. */
int gp_init(int device);
const char *gp_last_error(void);
/* Number of compute units, wavefront clock in kHz and the device name (name_len bytes). */
int gp_device_info(int *compute_units, int *clock_khz, char *name, size_t name_len);

/* ---- streams, events ---------------------------------------------------------------------
 * Replaces GPUStreamCreate / GPUStreamSynchronize (include/util/gpu_util.h:74-139).  `priority`
 * is the tenant priority of the reference (0 = high, 1 = low, larger = lower); it is recorded
 * on the handle and selects which preempt flag level the tenant obeys.  The HIP stream itself
 * is always created at the default hardware priority. */
int gp_stream_create(int priority, gp_stream *out);
int gp_stream_destroy(gp_stream s);
int gp_stream_sync(gp_stream s);
int gp_stream_query(gp_stream s, int *idle); /* *idle = 1 when all work has completed */
int gp_stream_priority(gp_stream s, int *priority);
/* Replaces the driver call behind set_priority (src/gpreempt.cpp:61-72: the context's timeslice):
 * re-labels the tenant priority recorded on the handle.  The HIP stream is not touched. */
int gp_stream_set_priority(gp_stream s, int priority);
void *gp_stream_native(gp_stream s); /* the hipStream_t, for callers that own HIP code */

int gp_event_create(gp_event *out);
int gp_event_destroy(gp_event e);
int gp_event_record(gp_event e, gp_stream s);
int gp_event_sync(gp_event e);
int gp_event_query(gp_event e, int *done); /* *done = 1 when the event has completed (hipEventQuery) */
int gp_event_elapsed_ms(gp_event start, gp_event stop, float *ms);

/* ---- memory ------------------------------------------------------------------------------
 * Replaces GPUMemAlloc / GPUMemFree / GPUMemcpy* / GPUMemsetAsync / GPUMemHostAlloc
 * (include/util/gpu_util.h:74-139; uses in src/model.cpp:101-113,268-279,296-327). */
int gp_malloc(void **dev, size_t bytes);
int gp_free(void *dev);
int gp_host_alloc(void **host, size_t bytes); /* pinned */
int gp_host_free(void *host);
int gp_memcpy_h2d(void *dev, const void *host, size_t bytes);
int gp_memcpy_d2h(void *host, const void *dev, size_t bytes);
int gp_memcpy_h2d_async(void *dev, const void *host, size_t bytes, gp_stream s);
int gp_memcpy_d2h_async(void *host, const void *dev, size_t bytes, gp_stream s);
int gp_memcpy_d2d_async(void *dst, const void *src, size_t bytes, gp_stream s);
/* Fills `count` 32-bit words with `value` using a fill kernel (safe inside a captured graph). */
int gp_fill32_async(void *dev, uint32_t value, size_t count, gp_stream s);

/* ---- preempt flag ------------------------------------------------------------------------
 * Replaces the GDRCopy-mapped device int of src/cuda-clients/blpclient.cpp:45-76 and the
 * managed int of src/hip-clients/blpclient.cpp:106: one int in fine-grained, coherent pinned
 * host memory.  The host sets it with a plain store through *host_ptr; kernels poll *dev_ptr
 * with system-scope loads. */
int gp_flag_create(volatile int **host_ptr, void **dev_ptr);
int gp_flag_destroy(volatile int *host_ptr);
/* A one-workgroup kernel on `s` that stores `value` in a gp_flag_create word (word_dev = its dev_ptr): when the host
 * reads the value there, everything submitted to `s` before the call has left the GPU.  What a host that polls for
 * "has my stream drained" (src/cuda-clients/blpclient.cpp:189-195 spins on a counter for the same purpose) uses
 * instead of stream queries, which cost 3-5 us apiece once the stream's last command is a kernel. */
int gp_store_word_async(gp_stream s, int *word_dev, int value);
/* Flag relay: one small resident kernel copies n host flag words (device-visible addresses of
 * gp_flag_create flags, flags_dev[i]) into device memory (mirror[i]) whenever they change, so
 * that kernels can poll a device address on every claim instead of crossing PCIe; a host store
 * reaches the mirror in a few microseconds.  The kernel leaves when *quit_dev (another
 * gp_flag_create word) becomes non-zero or after spin_limit polls; it occupies one wavefront of
 * stream `s` until then, so stop it (store 1 to the quit flag, then gp_stream_sync(s)) before
 * any call that synchronises the whole device (gp_free, gp_host_free).  n <= 8. */
int gp_flag_relay_start(void *const *flags_dev, int *mirror, int n, const int *quit_dev,
                        unsigned long long spin_limit, gp_stream s);

/* ---- block-level preemption context ------------------------------------------------------
 * The six trailing arguments that scripts/compile/convert_to_blp.py:35 appends to every kernel
 * (`int* preempted, int* pStopIndex, int total_block, int* executed, dim3 shape, int
 * kernel_id`), as one struct.  total_block and shape are derived by the launcher from the
 * operator's own tiling, as src/model.cpp:366-396 derives them from the launch grid.
 * A NULL context launches the same kernel non-preemptibly: one workgroup per tile. */
typedef struct gp_preempt_ctx {
    int *flag;       /* device address of the preempt flag (gp_flag_create's dev_ptr)          */
    int *stop_index; /* device int, -1 when no kernel has been stopped                          */
    int *executed;   /* device int: this kernel's tile claim counter                            */
    int kernel_id;   /* index written to *stop_index by the first workgroup that sees the flag */
    int inject_at;   /* test hook: the workgroup whose claim returns this value raises *flag    */
                     /* itself right after the claim; -1 = off                                  */
    int max_workgroups; /* 0 = occupancy-sized persistent grid; >0 caps it                      */
    int poll_every;  /* the claim numbered c reads the host flag when c % poll_every == 0; a power */
                     /* of two; 0 = default (8).  All claims check *stop_index (device memory),   */
                     /* which the polling workgroup sets, so 1 reproduces a poll per tile.  A      */
                     /* launch with fixed claims (gp_launch_info) and poll_every != 1 instead gets */
                     /* four workgroups more that own no claim and read the flag at launch         */
    int counter_groups; /* 0 or 1: *executed is one int (the reference's layout).  A power of two */
                     /* n > 1: executed points at n counters spaced 16 ints (64 bytes) apart;     */
                     /* every counter owns a contiguous slice of the tiles and is served by the    */
                     /* workgroups of one XCD (workgroup w runs on XCD w % 8; counter              */
                     /* (w % 8) * (n / 8) + (w / 8) % (n / 8) for n >= 8, see util/slice_map.h).   */
                     /* Spreads the claim atomics, which serialise on one address.                 */
    int fresh;       /* nonzero: the caller vouches that this kernel has not been launched since its    */
                     /* counters were last cleared.  With counter_groups > 1 a launch of at least as   */
                     /* many workgroups as claims then records its claims (a bit per workgroup in      */
                     /* ints 1..15 of each counter's 64 bytes, the count in int 0) without waiting     */
                     /* for the old values; 0 is always safe.  Clear all 16 ints of every counter.     */
                     /* 2: as 1, and the GEMM and convolution bodies start their tile without waiting   */
                     /* for the stop index (they look at it when their first operands have landed):     */
                     /* shorter launches, a longer drain of launches queued behind a stop.  Honoured    */
                     /* for launches whose workgroups all start at once; others behave as with 1.       */
    int *left_host;  /* programs only, may be NULL: device-visible address of a gp_flag_create    */
                     /* word; the last workgroup to leave a launch stores that launch's number    */
                     /* (info->shape[1] of gp_program_launch) there, so the host learns that the  */
                     /* GPU has been vacated without a queue query                                */
    void *ckpt;      /* may be NULL.  Workspace (gp_gemm_ckpt_bytes) that lets a long GEMM tile be   */
                     /* left between two K-steps: the workgroup stores its fp32 accumulators and    */
                     /* K position there and the relaunch (same grid) continues from them, still    */
                     /* bit-identical.  Without it a workgroup finishes the tile it owes.  Clear it */
                     /* with gp_ckpt_reset_async whenever the claim counters are cleared.  No       */
                     /* counterpart in the reference, whose tiles are never long enough to matter.  */
    unsigned long long ckpt_bytes;
    int *done;       /* may be NULL.  Counters laid out like `executed` (counter_groups of them, 16 ints apart,  */
                     /* cleared together with them) in which every worker workgroup of every launch of this     */
                     /* kernel counts itself when it leaves (a K-step earlier when it finishes its tile).  With  */
                     /* them a launch of long tiles (1.8 * 10^7 multiply-adds and more per tile) keeps one       */
                     /* workgroup in front of its workers reading the preempt flag until half of the last round  */
                     /* of them has counted itself, and its tiles look at the stop index every                    */
                     /* few K-stages: a tile that finds a stop recorded is given up (its claim is withdrawn, the */
                     /* relaunch computes it from the start: same bits).  The reference's wrapper can only stop  */
                     /* between tiles (convert_to_blp.py:45-58); a 32 x 32 x 25088 tile of VGG-16's first dense  */
                     /* layer runs 70 us.                                                                        */
    int done_launches; /* launches of this kernel since `done` was cleared                                     */
    unsigned long long *stamps; /* may be NULL (the default).  A measurement mode: GP_STAMP_WORDS 64-bit words of   */
                     /* device memory that the kernels fill with the device's constant-rate clock             */
                     /* (gp_device_clock gives its rate and its offset to the host's monotonic clock):        */
                     /* word 0 when the stop was recorded, word 1 at the first claim made while it was zero,   */
                     /* words 8 + (workgroup mod 1024) whenever a workgroup of a preemptible launch leaves.    */
                     /* What                                                                                  */
                     /* src/cuda-clients/blpclient.cpp:185-195 measures from the host, measured on the GPU.    */
    int *started_host; /* may be NULL: device-visible address of a gp_flag_create word.  The first workgroup of  */
                     /* the launch stores started_seq there when it starts, i.e. when every launch before it  */
                     /* on the stream has left the GPU.  A host that submits a model kernel by kernel          */
                     /* (src/executor.cpp:222-225) reads the word to keep a bounded number of launches queued  */
                     /* without events or queue queries, each of which costs the stream 3.7 us on MI355X.      */
    int started_seq;
} gp_preempt_ctx;
enum { GP_STAMP_STOP = 0, GP_STAMP_FIRST_CLAIM = 1, GP_STAMP_EXIT0 = 8, GP_STAMP_EXIT_SLOTS = 1024, GP_STAMP_WORDS = 8 + 1024 };
/* The device clock the stamps are taken from: *tick_ns = nominal nanoseconds per tick; *offset_ns = what to
 * add to ticks * tick_ns to get the host's CLOCK_MONOTONIC in nanoseconds, as of now (the minimum over
 * `rounds` exchanges of "a kernel stores its clock to host memory, the host notes when it sees it": good to
 * the one-way latency of such a store, 1-2 us); *ticks (may be NULL) = the device clock of that exchange.
 * The two clocks drift apart by tens of microseconds per second: to convert stamps taken over seconds, call
 * this before and after and interpolate between the two (ticks, host time) pairs. */
int gp_device_clock(gp_stream s, int rounds, double *tick_ns, double *offset_ns, unsigned long long *ticks);

/* What a launch did: filled when the `info` argument of a launcher is non-NULL. */
typedef struct gp_launch_info {
    int total_tiles;    /* = total_block of the reference                     */
    int shape[3];       /* = dim3 shape of the reference (tile grid)          */
    int grid;           /* workgroups launched                                */
    int block;          /* threads per workgroup                              */
    int fixed_claims;   /* 1: claims were fixed by workgroup index and recorded as bits (see  */
                        /* gp_preempt_ctx::fresh); 0: handed out through the counters          */
    int front;          /* of `grid`, the workgroups in front of the workers that own no claim: a launch */
                        /* with more claims than the device holds workgroups gets 8, the first of which  */
                        /* reads the preempt flag about every microsecond while claims are still being   */
                        /* made (the reference's wrapper reads it once per claim, convert_to_blp.py:45,   */
                        /* which on this GPU leaves gaps as long as a tile)                               */
} gp_launch_info;

/* ---- operators ---------------------------------------------------------------------------
 * These replace the TVM-generated device kernels that src/executor.cpp:157-162 launches by
 * name (fused_nn_conv2d_add_nn_relu*, fused_nn_dense*, fused_nn_softmax*, pooling, add,
 * layer_norm, erf GELU, take, batch_matmul; names implied by patch/tvm.patch:296-311).
 * Accumulation is fp32 for every dtype. */

/* C[b] = act(alpha * A[b] * op(B[b]) + bias[n] + residual[b]); A is M x K row-major.
 * b_is_nk = 0: B is K x N row-major; 1: B is N x K row-major (dense weights).
 * Batch strides are in elements; batch = 1 ignores them.  bias / residual may be NULL;
 * bias has the dtype of C; residual shares ldc / stride_c. */
typedef struct gp_gemm_params {
    int dtype;
    int M, N, K;
    const void *A; long lda; long stride_a;
    const void *B; long ldb; long stride_b; int b_is_nk;
    void *C; long ldc; long stride_c;
    const void *bias;
    const void *residual;
    float alpha;
    int act;
    int batch;
    /* second-level batch (attention heads): offset = (b / batch_inner) * stride_*_outer +
     * (b % batch_inner) * stride_*; batch_inner = 0 disables it. */
    int batch_inner; long stride_a_outer, stride_b_outer, stride_c_outer;
    int tile_m, tile_n; /* 0 = chosen by the launcher; 256, 128, 64 or 32 (square; 64 x 32 with the wide variants) */
    int variant;        /* enum gp_mat_variant; 0 = chosen by the launcher */
    /* Layer-norm prologue (ln_gamma == NULL: none): C = act(alpha * LN(A) * op(B) + bias + residual), where
     * LN normalises every row of A over its K elements (gamma, beta: K elements of A's dtype; eps), rounds it
     * to A's dtype and also writes it to ln_out (M x K, row stride K).  One launch where the exported graph
     * has two (layer_norm, then dense): at batch 1 a launch costs more than the layer-norm's arithmetic.
     * The result has the bits of gp_launch_layernorm followed by gp_launch_gemm.  Only for shapes that
     * gp_gemm_ln_supported accepts; ln_out must not overlap A, B, C, bias or residual. */
    const void *ln_gamma; const void *ln_beta; void *ln_out; float ln_eps;
} gp_gemm_params;
int gp_launch_gemm(const gp_gemm_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);
/* 1 when a layer-norm launch followed by the GEMM `p` (its ln_* fields are not looked at) can be replaced by
 * one launch with the prologue without changing a bit: 16-bit dtype, batch 1, B stored N x K, lda == K, K a
 * multiple of 64 and at most 832, at most one 32 x 64 tile per compute unit (every workgroup of a tile row
 * normalises the rows again, which must stay cheaper than a launch), and a plain GEMM of this shape would be summed in the prologue body's order
 * (K split over four wavefronts).  gp_launch_gemm itself takes the prologue for any shape that passes the
 * first five conditions. */
int gp_gemm_ln_supported(const gp_gemm_params *p);
/* No counterpart in the reference: gp_launch_gemm for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The
 * preemption state that gp_preempt_ctx otherwise brings in (32 claim counters per kernel, the stop
 * index) lives in a device array inside the library: 64 kernel slots, 131 136 bytes per GPU, held
 * until the process ends.  This call allocates and frees nothing.
 *   flag            device-visible address of the preempt flag (gp_flag_create), may be NULL
 *   slot            0..63: which kernel's counters to use; also the kernel id written to the stop index
 *   mode            GP_NOALLOC_CLEAR: zero the slot's counters first (a fresh run of this kernel);
 *                   GP_NOALLOC_REARM: set the stop index to -1 first (the first kernel of a submission
 *                   or of a resume); 0 continues from the counters as they are (BLPExecutor::resume)
 *   inject_at       test hook as gp_preempt_ctx::inject_at; -1 = off
 *   stop_index_out  may be NULL: device-visible int that receives the stop index after the launch
 * Every call on a GPU shares that GPU's array, which keeps the last call's contents: calls that
 * overlap on one GPU (two streams, two threads) race.  Long tiles are finished, not left half-way
 * (there is no checkpoint workspace).  Slots beyond 63 and GEMMs of more than 2^24 tiles are refused. */
enum { GP_NOALLOC_CLEAR = 1, GP_NOALLOC_REARM = 2 };
int gp_launch_gemm_noalloc(const gp_gemm_params *p, int *flag, int slot, int mode, int inject_at, int *stop_index_out,
                           gp_stream s, gp_launch_info *info);
/* Bytes of gp_preempt_ctx::ckpt workspace this GEMM can use (0: it runs on a body whose tiles are
 * short and always finished), and the reset of such a workspace.  Extension of the dispatcher that
 * scripts/compile/convert_to_blp.py:40-69 generates (which can only stop between tiles). */
int gp_gemm_ckpt_bytes(const gp_gemm_params *p, size_t *bytes);
int gp_ckpt_reset_async(void *ckpt, gp_stream s);

/* Implicit-GEMM convolution.  Activations are NHWC with a pixel stride (in elements) that may
 * exceed the channel count, so a layer can read or write a channel slice of a wider buffer
 * (DenseNet concatenation without a copy).  Weights are [Cout][R][S][Cin] ("OHWI").
 * Requires Cin % 4 == 0 (fp32) or Cin % 8 == 0 (fp16 / bf16).
 * out[n,ho,wo,co] = act(sum in[n,ho*sh-ph+r,wo*sw-pw+s,ci] * w[co,r,s,ci] + bias[co] + residual). */
typedef struct gp_conv_params {
    int dtype;
    int N, H, W, Cin, Cout, R, S, stride_h, stride_w, pad_h, pad_w;
    const void *in; long in_pix_stride;
    const void *weight;
    const void *bias;
    const void *residual; long res_pix_stride;
    void *out; long out_pix_stride;
    int act;
    int tile_m, tile_n;
    int variant;
} gp_conv_params;
int gp_launch_conv2d(const gp_conv_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);
/* As gp_gemm_ckpt_bytes, for a convolution (0 unless it runs on the 128 x 128 body). */
int gp_conv_ckpt_bytes(const gp_conv_params *p, size_t *bytes);

/* NCHW -> NHWC with zero padding of the channel count up to c_pad (input adapter: the
 * reference's "data" tensor is NCHW, src/tests/test-dnn.cpp:25-30). */
typedef struct gp_layout_params {
    int dtype_in, dtype_out;
    int N, C, H, W, c_pad;
    const void *in; void *out;
} gp_layout_params;
int gp_launch_nchw_to_nhwc(const gp_layout_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* Pooling on NHWC.  mode 0 = max, 1 = average (padding excluded from the count),
 * 2 = global average (R,S,stride,pad ignored; output N x 1 x 1 x C), 3 = average with the
 * padding counted as zeros (divisor R*S; relay's count_include_pad, used by Inception-v3). */
typedef struct gp_pool_params {
    int dtype;
    int N, H, W, C, R, S, stride, pad, mode;
    const void *in; long in_pix_stride;
    void *out; long out_pix_stride;
} gp_pool_params;
int gp_launch_pool2d(const gp_pool_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* Elementwise over `rows` pixels of `cols` channels:
 *   out = act((a [+ b]) * scale[c] + shift[c]); b, scale, shift may be NULL. */
typedef struct gp_eltwise_params {
    int dtype;
    long rows; int cols;
    const void *a; long a_stride;
    const void *b; long b_stride;
    const void *scale; const void *shift; /* per channel, dtype of a */
    void *out; long out_stride;
    int act;
} gp_eltwise_params;
int gp_launch_eltwise(const gp_eltwise_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* Row softmax over the last axis: out = softmax(scale * x). */
typedef struct gp_softmax_params {
    int dtype;
    long rows; int cols;
    const void *x; void *out;
    float scale;
} gp_softmax_params;
int gp_launch_softmax(const gp_softmax_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* out = layer_norm(x [+ residual]) * gamma + beta over the last axis (biased variance). */
typedef struct gp_layernorm_params {
    int dtype;
    long rows; int cols;
    const void *x; const void *residual;
    const void *gamma; const void *beta;
    void *out;
    float eps;
} gp_layernorm_params;
int gp_launch_layernorm(const gp_layernorm_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* Fused scaled-dot-product attention over the heads of packed Q / K / V activations: for every
 * batch b and head h, out[b*seq + i, h*64 .. h*64+63] = sum_j softmax_j(scale * <Q_i, K_j>) V_j,
 * where row t of Q (K, V) for head h is q (k, v) + t*ld_qkv + h*64.  Replaces the batch_matmul,
 * softmax, batch_matmul sequence of the exported BERT graph (scripts/compile/compile-bert.py:76-77)
 * and the two seq x seq tensors between them; the softmax runs in fp32 on unrounded scores.
 * fp16 / bf16 only, head_dim = 64, seq <= 512, 16-byte aligned rows. */
typedef struct gp_attention_params {
    int dtype;
    int batch, heads, seq, head_dim;
    const void *q; const void *k; const void *v; long ld_qkv;
    void *out; long ld_out;
    float scale;
} gp_attention_params;
int gp_launch_attention(const gp_attention_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* One kernel of the miniWeather workload (2-D stratified compressible flow; the reference's non-DNN
 * preemptible workload).  Replaces the six kernels of src/workloads/miniweather.tr.cu:
 * set_halo_values_x :504-520, compute_tendencies_x :283-349, compute_tendencies_x_r :351-393,
 * set_halo_values_z :523-552, compute_tendencies_z :399-468, compute_tendencies_z_r :470-502.
 * A tile is 256 consecutive element ids, as a thread block of the reference.
 *   state      forcing state, 4 x (nz+4) x (nx+4) fp32 (halo kernels write its halo cells)
 *   flux       4 x (nz+1) x (nx+1) fp32
 *   state_init / state_out   update kernels: out = init + dt * tendency(flux[, state])
 *   hydro      hydrostatic background in one buffer: cell density, cell density*theta (nz+4 each),
 *              interface density, density*theta, pressure (nz+1 each), 4 boundary density ratios
 * dt is the stage's step (dt/3, dt/2, dt of the Runge-Kutta stages). */
enum gp_mw_kernel { GP_MW_HALO_X = 0, GP_MW_FLUX_X = 1, GP_MW_UPDATE_X = 2, GP_MW_HALO_Z = 3, GP_MW_FLUX_Z = 4, GP_MW_UPDATE_Z = 5 };
typedef struct gp_miniweather_params {
    int kernel;
    int nx, nz;
    float dt, dx, dz;
    float *state; float *flux;
    const float *state_init; float *state_out;
    const float *hydro;
} gp_miniweather_params;
int gp_launch_miniweather(const gp_miniweather_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* One kernel of the graph workloads over a CSR graph (vertex_list: vertex_count+1 offsets,
 * edge_list: neighbour ids, both 64-bit as in the reference's files; weight_list: 32-bit edge
 * weights for SSSP).  Replaces the kernels of src/workloads/graphcompute.tr.cu: cc_kernel_coalesce
 * :59-127, bfs_kernel_coalesce :190-241, pr_initialize :298-335, pr_kernel_coalesce :338-384,
 * pr_update :386-425, sssp_kernel_coalesce :511-561, sssp_update :564-603.
 *   BFS_STEP     vertices with label == level give label level+1 to unlabelled (0xFFFFFFFF) neighbours
 *   CC_STEP      active vertices exchange component labels with their neighbours (smaller wins);
 *                the end that changed is marked in next_active
 *   CC_INIT      comp = own vertex id, active = 1, next_active = 0
 *   PR_INIT      value = 1-alpha, delta = (1-alpha)*alpha/degree, residual = 0, active = 1
 *   PR_PUSH      active vertices add delta to the residual of every neighbour, then go inactive
 *   PR_UPDATE    residual > tolerance: value += residual, delta = residual*alpha/degree, residual = 0, active
 *   SSSP_RELAX   active vertices offer new_cost[v] + weight to every neighbour (atomic min), then go inactive
 *   SSSP_UPDATE  new_cost < cost: cost = new_cost, active
 * *changed is set to 1 by any kernel that changed something (the host clears it). */
enum gp_graph_kernel { GP_GRAPH_BFS_STEP = 0, GP_GRAPH_CC_STEP = 1, GP_GRAPH_PR_INIT = 2, GP_GRAPH_PR_PUSH = 3,
                       GP_GRAPH_PR_UPDATE = 4, GP_GRAPH_SSSP_RELAX = 5, GP_GRAPH_SSSP_UPDATE = 6, GP_GRAPH_CC_INIT = 7 };
typedef struct gp_graph_params {
    int kernel;
    unsigned int level;                      /* BFS */
    unsigned long long vertex_count;
    const unsigned long long *vertex_list;
    const unsigned long long *edge_list;
    const unsigned int *weight_list;         /* SSSP */
    unsigned int *label;                     /* BFS: level per vertex */
    unsigned char *active, *next_active;     /* CC: current / next frontier; PageRank, SSSP: active */
    unsigned long long *comp;                /* CC: component label per vertex */
    float *delta, *residual, *value;         /* PageRank */
    float alpha, tolerance;
    unsigned int *cost, *new_cost;           /* SSSP */
    unsigned int *changed;
    int lanes_per_vertex;                    /* edge-parallel kernels: 16, 32 or 64 lanes walk one neighbour list (0 = 64); pick ~ the average degree */
} gp_graph_params;
int gp_launch_graph(const gp_graph_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* out[t,:] = tok[ids[t],:] + pos[t % seq,:] (+ seg[0,:]); ids are int64 (the reference feeds
 * BERT int64 token ids, src/tests/test-dnn.cpp:21-23). */
typedef struct gp_embed_params {
    int dtype;
    long tokens; int seq; int hidden; long vocab;
    const int64_t *ids;
    const void *tok; const void *pos; const void *seg;
    void *out;
} gp_embed_params;
int gp_launch_embed(const gp_embed_params *p, const gp_preempt_ctx *ctx, gp_stream s, gp_launch_info *info);

/* ---- whole-model program -------------------------------------------------------------------
 * The launch-bound inner loop of the reference (one GPULaunchKernel or graph node per kernel,
 * src/executor.cpp:119-134,176-196) as ONE persistent kernel: layers are added in execution
 * order with the same parameter blocks as the stand-alone launchers, each layer depends on the
 * one before it, and the resident workgroups walk the list claiming tiles.  Preemption and
 * resume work at tile granularity exactly as for single kernels; because nothing is queued
 * behind the running kernel, a preempted model leaves the GPU within about one tile.
 *   ctx->flag / ctx->stop_index  as for the launchers (stop_index receives the LAYER index)
 *   ctx->executed                ignored: the program owns one counter per layer
 *   ctx->kernel_id, inject_at    test hook: layer and claim number that raise the flag
 * info->shape[1] receives the launch number that ctx->left_host will be set to.
 * reset != 0 starts the model from its first tile (BLPExecutor::execute); reset == 0 continues
 * from the counters left by a preempted run (BLPExecutor::resume).  A NULL ctx runs the model
 * non-preemptibly (BaseExecutor). */
typedef struct gp_program_s *gp_program;
int gp_program_create(int dtype, gp_program *out);
int gp_program_destroy(gp_program p);
int gp_program_add_gemm(gp_program p, const gp_gemm_params *params);
int gp_program_add_conv2d(gp_program p, const gp_conv_params *params);
int gp_program_add_nchw_to_nhwc(gp_program p, const gp_layout_params *params);
int gp_program_add_pool2d(gp_program p, const gp_pool_params *params);
int gp_program_add_eltwise(gp_program p, const gp_eltwise_params *params);
int gp_program_add_softmax(gp_program p, const gp_softmax_params *params);
int gp_program_add_layernorm(gp_program p, const gp_layernorm_params *params);
int gp_program_add_attention(gp_program pr, const gp_attention_params *p);
int gp_program_add_embed(gp_program p, const gp_embed_params *params);
int gp_program_add_copy(gp_program p, const void *src, void *dst, size_t bytes); /* the reference's "nop" copy */
int gp_program_finalize(gp_program p);
int gp_program_launch(gp_program p, const gp_preempt_ctx *ctx, int reset, gp_stream s, gp_launch_info *info);
int gp_program_layers(gp_program p, int *n_layers);
/* Blocking read-back of per-layer claim / completion counters, the number of tiles handed out
 * so far over all layers (*cursor) and the error word (1 = a dependency wait gave up); any
 * pointer may be NULL. */
int gp_program_read_state(gp_program p, int *executed, int *done, int *cursor, int *error);

/* ---- gate kernels --------------------------------------------------------------------------
 * Replace gpu_block / gpu_noop (src/block.cu:1-7): one wave spins until *stop != 0.  Unlike the
 * reference the wait is bounded: after spin_limit polls the kernel leaves and stores 1 to
 * *timed_out (may be NULL), so a lost release can never hang the device. */
int gp_launch_gate(const int *stop, unsigned long long spin_limit, int *timed_out, gp_stream s);
int gp_launch_noop(gp_stream s);

/* ---- graphs --------------------------------------------------------------------------------
 * Replace GPUStreamBeginCapture / EndCapture / GraphInstantiate / GraphLaunch
 * (src/executor.cpp:119-122,176-196). */
int gp_graph_begin(gp_stream s);
int gp_graph_end(gp_stream s, gp_graph *out);
int gp_graph_launch(gp_graph g, gp_stream s);
int gp_graph_destroy(gp_graph g);

#ifdef __cplusplus
}
#endif
#endif /* GPREEMPT_HIP_H */
