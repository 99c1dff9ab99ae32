/*
 * ronn_bitnet_hip.h - C ABI of the MI355X (gfx950) BitNet ternary hot path.
 *
 * This is the boundary a host-language binding (the Rust `ronn-providers` crate
 * through an `extern "C"` block, or ctypes, or C++) calls.  Plain pointers and
 * sizes only.  Citations name the reference code each entry point stands in for,
 * relative to the reference checkout's crates/ronn-providers/src/bitnet/.
 *
 * Conventions
 *   - Every function returns RBN_OK (0) or a negative rbn_status.  Nothing throws
 *     or aborts across this boundary.  rbn_last_error() returns the message of the
 *     calling thread's most recent failure.
 *   - Pointers named d_* are device pointers (from rbn_malloc, or any hipMalloc'd
 *     memory of the same device); h_* are host pointers.  All are caller-owned.
 *   - A context owns one HIP stream of default priority.  Calls on one context are
 *     serialised by an internal lock, so a context may be shared by threads
 *     (the reference's CompiledKernel is Send + Sync, ronn-core types.rs:153).
 *     Compute calls are asynchronous on that stream unless they return a value
 *     through a host pointer; rbn_sync() waits for the stream.
 *   - Matrices are row-major.  A is activations [M,K], B is weights [K,N], the
 *     result is [M,N] (kernels.rs:134-178).
 *
 * Weight formats
 *   "packed"  The reference's TernaryTensor.packed_data (quantization.rs:131-153,
 *             249-260): element i of the flattened tensor is the 2-bit field at bit
 *             2*(i%4) of byte i/4; 00 = -1, 01 = 0, 10 = +1, 11 never produced and
 *             read as 0 (quantization.rs:285-290).  ceil(n/4) bytes; device buffers
 *             must have rbn_packed_capacity(n) bytes.
 *   "tiled"   Device-internal layout the matmul kernels stream.  Columns are grouped
 *             in quads of four, k in blocks of sixteen.  The 16 bytes at uint4 index
 *             q * KB + kb (KB = Kpad/16) are four u32 words, word c for column 4q+c;
 *             a word holds the 16 weights k = 16*kb + 4*s + b of its column as the
 *             2-bit field at bit 8*b + 2*s (so (word >> 2*s) & 0x03030303 is four
 *             int8-ready codes of four consecutive k).  A quad's weights are thus
 *             contiguous along k.  Code = value + 1 (same as "packed"); 11 and padding
 *             are stored as 01 (zero).  Kpad = K rounded up to 128, Npad = N rounded up
 *             to 64.  Built from "packed" by rbn_tile_weights().
 */
#ifndef RONN_BITNET_HIP_H
#define RONN_BITNET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rbn_ctx rbn_ctx;

typedef enum rbn_status {
    RBN_OK = 0,
    RBN_ERR_INVALID = -1,     /* bad argument (null pointer, zero/odd dimension, ...) */
    RBN_ERR_HIP = -2,         /* a HIP runtime call failed; message has the HIP error */
    RBN_ERR_OOM = -3,         /* device allocation failed */
    RBN_ERR_UNSUPPORTED = -4, /* shape or mode outside what the kernels cover */
    RBN_ERR_NO_DEVICE = -5    /* no gfx950 device visible / wrong architecture */
} rbn_status;

/* How the order-sensitive f32 sums of quantize_ternary are evaluated. */
typedef enum rbn_sum_mode {
    /* Bit-exact emulation of the reference's sequential f32 left fold
     * (`iter().sum::<f32>()`, quantization.rs:79 and :96). */
    RBN_SUM_STRICT_SEQ = 0,
    /* Deterministic f64 tree reduction: faster and more accurate, NOT
     * reference-exact on large tensors (threshold and scale differ). */
    RBN_SUM_TREE = 1
} rbn_sum_mode;

typedef struct rbn_device_info {
    char name[128];
    char arch[64];
    int compute_units;
    int clock_khz;          /* max engine clock */
    int mem_clock_khz;
    int mem_bus_bits;
    uint64_t hbm_bytes;
    uint64_t l2_bytes;
} rbn_device_info;

/* ---- library / context --------------------------------------------------- */
const char *rbn_version(void);
/* Message of the calling thread's last failed call ("" if none). */
const char *rbn_last_error(void);
/* Number of HIP devices visible (0 if none or HIP cannot initialise). */
int rbn_device_count(void);
/* Creates a context on `device`.  Replaces BitNetExecutionProvider::with_config's
 * resource set-up (provider.rs:77-114). */
int rbn_ctx_create(int device, rbn_ctx **out);
int rbn_ctx_destroy(rbn_ctx *ctx);
int rbn_get_device_info(rbn_ctx *ctx, rbn_device_info *out);

/* ---- device buffers (replaces BitNetMemoryAllocator::allocate/deallocate,
 *      allocator.rs:99-140, with device memory instead of SystemRAM) ------- */
int rbn_malloc(rbn_ctx *ctx, size_t bytes, void **d_out);
int rbn_free(rbn_ctx *ctx, void *d_ptr);
int rbn_h2d(rbn_ctx *ctx, void *d_dst, const void *h_src, size_t bytes);
int rbn_d2h(rbn_ctx *ctx, void *h_dst, const void *d_src, size_t bytes);
int rbn_d2d(rbn_ctx *ctx, void *d_dst, const void *d_src, size_t bytes);
int rbn_fill_u8(rbn_ctx *ctx, void *d_dst, int value, size_t bytes);
int rbn_sync(rbn_ctx *ctx);
/* Conditions that only a kernel can see are reported through one word of flags per
 * context: *h_flags receives the bits raised since the last call and the word is cleared.
 * Synchronises the stream.  No reference counterpart. */
#define RBN_FLAG_HISTORY_OVERFLOW 1u /* rbn_argmax_f32 / rbn_greedy_next_f32: position outside the history */
int rbn_device_flags(rbn_ctx *ctx, uint32_t *h_flags);
/* Bytes currently / at most allocated through rbn_malloc on this context
 * (MemoryInfo, allocator.rs:142-148). */
int rbn_memory_info(rbn_ctx *ctx, uint64_t *allocated, uint64_t *peak);

/* Size rules of the reference allocator (allocator.rs:39-75): bytes for a tensor
 * of `element_count` elements; dtype: 0=F32 1=F16 2=BF16 6=U8 (2-bit ternary)
 * 8=Bool (1-bit).  Returns -1 for other dtypes. */
int64_t rbn_tensor_bytes(uint64_t element_count, int dtype);
size_t rbn_tensor_alignment(int dtype);
/* Device capacity, in bytes, a "packed" buffer of n elements must have
 * (ceil(n/4) rounded up to 16). */
size_t rbn_packed_capacity(uint64_t n);
/* Bytes of the "tiled" layout of a [K,N] weight matrix. */
size_t rbn_tiled_bytes(uint64_t K, uint64_t N);
/* Row pitch, in bytes, of quantised activations for inner dimension K (K rounded up to 128). */
size_t rbn_act_pitch(uint64_t K);

/* ---- timing on the context's stream -------------------------------------- */
/* Records a start event on the stream.  rbn_timer_stop records the stop event,
 * waits for it and returns the elapsed milliseconds between the two. */
int rbn_timer_start(rbn_ctx *ctx);
int rbn_timer_stop(rbn_ctx *ctx, float *h_ms);

/* ---- HIP graphs ----------------------------------------------------------- */
/* Launch-bound sequences (a decode step is tens of kernels of a few microseconds)
 * are captured once and replayed.  Between begin and end every asynchronous compute
 * call on this context (pack, tile, act_quant_i8, gemv, gemm, matmul, d2d, fill) is
 * recorded instead of run; calls that return scalars to the host or allocate are not
 * allowed while capturing.  No reference counterpart. */
typedef struct rbn_graph rbn_graph;
int rbn_graph_begin_capture(rbn_ctx *ctx);
int rbn_graph_end_capture(rbn_ctx *ctx, rbn_graph **out);
int rbn_graph_launch(rbn_ctx *ctx, rbn_graph *graph);
int rbn_graph_destroy(rbn_ctx *ctx, rbn_graph *graph);

/* ---- (1) ternarize + pack: BitNetQuantizer::quantize_ternary,
 *      quantization.rs:67-109, and pack_ternary_bits, :131-153 -------------- */
/* sum_i |x_i| in f32, as the reference's fold evaluates it (mode STRICT_SEQ) or
 * as an f64 tree rounded once to f32 (mode TREE).  With use_mask != 0 only
 * elements with |x_i| > mask_threshold are summed (the survivors of
 * quantization.rs:82-91) and *h_count receives how many there were; otherwise
 * *h_count = n.  h_count may be NULL. */
int rbn_abs_sum_f32(rbn_ctx *ctx, const float *d_x, uint64_t n, int mode, int use_mask,
                    float mask_threshold, float *h_sum, uint64_t *h_count);
/* pack_ternary_bits for a given threshold: writes the "packed" format. */
int rbn_pack_ternary(rbn_ctx *ctx, const float *d_x, uint64_t n, float threshold,
                     uint8_t *d_packed);
/* The whole of quantize_ternary: threshold (quantization.rs:79), scale (:82-97),
 * pack (:100).  Synchronous (returns scalars).  h_survivors may be NULL. */
int rbn_quantize_ternary(rbn_ctx *ctx, const float *d_x, uint64_t n, int mode,
                         uint8_t *d_packed, float *h_scale, float *h_threshold,
                         uint64_t *h_survivors);
/* dequantize_ternary, quantization.rs:182-207: code -> {-scale, 0, +scale}. */
int rbn_dequantize_ternary(rbn_ctx *ctx, const uint8_t *d_packed, uint64_t n, float scale,
                           float *d_out);
/* TernaryTensor::get_value for every element (quantization.rs:275-291): int8 in
 * {-1,0,+1}.  With rows/cols/pitch it writes a [rows, pitch] matrix whose columns
 * >= cols are zero (pitch = rbn_act_pitch(cols) gives the activation format the
 * matmuls take); rows*cols = element count.  d_rowsum (optional) gets the int32 sum
 * of each row. */
int rbn_unpack_ternary_i8(rbn_ctx *ctx, const uint8_t *d_packed, uint64_t rows, uint64_t cols,
                          uint64_t pitch, int8_t *d_q, int32_t *d_rowsum);
/* "packed" [K,N] -> "tiled" (device-internal).  No reference counterpart: the
 * reference multiplies straight out of packed_data with get_value. */
int rbn_tile_weights(rbn_ctx *ctx, const uint8_t *d_packed, uint64_t K, uint64_t N,
                     uint32_t *d_tiled);

/* ---- (2) activation quantisation ------------------------------------------ */
/* Per-token absmax int8 (build-defined, no reference counterpart; the reference
 * ternarises activations, kernels.rs:277):
 *   g = max(max_k |x[m,k]|, 1e-5f); q = clamp(rne(x * (127/g)), -128, 127);
 *   act_scale[m] = g / 127; rowsum[m] = sum_k q.
 * d_q is [M, rbn_act_pitch(K)] int8 with zero padding. */
int rbn_act_quant_i8(rbn_ctx *ctx, const float *d_x, uint64_t M, uint64_t K, int8_t *d_q,
                     float *d_act_scale, int32_t *d_rowsum);
/* Reference-mode activations: quantize_ternary over the whole [M,K] tensor
 * (kernels.rs:277), expanded to int8 {-1,0,+1} in the same [M, pitch] format;
 * act_scale[m] = the tensor's scale for every m.  Synchronous. */
int rbn_act_quant_ternary(rbn_ctx *ctx, const float *d_x, uint64_t M, uint64_t K, int mode,
                          int8_t *d_q, float *d_act_scale, int32_t *d_rowsum, float *h_scale,
                          float *h_threshold);

/* ---- (3)(4)(5) ternary matmul: BitNetKernel::execute_ternary_matmul,
 *      kernels.rs:134-178, with the fused epilogue of :168 ------------------ */
/* out[m,n] = ((float)acc[m,n] * act_scale[m]) * w_scale, acc = sum_k q[m,k]*w[k,n]
 * in int32.  d_acc may be NULL; when given it receives the int32 accumulators.
 * rbn_gemv_t2_i8: decode regime (M <= RBN_GEMV_MAX_M), streams the tiled weights
 * once with int8 dot instructions.  rbn_gemm_t2_i8_skinny: small batches
 * (M <= RBN_SKINNY_MAX_M), the same streaming read with 16x16x64 int8 MFMA doing
 * the dot products.  rbn_gemm_t2_i8_mfma: prefill regime, 128x256 tiles of int8
 * MFMA.  rbn_matmul_t2_i8 picks one by M, K and N (gemv for 1 and 2 tokens - not for 2 when
 * K <= 3072 and K*N >= 2^25 - and up to 4 when K*N <= 2^24; skinny up to 16 tokens, up to 32
 * when K*N < 2^27, up to 64 when K*N < 2^25; mfma otherwise).
 * All three give identical results.
 * d_q and d_tiled must be 16-byte aligned; so must d_out and d_acc for every entry point
 * except rbn_gemv_t2_i8, which accepts any float/int32 alignment there (memory from
 * rbn_malloc is 256-byte aligned).  A misaligned pointer is RBN_ERR_INVALID. */
#define RBN_GEMV_MAX_M 16
#define RBN_SKINNY_MAX_M 64
int rbn_gemv_t2_i8(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                   const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale, uint64_t M,
                   uint64_t K, uint64_t N, int32_t *d_acc, float *d_out);
/* rbn_gemv_t2_i8, launched so that the kernel's own begin and end timestamps are recorded:
 * *h_kernel_us receives the duration of this one dispatch (what a profiler's kernel trace
 * reports).  Synchronises the stream and uses the context's timer events, so it must not sit
 * between rbn_timer_start and rbn_timer_stop, nor inside a graph capture.  For measurement;
 * no counterpart in the reference. */
int rbn_gemv_t2_i8_kernel_time(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                               const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                               uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out,
                               float *h_kernel_us);
/* Several independent decode GEMVs of one shape in ONE launch (q/k/v or gate/up projections of
 * a token, the experts or adapters of a layer, the same layer of several sequences).  Every
 * problem is a complete rbn_gemv_t2_i8 with its own activations, weights and outputs, and
 * gives the bits rbn_gemv_t2_i8 gives.  What the grouping buys is time: a single GEMV of a few
 * MB is shorter than the gap between two launches plus the ramp of its first loads, and in one
 * grid the problems overlap.  h_problems is a HOST array of `count` descriptors (1 to
 * RBN_GEMV_GROUP_MAX); the pointers inside are device pointers.  The descriptors are copied
 * into the launch's arguments, so the array may be reused as soon as the call returns and the
 * call can be captured in a graph.  No reference counterpart (the reference multiplies one
 * pair of tensors per execute(), kernels.rs:271-283). */
#define RBN_GEMV_GROUP_MAX 32
typedef struct rbn_gemv_problem {
    const int8_t *d_q;        /* [M, rbn_act_pitch(K)] int8 */
    const float *d_act_scale; /* [M] */
    const int32_t *d_rowsum;  /* [M] */
    const uint32_t *d_tiled;  /* tiled weights [K,N] */
    float *d_out;             /* [M,N] f32 */
    int32_t *d_acc;           /* [M,N] int32 accumulators, or NULL */
    float w_scale;
    uint32_t reserved;        /* set to 0 */
} rbn_gemv_problem;
int rbn_gemv_t2_i8_grouped(rbn_ctx *ctx, const rbn_gemv_problem *h_problems, uint64_t count,
                           uint64_t M, uint64_t K, uint64_t N);
int rbn_gemm_t2_i8_skinny(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                          const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                          uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out);
int rbn_gemm_t2_i8_mfma(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                        const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                        uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out);
/* The launch shape rbn_gemm_t2_i8_skinny picks for a product (needs no device; for tests and
 * tuning): shape[0] = 1 when the operands travel through a ring in LDS (up to 16 tokens), 0 for
 * the register ring; [1] workgroups along N; [2] workgroups that share a column group along
 * k; [3] waves per workgroup; [4] k of one step (64 or 128); [5] steps in all; [6] most steps
 * any wave gets; [7] bytes of dynamic LDS.  Returns RBN_ERR_UNSUPPORTED for a shape the kernels
 * would not be launched with (every wave must own at least one step, at most 16 waves, at most
 * 128 KiB of LDS), RBN_ERR_INVALID for arguments outside the entry point's range. */
int rbn_skinny_launch_shape(uint64_t M, uint64_t K, uint64_t N, int32_t shape[8]);
/* rbn_gemm_t2_i8_skinny for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  Same arguments, same kernels, same bits; the difference is where narrow
 * matrices exchange their split-k partial tiles: in a static device array of the library
 * (RBN_STATIC_SCRATCH_BYTES per GPU, held until the process ends) instead of the workspace a
 * context allocates.  Nothing on this path calls hipMalloc, hipFree or any allocating routine.
 * A shape whose launch would need more than RBN_STATIC_SCRATCH_TILES partial tiles of 16 x 64
 * int32 (ceil(N/64) * splits * ceil(M/16), only when the matrix is narrow enough to be split
 * along k; M <= 16 always fits) is refused with RBN_ERR_UNSUPPORTED and a message that names
 * the need and the limit.  All calls on one GPU share the array: calls that overlap on one GPU
 * would race, so the first context that calls this entry point on a GPU holds the array until
 * that context is destroyed (calls on one context are serialised by its lock and stream) and
 * a call from any other context on that GPU is refused with RBN_ERR_INVALID. */
#define RBN_STATIC_SCRATCH_TILES 1024
#define RBN_STATIC_SCRATCH_BYTES (RBN_STATIC_SCRATCH_TILES * 4096 + 128 * 4)
int rbn_gemm_t2_i8_skinny_static(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                 const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                                 uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out);
int rbn_matmul_t2_i8(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                     const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                     uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out);
/* Which of the three kernels rbn_matmul_t2_i8 runs for a shape (needs no device). */
#define RBN_KERNEL_GEMV 0
#define RBN_KERNEL_SKINNY 1
#define RBN_KERNEL_MFMA 2
int rbn_matmul_kernel_choice(uint64_t M, uint64_t K, uint64_t N);

/* ---- whole execute(): CompiledKernel::execute, TernaryMatMul arm,
 *      kernels.rs:271-283 ---------------------------------------------------- */
/* Host f32 A [M,K] and B [K,N] in, host f32 [M,N] out; both operands ternarised
 * per tensor on every call exactly as the reference does.  h_acc (optional) gets
 * the int32 accumulators.  mode is an rbn_sum_mode. */
int rbn_execute_ternary_matmul(rbn_ctx *ctx, const float *h_a, const float *h_b, uint64_t M,
                               uint64_t N, uint64_t K, int mode, float *h_out, int32_t *h_acc);

/* ---- decoder building blocks (no reference counterpart) --------------------- */
/* The reference's BitNet provider stops at the matmul; these are the usual
 * LLaMA / BitNet-b1.58 operations a decoder needs around it, so that a whole decode
 * step runs on the device and can be captured in a graph (positions and tokens are
 * read from device memory).  All row-major f32 unless said otherwise. */
/* One-token BitLinear in one launch: RMSNorm of d_x [K] (or of silu(gate) * up when
 * d_gate_up [2K] is given instead), per-token int8 quantisation as in
 * rbn_rmsnorm_quant_i8, ternary GEMV, fused dequantisation, and
 * out[n] = d_residual[n] + result when d_residual is given (it may be d_out itself).
 * K % 16 == 0, K <= 8192.  The int8 codes can differ from rbn_rmsnorm_quant_i8's by one
 * step where a value sits on a rounding boundary (different summation order). */
int rbn_bitlinear_gemv_f32(rbn_ctx *ctx, const float *d_x, const float *d_gate_up,
                           const float *d_gamma, float eps, const uint32_t *d_tiled,
                           float w_scale, uint64_t K, uint64_t N, const float *d_residual,
                           float *d_out);
/* x[m,:] = table[tokens[m],:] (token ids clamped to [0, vocab)). */
int rbn_embed_f32(rbn_ctx *ctx, const float *d_table, const int32_t *d_tokens, uint64_t M,
                  uint64_t H, uint64_t vocab, float *d_x);
/* Input row: x[m,:] (H values); or, when d_delta is given, x += delta, written back
 * (the residual stream); or, when d_gate_up [M, 2H] is given instead of d_x,
 * x = silu(gate) * up (SwiGLU on the way in; nothing is written back).  Then
 * y = (x * gamma) * rsqrt(mean(x^2) + eps), quantised per token exactly as
 * rbn_act_quant_i8 does (same output format).  H <= 8192. */
int rbn_rmsnorm_quant_i8(rbn_ctx *ctx, float *d_x, const float *d_delta, const float *d_gate_up,
                         const float *d_gamma, float eps, uint64_t M, uint64_t H, int8_t *d_q,
                         float *d_act_scale, int32_t *d_rowsum);
/* d_qkv [M, 3*heads*head_dim] = (q | k | v).  Rotary embedding (pairs
 * (i, i + head_dim/2), angle pos * theta^(-2i/head_dim), pos = *d_pos0 + m) of q in
 * place and of k on its way into the cache: rotated k and v go to the f16 caches
 * [heads][max_seq][head_dim] at pos; k and v in d_qkv stay as they were. */
int rbn_rope_kv_store_f16(rbn_ctx *ctx, float *d_qkv, const int32_t *d_pos0, uint64_t M,
                          uint64_t heads, uint64_t head_dim, float theta, void *d_kcache,
                          void *d_vcache, uint64_t max_seq);
/* Causal softmax(q.k / sqrt(head_dim)).v of token m over cache positions
 * 0 .. *d_pos0 + m; head_dim must be 128.  d_out [M, heads*head_dim]. */
int rbn_attention_f16kv(rbn_ctx *ctx, const float *d_qkv, const int32_t *d_pos0, uint64_t M,
                        uint64_t heads, uint64_t head_dim, const void *d_kcache,
                        const void *d_vcache, uint64_t max_seq, float *d_out);
/* One token: rbn_rope_kv_store_f16 and rbn_attention_f16kv in one launch (d_qkv is
 * not modified: the rotated q stays inside the kernel). */
int rbn_attention_decode_f16kv(rbn_ctx *ctx, const float *d_qkv, const int32_t *d_pos, uint64_t heads,
                               uint64_t head_dim, float theta, void *d_kcache, void *d_vcache,
                               uint64_t max_seq, float *d_out);
/* h[m,f] = silu(gu[m,f]) * gu[m,F+f], gu [M, 2F]. */
int rbn_swiglu_f32(rbn_ctx *ctx, const float *d_gate_up, uint64_t M, uint64_t F, float *d_h);
/* *d_index = index of the largest value (lowest index among equals).  If d_history
 * (history_capacity int32 entries) is given the index is also written to
 * d_history[*d_history_pos]; a position outside [0, history_capacity) writes nothing and
 * raises RBN_FLAG_HISTORY_OVERFLOW (rbn_device_flags). */
int rbn_argmax_f32(rbn_ctx *ctx, const float *d_values, uint64_t n, int32_t *d_index,
                   int32_t *d_history, const int32_t *d_history_pos, uint64_t history_capacity);
/* The tail of a greedy decode step in one launch: *d_pos += 1; t = arg-max of the vocab
 * logits (lowest index among equals); *d_token = t; d_history[*d_pos] = t; d_x[0..H) =
 * d_table[t, :] (the next step's embedding).  d_history holds history_capacity entries:
 * when *d_pos + 1 would leave it, the position stays, nothing is written to the history
 * and RBN_FLAG_HISTORY_OVERFLOW is raised (*d_token and d_x are still written).  The
 * attention kernels clamp positions to max_seq - 1 on their own: past the end of the K/V
 * cache they overwrite its last row and the output is meaningless, so a caller has to
 * stop at the capacity.  No counterpart in the reference (decoder harness). */
int rbn_greedy_next_f32(rbn_ctx *ctx, const float *d_logits, uint64_t vocab, int32_t *d_token,
                        int32_t *d_history, int32_t *d_pos, uint64_t history_capacity,
                        const float *d_table, uint64_t H, float *d_x);
/* *d_value += delta (the position counter of a captured decode step). */
int rbn_add_i32(rbn_ctx *ctx, int32_t *d_value, int32_t delta);
/* Normal(0, sigma) values generated on the device (counter-based, f32 Box-Muller);
 * for random-initialised weights; not the generator of rbn_synth_normal_f32. */
int rbn_synth_normal_device_f32(rbn_ctx *ctx, uint64_t seed, float sigma, float *d_out, uint64_t n);

/* ---- calibration probe (no reference counterpart) -------------------------- */
/* Runs a loop of nothing but v_mfma_i32_32x32x32_i8 on every SIMD (operands in
 * registers) and returns the dense int8 rate in TOP/s: the ceiling a GEMM on this
 * machine can be priced against besides the published 5.0 POP/s.  The sustained
 * clock depends on the operand values; operand_kind picks them. */
enum rbn_probe_operands {
    RBN_PROBE_CONSTANT = 0,   /* every byte 1 */
    RBN_PROBE_I8_TERNARY = 1, /* random int8 x ternary codes {0,1,2}: this path's data */
    RBN_PROBE_I8_I8 = 2       /* random int8 x random int8 */
};
int rbn_probe_mfma_i8(rbn_ctx *ctx, int operand_kind, double *h_tops);
/* The floor of a streaming kernel on this machine, for pricing the GEMV: one launch that does
 * nothing (rbn_probe_empty_launch), and one that only reads `bytes` of d_src with the GEMV's
 * access pattern (16-byte loads, 4 KiB of consecutive memory per wave; non-temporal or
 * plain) and stores nothing.  Asynchronous on the context's stream and capturable, so they
 * are timed the way the GEMV is (graph replay, rbn_timer_*). */
int rbn_probe_empty_launch(rbn_ctx *ctx);
int rbn_probe_stream_read(rbn_ctx *ctx, const void *d_src, uint64_t bytes, int nontemporal);

/* ---- synthetic inputs (host) ----------------------------------------------- */
/* out[i] = (float)(sigma * z_i), z_i standard normal from a counter-based
 * generator: two 24-bit uniforms from splitmix64(seed, i/2), Box-Muller in
 * double.  Deterministic for (seed, i); safe to call from several threads on
 * disjoint ranges via `first`. */
void rbn_synth_normal_f32(uint64_t seed, double sigma, uint64_t first, uint64_t count,
                          float *h_out);

#ifdef __cplusplus
}
#endif
#endif /* RONN_BITNET_HIP_H */
