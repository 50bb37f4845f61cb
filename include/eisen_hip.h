/*
 * eisen_hip.h -- C-ABI of libeisen_hip.so, the MI355X (gfx950) device backend for eisen's
 * training step.
 *
 * This is the surface a `Device::Gpu` backend binds over FFI in place of the cudarc driver
 * calls and the by-name CUDA kernels of the reference.  Plain C: opaque handles, raw device
 * pointers, sizes; no C++ or torch types.  Every function returns 0 on success, a positive
 * hipError_t on a HIP failure, or a negative EISEN_E_* code on an argument error; none of
 * them aborts.  `eisen_hip_last_error(ctx)` returns the message of the last failure.
 *
 * Conventions
 *   - One context = one device + one HIP stream (the reference is single-stream:
 *     src/tensor.rs:18-22 `Device::Gpu(ctx, stream)`).  Every op is enqueued on that stream
 *     and returns without synchronising unless stated.
 *   - `dtype` arguments take EISEN_F32 or EISEN_BF16 and name the element type of the
 *     activation buffers of the call.  Parameter gradients, norm gains, moments and master
 *     weights are always f32.
 *   - `accumulate` != 0 means `dst += value` (the reference's backward semantics,
 *     every backward_fn adds into `.grad`), 0 means `dst = value` (first writer of a
 *     gradient buffer; saves the zero-fill and the read).
 *   - Matrices are row-major and contiguous; linear weights are [in, out]
 *     (src/nn/linear.rs:40).
 */
#ifndef EISEN_HIP_H
#define EISEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct eisen_ctx eisen_ctx;
typedef struct eisen_module eisen_module;
typedef struct eisen_function eisen_function;

enum { EISEN_F32 = 0, EISEN_BF16 = 1 };

enum {
    EISEN_E_ARG = -1,      /* null pointer, zero/negative size, unknown dtype */
    EISEN_E_SHAPE = -2,    /* shape the kernel family does not support (message says which) */
    EISEN_E_ALIGN = -3,    /* pointer or row pitch not aligned as the kernel needs */
    EISEN_E_NOMEM = -4,    /* workspace could not be allocated */
    EISEN_E_STATE = -5     /* call order violated (e.g. timer stop without start) */
};

#define EISEN_IGNORE_INDEX (-1) /* target id of a masked row (reference: usize::MAX, src/data/fim.rs:173) */

/* ---- runtime: replaces the cudarc calls counted at src/graph/mod.rs:152-307 ------------- */

/* CudaContext::new(0) + ctx.default_stream() (tests/gpu_kernels.rs:6-14, src/main.rs:9-11). */
int eisen_hip_init(int device, eisen_ctx** out);
int eisen_hip_destroy(eisen_ctx* ctx);
const char* eisen_hip_last_error(eisen_ctx* ctx);
/* stream.synchronize() (e.g. src/graph/mod.rs:776-788). */
int eisen_hip_stream_sync(eisen_ctx* ctx);
/* A second stream of the context for work whose result nothing on the main stream needs soon (a weight-gradient GEMM
 * beside the input-gradient chain): calls between side_begin and side_end are ordered after everything issued before
 * side_begin and run concurrently with what is issued after side_end; side_wait orders the main stream after them
 * (eisen_hip_stream_sync waits for both).  Buffers the side work reads must not be written or freed before side_wait.
 * No counterpart in the reference, which runs one stream (src/graph/mod.rs:776-788). */
int eisen_hip_side_begin(eisen_ctx* ctx);
int eisen_hip_side_end(eisen_ctx* ctx);
int eisen_hip_side_wait(eisen_ctx* ctx);
/* The hipStream_t of the context, as void*, for callers that enqueue their own work. */
void* eisen_hip_stream(eisen_ctx* ctx);

/* stream.alloc_zeros / Graph::safe_alloc_zeros (src/graph/memory.rs:189-266) and the
 * size-keyed vram_pool in front of it (src/graph/mod.rs:437-556).  Stream-ordered:
 * a freed block may be handed out again to a later call on the same stream. */
int eisen_hip_malloc(eisen_ctx* ctx, size_t bytes, void** out);
int eisen_hip_malloc_zeroed(eisen_ctx* ctx, size_t bytes, void** out);
int eisen_hip_free(eisen_ctx* ctx, void* ptr);
/* Drop every cached block back to the driver (the OOM fallback's "clear pools" step). */
int eisen_hip_pool_trim(eisen_ctx* ctx);
/* ctx.mem_get_info() (src/graph/memory.rs:429-470). */
int eisen_hip_mem_info(eisen_ctx* ctx, size_t* free_bytes, size_t* total_bytes);
/* Bytes currently handed out / cached by the pool (diagnostics, tests). */
int eisen_hip_pool_stats(eisen_ctx* ctx, size_t* in_use_bytes, size_t* cached_bytes);
/* How often this context has asked the driver for memory so far (device-pool misses, workspace growth, rotary tables,
 * pinned staging): a caller that must not allocate checks that a call leaves it unchanged (diagnostics, tests). */
int eisen_hip_driver_allocs(eisen_ctx* ctx, size_t* count_out);
/* Largest value in_use_bytes has had since the last call with reset != 0 (the activation high-water mark of a step). */
int eisen_hip_pool_peak(eisen_ctx* ctx, size_t* peak_in_use_bytes, int reset);

/* stream.memcpy_htod / clone_htod (src/graph/mod.rs:368-430, src/tensor.rs:156-160):
 * asynchronous on the stream; the host buffer is copied to a staging area first, so it may
 * be reused as soon as the call returns. */
int eisen_hip_htod(eisen_ctx* ctx, void* dst_device, const void* src_host, size_t bytes);
/* stream.clone_dtoh (src/tensor.rs:177-223): synchronises the stream before returning. */
int eisen_hip_dtoh(eisen_ctx* ctx, void* dst_host, const void* src_device, size_t bytes);
/* clone_dtoh in two halves, for a value the host wants without draining the stream (the loss of a micro-batch,
 * examples/train_llm.rs:450, read while the backward pass is already queued): `begin` enqueues the copy into pinned
 * memory of the library and returns a ticket, `finish` waits for that copy alone and fills dst_host.  At most 8 tickets
 * may be outstanding; bytes <= 8 MiB. */
int eisen_hip_dtoh_begin(eisen_ctx* ctx, const void* src_device, size_t bytes, int* ticket_out);
int eisen_hip_dtoh_finish(eisen_ctx* ctx, int ticket, void* dst_host, size_t bytes);
int eisen_hip_dtod(eisen_ctx* ctx, void* dst_device, const void* src_device, size_t bytes);
int eisen_hip_memset_zero(eisen_ctx* ctx, void* dst_device, size_t bytes);

/* ctx.load_module(ptx) / module.load_function(name) / stream.launch_builder(f)...launch(cfg)
 * (src/graph/mod.rs:155-266; e.g. src/graph/ops/normalization.rs:47-88).  `image` is a
 * gfx950 code object (hipcc --genco).  `args` follows hipModuleLaunchKernel: an array of
 * pointers to the argument values, in order. */
int eisen_hip_module_load(eisen_ctx* ctx, const void* image, size_t len, eisen_module** out);
int eisen_hip_module_unload(eisen_ctx* ctx, eisen_module* mod);
int eisen_hip_get_function(eisen_ctx* ctx, eisen_module* mod, const char* name, eisen_function** out);
int eisen_hip_launch(eisen_ctx* ctx, eisen_function* fn, const unsigned grid[3], const unsigned block[3],
                     unsigned shared_bytes, void** args);

/* HIP-event stopwatch on the context's stream (the reference only has host Instant timers,
 * examples/train_llm.rs:484-496).  stop() synchronises and returns milliseconds. */
int eisen_hip_timer_start(eisen_ctx* ctx);
int eisen_hip_timer_stop(eisen_ctx* ctx, float* ms_out);

/* Per-kernel timing for roofline reports: between start and stop every instrumented launch is
 * bracketed by two HIP events on the context's stream.  stop() synchronises and returns one
 * entry per kernel family that ran: total milliseconds, launches, and the algorithmic work
 * (flops for the MFMA kernels, bytes for the HBM-bound ones) those launches were asked for. */
typedef struct {
    char name[48];
    double ms;
    double work;
    unsigned long long launches;
    int work_is_flops;
} eisen_prof_entry;
int eisen_hip_profile_start(eisen_ctx* ctx);
int eisen_hip_profile_stop(eisen_ctx* ctx, eisen_prof_entry* out, size_t capacity, size_t* count_out);
/* Measured MFMA ceiling of this GPU, for the roofline figures (no counterpart in the reference, whose kernels use no matrix
 * instructions): runs a kernel of nothing but v_mfma_f32_32x32x16_bf16 on every CU (two waves per SIMD, four independent
 * 32x32 accumulators per wave, `iters` x 16 MFMAs per wave), once untimed and once between two events on the context's
 * stream, and returns the achieved TFLOP/s.  lds_reads_per_16_mfma = 0: operands stay in registers; 16: every contraction
 * step re-reads two A and two B operands from LDS (the ratio of a 64x64 wave tile); 8: the ratio of a 128x128 wave tile;
 * 24, 32: one and a half times and twice the reads of a 64x64 wave tile (where the LDS begins to hold the MFMAs back).
 * Synchronises the stream. */
int eisen_hip_mfma_ceiling(eisen_ctx* ctx, int lds_reads_per_16_mfma, int iters, double* tflops_out);
/* The same loops on operands whose bits change from one MFMA to the next (random sign, exponent and mantissa) instead
 * of a few dozen distinct small values.  The clock this GPU holds under matrix load depends on the operands: the same GEMM
 * runs a third faster on all-zero or constant matrices than on random ones, so this is the ceiling to read a kernel on
 * real data against. */
int eisen_hip_mfma_ceiling_random(eisen_ctx* ctx, int lds_reads_per_16_mfma, int iters, double* tflops_out);

/* ---- elementwise ---------------------------------------------------------------------- */

/* fill_f32 / scale_f32 (kernels/ops_f32.cu:101,107; callers src/graph/mod.rs:683-693,
 * src/nn/optim.rs:183-192,224-235). */
int eisen_hip_fill(eisen_ctx* ctx, void* dst, int dtype, float value, size_t n);
int eisen_hip_scale(eisen_ctx* ctx, void* dst, int dtype, float factor, size_t n);
/* dst *= *factor_device (factor read on the device: no host round trip). */
int eisen_hip_scale_by_device_scalar(eisen_ctx* ctx, void* dst, int dtype, const float* factor_device, size_t n);
/* cast_f32_to_bf16 / cast_bf16_to_f32 (kernels/ops_bf16.cu:4,11), round-to-nearest-even. */
int eisen_hip_cast(eisen_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype, size_t n);
/* accumulate_f32 without broadcast (kernels/ops_f32.cu:84; add/reshape/copy backward,
 * src/graph/ops/elementwise.rs:116-137, transform.rs:365-380): dst (+)= src. */
int eisen_hip_accumulate(eisen_ctx* ctx, void* dst, const void* src, int dtype, size_t n, int accumulate);
/* add_f32 / mul_f32 same-shape fast path (kernels/ops_f32.cu:66,113). */
int eisen_hip_add(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, size_t n);
int eisen_hip_mul(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, size_t n);
/* Broadcasting add/mul, rank <= 4 (Graph::add / Graph::mul, src/graph/ops/elementwise.rs:15-145,
 * :188-293).  out_shape has `rank` entries; a_strides/b_strides are element strides in the
 * broadcast shape (0 on broadcast dims, src/tensor.rs:249-263). */
int eisen_hip_add_bcast(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, int rank,
                        const size_t* out_shape, const size_t* a_strides, const size_t* b_strides);
int eisen_hip_mul_bcast(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, int rank,
                        const size_t* out_shape, const size_t* a_strides, const size_t* b_strides);
/* Backward of a broadcast operand: dst[bcast_idx(i)] += src[i] * (mul ? other[other_idx(i)] : 1),
 * reduced deterministically (one thread owns one dst element and walks its sources in
 * ascending i) -- replaces accumulate_f32's atomicAdd (kernels/ops_f32.cu:84-99). */
int eisen_hip_bcast_backward(eisen_ctx* ctx, void* dst, const void* grad_out, const void* other, int dtype,
                             int rank, const size_t* out_shape, const size_t* dst_strides,
                             const size_t* other_strides, size_t dst_numel, int accumulate);
/* The same with an f32 destination whatever `dtype` the operands have: the gradient of a parameter operand (a Linear
 * bias, src/nn/linear.rs:88-93 `g.add(out, bias)`) in mixed precision, where gradients of activations are bf16 and
 * gradients of parameters f32.  Also covers an operand of the full output shape (no reduced dimension). */
int eisen_hip_bcast_backward_f32(eisen_ctx* ctx, float* dst, const void* grad_out, const void* other, int dtype,
                                 int rank, const size_t* out_shape, const size_t* dst_strides,
                                 const size_t* other_strides, size_t dst_numel, int accumulate);
/* mul_backward_f32 same-shape (kernels/ops_f32.cu:119): ga (+)= b*go, gb (+)= a*go.
 * ga or gb may be NULL (constant operand). */
int eisen_hip_mul_backward(eisen_ctx* ctx, const void* a, const void* b, const void* go, void* ga, void* gb,
                           int dtype, size_t n, int accumulate_a, int accumulate_b);
/* silu_f32 / silu_backward_f32 (kernels/ops_f32.cu:135,142; src/graph/ops/elementwise.rs:337-465). */
int eisen_hip_silu(eisen_ctx* ctx, const void* x, void* out, int dtype, size_t n);
int eisen_hip_silu_backward(eisen_ctx* ctx, const void* x, const void* go, void* gx, int dtype, size_t n,
                            int accumulate);
/* Fused silu(gate)*up and its backward: the gate/silu/up/mul chain of
 * TransformerBlock::forward_with_mask (src/nn/transformer.rs:40-43) in one pass each way. */
int eisen_hip_swiglu(eisen_ctx* ctx, const void* gate, const void* up, void* out, int dtype, size_t n);
int eisen_hip_swiglu_backward(eisen_ctx* ctx, const void* gate, const void* up, const void* go, void* dgate,
                              void* dup, int dtype, size_t n, int accumulate_gate, int accumulate_up);

/* ---- normalisation, rotary, layout ----------------------------------------------------- */

/* rmsnorm_f32 / rmsnorm_backward_f32 (kernels/ops_f32.cu:539-578; Graph::rms_norm,
 * src/graph/ops/normalization.rs:8-184).  w, rrms, gw are f32.  rrms [rows] is written by the
 * forward and read by the backward.  gw += sum over rows (two-stage, fixed order, no atomics). */
int eisen_hip_rms_norm(eisen_ctx* ctx, const void* x, const float* w, void* out, float* rrms, int dtype,
                       size_t rows, size_t dim, float eps);
int eisen_hip_rms_norm_backward(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go,
                                void* gx, float* gw, int dtype, size_t rows, size_t dim, int accumulate_x);

/* eisen_hip_rms_norm_backward in two parts, for a caller with many norms (a transformer block has two): `_partial`
 * writes dx and leaves the gain gradient as *nrows_out rows of per-workgroup column sums in `partial`
 * ([EISEN_RMS_NORM_PARTIAL_ROWS][dim] f32, caller's buffer); `_finish` adds the rows of n such buffers to their
 * gain gradients (gw_i += column sums of partial_i, fixed order, distinct gw_i) in one launch; where assign[i] != 0
 * (assign may be NULL) gw_i is overwritten instead, for a gradient whose clearing is still pending.  The reference runs
 * one rmsnorm_backward_f32 per norm (src/graph/ops/normalization.rs:157-171). */
#define EISEN_RMS_NORM_PARTIAL_ROWS 256
int eisen_hip_rms_norm_backward_partial(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go, void* gx,
                                        float* partial, size_t* nrows_out, int dtype, size_t rows, size_t dim, int accumulate_x);
/* eisen_hip_rms_norm_backward_partial whose input gradient is gx = gx_in + dx: what it adds to is read from another
 * buffer than the one it writes (gx_in may also be gx itself).  For a caller that must keep gx_in as it is. */
int eisen_hip_rms_norm_backward_partial_add(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go, const void* gx_in,
                                            void* gx, float* partial, size_t* nrows_out, int dtype, size_t rows, size_t dim);
int eisen_hip_rms_norm_dw_finish(eisen_ctx* ctx, size_t n, const float* const* partial, float* const* gw, const size_t* nrows, size_t dim,
                                 const int* assign);
/* rope_f32 / rope_backward_f32 (kernels/ops_f32.cu:724-760; Graph::rope,
 * src/graph/ops/transform.rs:467-610): x [batch, seq, hidden], interleaved pairs within each
 * head of `head_dim`, base 10000, position = index along dim 1. */
int eisen_hip_rope(eisen_ctx* ctx, const void* x, void* out, int dtype, size_t batch, size_t seq, size_t hidden,
                   size_t head_dim);
int eisen_hip_rope_backward(eisen_ctx* ctx, const void* go, void* gx, int dtype, size_t batch, size_t seq,
                            size_t hidden, size_t head_dim, int accumulate);

/* rope(x W) as one kernel: a projection of GroupedQueryAttention::forward_with_mask with the `g.rope` that follows it
 * (src/nn/attention.rs:300-305, :316-317; Graph::matmul, src/graph/ops/linear.rs:235-259, then Graph::rope,
 * src/graph/ops/transform.rs:467-610).  A [M, K] (M = batches of `seq` rows) is shared by `batch` products with their own
 * B [K, N] (stride_b elements apart) and C [M, N] (stride_c apart); the first `rope_members` of them leave rotated
 * (heads of `head_dim` columns, row m at position m % seq), the others as plain products (the v projection beside k).
 * The product is rounded to the element type before it is rotated: the same bits as eisen_hip_gemm followed by
 * eisen_hip_rope, which is also what shapes outside the fused kernel's tiles run. */
int eisen_hip_gemm_rope(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype, size_t batch, size_t M, size_t N, size_t K,
                        long long stride_b, long long stride_c, size_t rope_members, size_t seq, size_t head_dim);

/* eisen_hip_rope of two tensors that share batch, seq and head_dim in one launch: the q and k projections of
 * GroupedQueryAttention::forward_with_mask (src/nn/attention.rs:304-305, two `g.rope` calls). */
int eisen_hip_rope_pair(eisen_ctx* ctx, const void* q, void* q_out, size_t hidden_q, const void* k, void* k_out, size_t hidden_k, int dtype,
                        size_t batch, size_t seq, size_t head_dim);
/* transpose_0213_f32 / _backward (kernels/ops_f32.cu:694,709; src/graph/ops/transform.rs:7-127):
 * [b, s, h, d] -> [b, h, s, d]; the backward is the same permutation applied to the grad. */
int eisen_hip_transpose_0213(eisen_ctx* ctx, const void* in, void* out, int dtype, size_t b, size_t s, size_t h,
                             size_t d, int accumulate);
/* repeat_kv_f32 / _backward (kernels/ops_f32.cu:787-838; src/graph/ops/gqa.rs:13-194). */
int eisen_hip_repeat_kv(eisen_ctx* ctx, const void* in, void* out, int dtype, size_t batch, size_t kv_heads,
                        size_t seq, size_t head_dim, size_t repeats);
int eisen_hip_repeat_kv_backward(eisen_ctx* ctx, const void* go, void* gin, int dtype, size_t batch,
                                 size_t kv_heads, size_t seq, size_t head_dim, size_t repeats, int accumulate);
/* softmax_f32 / softmax_backward_f32 over the last dim (kernels/ops_f32.cu:625,636;
 * src/graph/ops/reduction.rs:397-523). */
int eisen_hip_softmax(eisen_ctx* ctx, const void* x, void* out, int dtype, size_t rows, size_t n);
int eisen_hip_softmax_backward(eisen_ctx* ctx, const void* out, const void* go, void* gx, int dtype, size_t rows,
                               size_t n, int accumulate);

/* ---- contractions ---------------------------------------------------------------------- */

/* C[M,N] (+)= op(A) * op(B), row-major.  op(A) = A stored [M,K], or A stored [K,M] when
 * trans_a; op(B) = B stored [K,N], or B stored [N,K] when trans_b.  Covers
 *   Graph::matmul forward (matmul_f32 / matmul_bf16_f32, kernels/ops_f32.cu:158, ops_bf16.cu:26;
 *     src/graph/ops/linear.rs:35-263):                       trans_a=0, trans_b=0
 *   dX = dY * W^T (matmul_backward_a_f32, ops_f32.cu:192; linear.rs:266-277):  trans_b=1
 *   dW += X^T * dY (matmul_backward_b_f32, ops_f32.cu:225; linear.rs:278-287): trans_a=1, accumulate=1
 *   tied lm_head (matmul_trans_b_f32 / matmul_trans_a_f32, ops_f32.cu:842-882; linear.rs:301-517).
 * dtype_ab: element type of A and B; dtype_c: element type of C (f32 operands need f32 C).
 * bf16 operands run on MFMA with f32 accumulation; f32 operands on an FMA kernel. */
int eisen_hip_gemm(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                   int trans_b, size_t M, size_t N, size_t K, int accumulate);
/* Batched form with contiguous batches (bmm_f32 and its four backward kernels,
 * kernels/ops_f32.cu:342-510; Graph::bmm, src/graph/ops/linear.rs:1198-1511). */
int eisen_hip_bmm(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                  int trans_b, size_t batch, size_t M, size_t N, size_t K, int accumulate);
/* The same with explicit batch strides in elements (any sign, 0 = operand shared by every batch).  This is how
 * linear layers that read the same input run as one launch: K and V projections, or the gate and up
 * projections of the MLP (src/nn/attention.rs:300-302, src/nn/transformer.rs:41-44 issue them as separate
 * matmuls): A shared, B and C "strided" by the distance between the two weight / output tensors. */
int eisen_hip_gemm_strided_batched(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                                   int trans_b, size_t batch, size_t M, size_t N, size_t K, long long stride_a,
                                   long long stride_b, long long stride_c, int accumulate);

/* C = R + op(A) * op(B), R with C's shape and element type (R may be C).  A linear layer followed by the
 * residual add of the transformer block (src/nn/transformer.rs:36, :47: `g.add(x_id, attn_out)`,
 * `g.add(res1_out, ffn2_out)`) as one kernel: the product is added to the residual in f32 and rounded once. */
int eisen_hip_gemm_residual(eisen_ctx* ctx, const void* A, const void* B, const void* R, void* C, int dtype_ab, int dtype_c,
                            int trans_a, int trans_b, size_t M, size_t N, size_t K);

/* C_p (+)= op(A_p) * op(B_p) for p < n <= 8: products that share M, K, the operand orders and the element types but
 * have their own operands, outputs and N_p.  Stands for n calls of the matmul backward's dB GEMM
 * (src/graph/ops/linear.rs:279-287), e.g. the weight gradients of the Q, K, V, output, gate and up projections of one
 * transformer block; they run as one grid when that fills the chip better than the separate launches. */
int eisen_hip_gemm_grouped(eisen_ctx* ctx, size_t n, const void* const* A, const void* const* B, void* const* C, const size_t* N,
                           int dtype_ab, int dtype_c, int trans_a, int trans_b, size_t M, size_t K, int accumulate);

/* C_p (+)= sum_{s < n_segments} A_ps^T B_ps for p < n_products: the dB += A^T dC of the matmul backward
 * (src/graph/ops/linear.rs:279-287) for several weights and several micro-batches of a gradient-accumulation
 * window at once.  A[p * n_segments + s] is bf16 [seg_k, M_p] (the activations weight p multiplied in micro-batch s),
 * B[p * n_segments + s] bf16 [seg_k, N_p] (the gradient of that product), C[p] f32 [M_p, N_p].  The reference adds one
 * micro-batch at a time, in f32; here the pieces of a product are summed in the MFMA accumulators of one launch (any
 * number of products of up to 8 pieces, every M_p and N_p a multiple of 256, seg_k of 128, at least 176 tiles of
 * 256 x 256 in all), which reads and writes each gradient once per window instead of once per micro-batch.  Other
 * shapes run one accumulating GEMM per product and piece, in piece order. */
#define EISEN_GEMM_MAX_KSEGMENTS 8
int eisen_hip_gemm_grouped_ksegments(eisen_ctx* ctx, size_t n_products, size_t n_segments, const void* const* A, const void* const* B,
                                     void* const* C, const size_t* M, const size_t* N, size_t seg_k, int accumulate);

/* Tuning of the one-launch form of eisen_hip_gemm_grouped_ksegments (no counterpart in the reference).  An XCD of the GPU
 * runs 32 tiles at a time, which share twelve operand panels in its L2 as long as they walk their contraction close
 * together; left alone they drift apart over the launch and fetch the panels several times.  So a workgroup counts itself
 * in at its group of 32 tiles and waits until the group is complete or `microseconds` have passed, whichever comes first
 * (default 40; 0 switches the meeting points off).  The wait is bounded and no result depends on it: the same bits either
 * way.  At config 5 it cuts the bytes these launches fetch past the L2 by a quarter. */
int eisen_hip_gemm_window_meet(eisen_ctx* ctx, int microseconds);

/* G = X Wg, U = X Wu, H = silu(G) * U: the gate and up projections of the feed-forward block and their SwiGLU
 * (src/nn/transformer.rs:41-46: `ffn_gate.forward`, `g.silu`, `ffn1.forward`, `g.mul`) as one kernel.  X [M, K],
 * Wg, Wu [K, N], G, U, H [M, N] of `dtype`; G and U are written because the backward pass reads them. */
int eisen_hip_gemm_swiglu_forward(eisen_ctx* ctx, const void* X, const void* Wg, const void* Wu, void* G, void* U, void* H, int dtype,
                                  size_t M, size_t N, size_t K);

/* [dgate, dup] = d(silu(gate) * up) for dH = op(A) * op(B): the input gradient of the down projection
 * (src/graph/ops/linear.rs:269-277, dA = dC B^T) followed by the backward of `g.mul(g.silu(gate), up)`
 * (src/nn/transformer.rs:44-46; src/graph/ops/elementwise.rs:442-455 silu, :294-331 mul) in one kernel: dH is
 * never stored, the two gradients are formed from the f32 accumulators.  gate, up, dgate, dup are [M, N] of
 * `dtype`; the results are assigned (no accumulation). */
int eisen_hip_gemm_swiglu_backward(eisen_ctx* ctx, const void* A, const void* B, const void* gate, const void* up, void* dgate,
                                   void* dup, int dtype, int trans_a, int trans_b, size_t M, size_t N, size_t K);
/* C (+)= sum over up to three segments s of op(A_s) * op(B_s), each segment with its own operands and
 * contraction length K_s (A_s is [M,K_s] or, transposed, [K_s,M]; B_s is [K_s,N] or [N,K_s]).  This is the
 * input gradient of several linear layers that read the same tensor (dX = dQ Wq^T + dK Wk^T + dV Wv^T, which
 * the reference accumulates with three matmul backward calls, src/graph/ops/linear.rs:266-277) as one launch
 * and one write of dX.  Segments that are not multiples of 64 run as consecutive accumulating GEMMs. */
int eisen_hip_gemm_ksegments(eisen_ctx* ctx, size_t n_segments, const void* const* A, const void* const* B, const size_t* K, void* C,
                             int dtype_ab, int dtype_c, int trans_a, int trans_b, size_t M, size_t N, int accumulate);

/* ---- attention ------------------------------------------------------------------------- */

/* Causal grouped-query attention with saved log-sum-exp, and its backward.  Computes what
 * GroupedQueryAttention::forward_with_mask builds from reshape / transpose_0213 / repeat_kv /
 * bmm / mul(scale) / add(mask) / softmax / bmm (src/nn/attention.rs:300-375) and what that
 * chain's backward closures accumulate (src/graph/ops/linear.rs:1452-1498, reduction.rs:504-512,
 * gqa.rs:168-184), without materialising scores or repeated K/V.  The reference's own fused
 * kernel is forward/inference only (flash_attention_f32, kernels/ops_f32.cu:648-692;
 * src/graph/ops/attention.rs:7-18).
 *   q, out, dout, dq : [B, S, Hq, hd];  k, v, dk, dv : [B, S, Hkv, hd];  lse : [B, Hq, S] f32.
 * q_strides / kv_strides: optional {batch, seq, head} element strides (NULL = the contiguous
 * layouts above; {Hq*S*hd, hd, S*hd} addresses the reference's [B,H,S,hd] tensors).
 * Query head h attends KV head h / (Hq/Hkv); dk, dv are summed over the heads of each group.
 * dq, dk, dv are overwritten.  bf16: hd in {32, 64, 128}; f32: hd <= 256, S <= 8192. */
int eisen_hip_attention_forward(eisen_ctx* ctx, const void* q, const void* k, const void* v, void* out, float* lse,
                                int dtype, size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd,
                                const long long* q_strides, const long long* kv_strides, float scale, int causal);
int eisen_hip_attention_backward(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                 const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype, size_t B,
                                 size_t S, size_t Hq, size_t Hkv, size_t hd, const long long* q_strides,
                                 const long long* kv_strides, float scale, int causal);

/* eisen_hip_attention_backward for callers that cannot allocate (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and the same
 * results; the scratch the kernels need beyond the inputs and outputs, D = rowsum(dO o O) and -LSE/scale with one float
 * each per (batch, query head, position), lives in a fixed 8 MiB device array of the library instead of the context's growing
 * workspace, so the call reaches no hipMalloc / hipFree / pool routine.  Limit: B * Hq * S <= 1,048,576, larger
 * shapes return EISEN_E_SHAPE.  Every call on one GPU uses that GPU's one array.  Outside graph capture the library puts
 * such calls in order itself: each call's stream first waits for an event recorded behind the previous call's kernels
 * (another context on the GPU, or the context's other stream), so they cannot overlap.  Under graph capture no event
 * from outside the graph can be waited for: calls captured into graphs that may run at the same time on one GPU race,
 * and ordering them is the caller's job.  Nothing in the array has to be cleared between calls: the dQ kernel writes
 * every row that the dK/dV kernel reads. */
int eisen_hip_attention_backward_noalloc(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                         const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype, size_t B,
                                         size_t S, size_t Hq, size_t Hkv, size_t hd, const long long* q_strides,
                                         const long long* kv_strides, float scale, int causal);

/* Measurement aid for the two bf16 backward kernels at head_dim 64 with four query heads per KV head (no counterpart in
 * the reference): until called again with 0, every eisen_hip_attention_backward* call on this context runs kernels that
 * leave one part of their tile loop out, so that the part's share of the kernel's duration can be read from the
 * difference.  THE RESULTS OF SUCH A CALL ARE WRONG BY CONSTRUCTION; the memory accesses that remain are those of the
 * full kernels.  part: 1 the LDS transpose reads, 2 the 16-byte LDS operand reads, 3 the MFMAs after the softmax,
 * 4 the global-to-LDS loads of every tile after the first, 5 the softmax arithmetic, 6 the S and dP MFMAs; 0 none. */
int eisen_hip_attention_ablation(eisen_ctx* ctx, int part);

/* Measurement aid for the three bf16 attention kernels at head_dim 64 with four query heads per KV head (no counterpart in
 * the reference): while a buffer is set, every wave of those kernels drops time stamps of its progress, the results are
 * the usual ones.  stamps: device memory for 3 * waves * 16 values of 8 bytes, laid out [kernel: 0 forward, 1 dQ,
 * 2 dK/dV][wave = block * 4 + wave of the block][stamp 0..7][0: the GPU's 100 MHz counter, 1: its shader clock]; waves
 * beyond `waves` drop nothing.  Stamp 0: kernel entered; 1, 2: first tile loop begins, ends; 3: its results stored; 4, 5,
 * 6: the same for the second query (key) block of a paired workgroup, zero where there is none.  (nullptr, 0) ends it. */
int eisen_hip_attention_timeline(eisen_ctx* ctx, long long* stamps, size_t waves);

/* Measurement aid (no counterpart in the reference): a model of the tile loop of the key-stationary attention-backward
 * kernel at head_dim 64, built from the same instructions on made-up data, timed with any of its parts alone or together.
 * parts: 1 the sixteen MFMAs of a tile; 3 those and the vector work between them; 7 those and the tile's LDS reads; 8 only
 * the eight 1 KB direct-to-LDS loads that bring a wave's next tile (from a region that stays in the L2); 15 everything.
 * parts 16: the tile loop a one-pass backward would have instead (score tile and dP computed once; the four waves of a
 * workgroup own 128 keys, work on one 32-query tile at a time, share its Q / dO tile, exchange their dS tiles through LDS
 * behind one barrier per tile and write a dQ partial of 8 KB per workgroup and tile); 32: the same without those writes.
 * waves_per_simd: 1 or 2 (the kernel runs two).  *ns_per_tile_out: time per tile and SIMD over `iters` tiles per wave. */
int eisen_hip_attention_tile_model(eisen_ctx* ctx, int parts, int waves_per_simd, int iters, double* ns_per_tile_out);

/* Measurement aid (no counterpart in the reference): the two small kernels that a one-pass attention backward would need
 * around its main kernel, timed on made-up data at head_dim 64, to be set beside the one-pass tile model
 * (eisen_hip_attention_tile_model, parts 16 / 32).  *rowdot_us_out: D = rowsum(dO o O) over `rows` bf16 rows of 64.
 * *partial_sum_us_out: dQ as the sum, in a fixed order, of the f32 partials of the key chunks a causal query sees
 * (position / chunk + 1 of them; rows = whole sequences of `seq`), stored as bf16.  Averages over 10 launches. */
int eisen_hip_attention_onepass_parts(eisen_ctx* ctx, size_t rows, int seq, int chunk, double* rowdot_us_out, double* partial_sum_us_out);

/* eisen_hip_attention_backward for q and k that are rotary-embedded projections, q = rope(q0), k = rope(k0)
 * (src/nn/attention.rs:316-317 applies `g.rope` to both before the attention chain): dq and dk receive the
 * gradients of q0 and k0, i.e. the rotary backward (src/graph/ops/transform.rs:592-595) is applied to the f32
 * results as they are stored instead of in two further passes over dq and dk.  Contiguous [B, S, H, hd]
 * layouts only; positions are the sequence index. */
int eisen_hip_attention_rope_backward(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                      const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype,
                                      size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd, float scale, int causal);

/* ---- embedding ------------------------------------------------------------------------- */

/* gather_f32 (kernels/ops_f32.cu:513; Graph::gather, src/graph/ops/transform.rs:132-324).
 * ids are int32 on the device (the reference stores them as f32 and casts, :294). */
int eisen_hip_gather(eisen_ctx* ctx, const void* weight, const int32_t* ids, void* out, int dtype, size_t n_ids,
                     size_t vocab, size_t hidden);
/* Embedding-gradient scatter, deterministic (replaces gather_backward_f32's atomicAdd,
 * kernels/ops_f32.cu:526-537).  gw[ids[i], :] += go[i, :], every row receiving its addends
 * in ascending i exactly like the CPU arm (src/graph/ops/transform.rs:306-315).
 * `ids_host` is the host copy of the ids (they originate on the host in every caller,
 * examples/train_llm.rs:433-435); the call checks them, uploads them and indexes them on the device where
 * eisen_hip_gather_backward_dev can, otherwise it builds the stable position index on the host. */
int eisen_hip_gather_backward(eisen_ctx* ctx, const int32_t* ids_host, const void* go, float* gw, int dtype,
                              size_t n_ids, size_t vocab, size_t hidden);
/* The same scatter with the ids already on the device (the int32 buffer eisen_hip_gather read): nothing is sorted or
 * uploaded by the host.  Up to 16384 ids with vocab * next_pow2(n_ids) < 2^32 are indexed by one workgroup (a stable
 * sort of the positions by id in LDS) and scattered run by run; other shapes read the ids back (which synchronises)
 * and take eisen_hip_gather_backward.  The ids must lie in [0, vocab), as they did for the gather; an id outside is
 * skipped on the device route. */
int eisen_hip_gather_backward_dev(eisen_ctx* ctx, const int32_t* ids_dev, const void* go, float* gw, int dtype,
                                  size_t n_ids, size_t vocab, size_t hidden);
/* eisen_hip_gather_backward_dev in two halves, for a caller that knows the ids long before the gradient exists (the token
 * ids of a training step are known when its forward pass starts).  _index_dev builds the position index of the ordered
 * scatter from the ids alone: `index` receives 3 * n_ids int32 (device memory); EISEN_E_SHAPE when the batch is more
 * than the device-side index takes (more than 16384 ids, or vocab * ids beyond 32 bits): then use _backward_dev.
 * _backward_indexed adds the rows of dOut into the f32 gradient in ascending position with that index, the result of
 * eisen_hip_gather_backward_dev bit for bit (src/graph/ops/transform.rs:306-315 is the order it keeps). */
int eisen_hip_gather_index_dev(eisen_ctx* ctx, const int32_t* ids_dev, size_t n_ids, size_t vocab, int32_t* index);
int eisen_hip_gather_backward_indexed(eisen_ctx* ctx, const int32_t* index, const void* go, float* gw, int dtype, size_t n_ids,
                                      size_t vocab, size_t hidden);

/* ---- loss ------------------------------------------------------------------------------ */

/* Fused softmax-cross-entropy forward+backward in one pass over the logits
 * (cross_entropy_f32 + cross_entropy_backward_f32, kernels/ops_f32.cu:580-623, and the masked
 * pair :5-64; Graph::cross_entropy / cross_entropy_masked, src/graph/ops/reduction.rs:529-944).
 *   loss_out[0] = normalizer * sum_rows -ln(p_target + 1e-8)      (rows with target -1 skipped)
 *   dlogits     = (p - onehot(target)) * normalizer * grad_scale  (zero for skipped rows)
 * normalizer = 1/rows, or 1/valid_rows when any target is EISEN_IGNORE_INDEX.
 * targets: int32 on the device.  row_loss [rows] f32 scratch owned by the caller.
 * argmax_out (int32 [rows]) and target_logit_out (f32 [rows]) may be NULL; when given they
 * receive the first index of the row maximum and the logit at the target (0 for skipped rows). */
int eisen_hip_cross_entropy(eisen_ctx* ctx, const void* logits, const int32_t* targets, void* dlogits,
                            float* row_loss, float* loss_out, int32_t* argmax_out, float* target_logit_out,
                            int dtype, size_t rows, size_t classes, float normalizer, float grad_scale);

/* ---- optimiser ------------------------------------------------------------------------- */

/* One parameter tensor of a fused multi-tensor optimiser call. */
typedef struct {
    float* w;          /* f32 master weight */
    const float* g;    /* f32 gradient */
    float* m;          /* f32 first moment */
    float* v;          /* f32 second moment */
    void* w_bf16;      /* optional bf16 copy of the updated weight (NULL: none) */
    size_t n;          /* elements */
} eisen_param_slot;

/* adamw_step_f32 (kernels/ops_f32.cu:762-784; AdamW::step, src/nn/optim.rs:334-562) over all
 * tensors in one launch.  bc1/bc2 are the reciprocal bias corrections 1/(1-beta^t) computed
 * by the caller (src/nn/optim.rs:336-338).  grad_scale_device: optional device f32 the
 * gradient is multiplied with first (the clip coefficient); NULL = 1. */
int eisen_hip_adamw_step(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots, float lr, float beta1,
                         float beta2, float eps, float weight_decay, float bc1, float bc2,
                         const float* grad_scale_device);
/* AdamW::clip_grad_norm without the D2H of every gradient (src/nn/optim.rs:250-321):
 * out_device[0] = sqrt(sum g^2) with f64 accumulation, out_device[1] = clip coefficient
 * min(1, max_norm/(norm+1e-6)) (1 when norm == 0).  Deterministic two-stage reduction. */
int eisen_hip_grad_norm(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots, float max_norm,
                        float* out_device);
/* AdamW::zero_grad over all tensors in one launch (src/nn/optim.rs:207-245). */
int eisen_hip_zero_grads(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots);

#ifdef __cplusplus
}
#endif
#endif /* EISEN_HIP_H */
