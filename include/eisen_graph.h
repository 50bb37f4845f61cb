/*
 * eisen_graph.h -- C-ABI of the host-side Graph / nn / AdamW layer in libeisen_hip.so.
 *
 * The reference's host layer is Rust (`Graph`, `Tensor`, the `Module` trait, `AdamW`;
 * src/graph/mod.rs and the files under src/nn/).  Where a Rust toolchain is present that layer binds
 * include/eisen_hip.h directly; this header exposes the C++ mirror of it that ships in the
 * library, with the same operations, argument meaning and error behaviour, so tests, the
 * benchmark and non-Rust hosts can drive a full training step.
 *
 * Every function returns 0 on success and non-zero on failure (the reference panics; a host
 * may turn non-zero into a panic).  `eisen_graph_last_error` returns the message.  Tensor ids
 * are the reference's `usize` ids: indices into `Graph.tensors`.  Shapes are size_t arrays.
 */
#ifndef EISEN_GRAPH_H
#define EISEN_GRAPH_H

#include <stddef.h>
#include <stdint.h>

#include "eisen_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct eisen_graph eisen_graph;
typedef struct eisen_lm eisen_lm;
typedef struct eisen_adamw eisen_adamw;

enum { EISEN_PRECISION_FP32 = 0, EISEN_PRECISION_BF16_MIXED = 1 }; /* PrecisionMode, src/graph/mod.rs:48-53 */
#define EISEN_MAX_RANK 8

/* Graph::new(Device::Gpu(ctx, stream)) (src/graph/mod.rs:152-307). */
int eisen_graph_new(eisen_ctx* ctx, int precision, eisen_graph** out);
int eisen_graph_free(eisen_graph* g);
const char* eisen_graph_last_error(eisen_graph* g);

/* Graph::alloc / alloc_pooled / load_tensor_data / mark_params / mark_save_point /
 * restore_save_point / clear_activations / reinterpret_shape / no_grad
 * (src/graph/mod.rs:328-598, src/graph/ops/transform.rs:413-426). */
int eisen_graph_alloc(eisen_graph* g, const size_t* shape, int rank, const float* data, size_t* id_out);
int eisen_graph_alloc_pooled(eisen_graph* g, const size_t* shape, int rank, size_t* id_out);
int eisen_graph_load_tensor_data(eisen_graph* g, size_t id, const float* host, size_t n);
int eisen_graph_mark_params(eisen_graph* g);
int eisen_graph_mark_save_point(eisen_graph* g, size_t* save_point_out);
int eisen_graph_restore_save_point(eisen_graph* g, size_t save_point);
/* restore_save_point that keeps one of the dropped tensors: `keep` (>= save_point) becomes tensor `save_point`
 * (its new id is returned), everything else above the save point goes back to the pool.  The reference's test of the
 * primitives (tests/gpu_kernels.rs:560-610) copies the block output to the host instead; recompute block by block
 * needs it to stay on the device. */
/* Weight gradients over a window of backward passes (no counterpart in the reference, whose Linear backward adds
 * A^T dC to the gradient in every pass, src/graph/ops/linear.rs:279-287).  With backward_passes = n in 2..8 the weight
 * gradients of bf16 Linear layers of at least 16 tiles of 256 x 256 are not formed by the pass that produces their
 * operands: the operands stay allocated (they outlive clear_activations) and one launch per group of equally shaped
 * weights contracts over all passes of the window (eisen_hip_gemm_grouped_ksegments) when the n-th pass ends, or as
 * soon as a parameter's gradient is read, cleared or handed to the optimizer.  The sums are the reference's in another
 * rounding order.  0 or 1 (the default): every pass forms its own.  _flush runs what the window holds now. */
int eisen_graph_set_weight_gradient_window(eisen_graph* g, size_t backward_passes);
/* 1 (the default): without a window, the weight-gradient GEMMs of narrow layers (fewer 128 x 128 tiles than the chip has
 * CUs; bf16 graphs) run on the context's side stream beside the chain of input gradients, their operands kept until
 * the backward pass has ended and the main stream has waited for the side stream.  Same kernels and bits as 0, where
 * every GEMM runs in tape order on the one stream, as in the reference (src/graph/mod.rs:670-796). */
int eisen_graph_set_weight_gradients_beside(eisen_graph* g, int on);
int eisen_graph_flush_weight_gradients(eisen_graph* g);
int eisen_graph_restore_save_point_keep(eisen_graph* g, size_t save_point, size_t keep, size_t* new_id_out);
int eisen_graph_clear_activations(eisen_graph* g);
int eisen_graph_reinterpret_shape(eisen_graph* g, size_t id, const size_t* shape, int rank);
int eisen_graph_set_no_grad(eisen_graph* g, int no_grad);
int eisen_graph_num_tensors(eisen_graph* g, size_t* out);
int eisen_graph_num_params(eisen_graph* g, size_t* out);
int eisen_graph_tape_len(eisen_graph* g, size_t* out);
int eisen_graph_tensor_shape(eisen_graph* g, size_t id, size_t* shape_out, int* rank_out);
/* Tensor::sync_to_cpu / Graph::sync_grad_to_cpu (src/tensor.rs:177-223, src/graph/mod.rs:629-668):
 * n must equal the element count; bf16 storage is widened to f32. */
int eisen_graph_sync_to_cpu(eisen_graph* g, size_t id, float* out, size_t n);
int eisen_graph_sync_grad_to_cpu(eisen_graph* g, size_t id, float* out, size_t n);
/* What the kernels read for tensor `id`, widened to f32: in Bf16Mixed mode the bf16 copy of a parameter that AdamW
 * refreshes next to the f32 master weight (the reference keeps its bf16 weights themselves, alloc_param_bf16,
 * src/graph/mod.rs:567-598); for every other tensor the same values as eisen_graph_sync_to_cpu. */
int eisen_graph_sync_compute_copy_to_cpu(eisen_graph* g, size_t id, float* out, size_t n);
int eisen_graph_synchronize(eisen_graph* g);

/* Ops: one per `impl Graph` method under src/graph/ops/ (file:line at each definition in
 * eisen_amd/csrc/host/graph.cpp).  Each writes the output tensor id. */
int eisen_graph_add(eisen_graph* g, size_t a, size_t b, size_t* out);
int eisen_graph_mul(eisen_graph* g, size_t a, size_t b, size_t* out);
int eisen_graph_silu(eisen_graph* g, size_t a, size_t* out);
int eisen_graph_swiglu(eisen_graph* g, size_t gate, size_t up, size_t* out);
int eisen_graph_matmul(eisen_graph* g, size_t a, size_t b, size_t* out);
int eisen_graph_matmul_trans_b(eisen_graph* g, size_t a, size_t b, size_t* out);
int eisen_graph_bmm(eisen_graph* g, size_t a, size_t b, int trans_b, size_t* out);
int eisen_graph_softmax(eisen_graph* g, size_t a, size_t* out);
/* targets: int64, -1 = IGNORE_INDEX (usize::MAX, src/data/fim.rs:173) for the masked form. */
int eisen_graph_cross_entropy(eisen_graph* g, size_t logits, const int64_t* targets, size_t n_targets, size_t* out);
int eisen_graph_cross_entropy_masked(eisen_graph* g, size_t logits, const int64_t* targets, size_t n_targets, size_t* out);
int eisen_graph_transpose_0213(eisen_graph* g, size_t a, size_t* out);
int eisen_graph_gather(eisen_graph* g, size_t weights, size_t indices, size_t* out);
int eisen_graph_reshape(eisen_graph* g, size_t a, const size_t* shape, int rank, size_t* out);
int eisen_graph_rope(eisen_graph* g, size_t a, size_t head_dim, size_t* out);
int eisen_graph_rms_norm(eisen_graph* g, size_t x, size_t w, float eps, size_t* out);
int eisen_graph_repeat_kv(eisen_graph* g, size_t x, size_t repeats, size_t* out);
int eisen_graph_flash_attention(eisen_graph* g, size_t q, size_t k, size_t v, float scale, int causal, size_t* out);
int eisen_graph_attention_gqa(eisen_graph* g, size_t q, size_t k, size_t v, size_t heads, size_t kv_heads, float scale, int causal,
                              size_t* out);
/* Graph::backward (src/graph/mod.rs:670-796). */
int eisen_graph_backward(eisen_graph* g, size_t loss_id);

/* TransformerLM (src/nn/transformer.rs:70-211).  Parameters are created in the reference's
 * order with the reference's initialisers; load other weights with eisen_graph_load_tensor_data. */
int eisen_lm_new(eisen_graph* g, size_t vocab, size_t hidden, size_t heads, size_t kv_heads, size_t ffn, size_t layers, int tie_weights,
                 eisen_lm** out);
int eisen_lm_free(eisen_lm* lm);
/* Module::params order (src/nn/transformer.rs:57-66, :198-210). */
int eisen_lm_params(eisen_lm* lm, size_t* ids_out, size_t capacity, size_t* count_out);
int eisen_lm_forward(eisen_graph* g, eisen_lm* lm, size_t x_id, size_t* logits_out);
/* 1: fused attention + SwiGLU ops (default); 0: the reference's materialised op chain. */
int eisen_lm_set_fused(eisen_lm* lm, int fused);
/* 1: per-block recompute on mark_save_point / restore_save_point (src/graph/mod.rs:332-365): forward keeps each block's
 * output only, backward re-runs the block before differentiating it.  Gradients are those of the plain step bit for
 * bit; the activation high-water mark drops from all blocks' activations to one block's.  Default 0. */
int eisen_lm_set_checkpointing(eisen_lm* lm, int on);
/* One micro-step of examples/train_llm.rs:433-458 (upload ids, forward, cross entropy, backward,
 * clear_activations).  ids: f32 token ids [mb*seq]; targets int64 [mb*seq].  loss_out may be
 * NULL, in which case nothing synchronises. */
int eisen_lm_micro_step(eisen_graph* g, eisen_lm* lm, const float* ids, const int64_t* targets, size_t micro_batch, size_t seq_len,
                        float* loss_out);

/* AdamW (src/nn/optim.rs). */
int eisen_adamw_new(eisen_graph* g, const size_t* params, size_t n_params, float lr, eisen_adamw** out);
int eisen_adamw_free(eisen_adamw* opt);
int eisen_adamw_config(eisen_adamw* opt, float lr, float beta1, float beta2, float eps, float weight_decay, float grad_clip_norm);
int eisen_adamw_init_moments(eisen_adamw* opt);
int eisen_adamw_zero_grad(eisen_adamw* opt);
int eisen_adamw_clip_grad_norm(eisen_adamw* opt, float max_norm, float* norm_out, float* coef_out);
int eisen_adamw_step(eisen_adamw* opt);
int eisen_adamw_last_grad_norm(eisen_adamw* opt, float* norm_out, float* scale_out);
/* Moments of the i-th parameter, copied to the host (tests). */
int eisen_adamw_moments_to_cpu(eisen_adamw* opt, size_t i, float* m_out, float* v_out, size_t n);
/* CosineScheduler::get_lr (src/nn/scheduler.rs:45-55). */
float eisen_cosine_lr(float lr_max, float lr_min, size_t warmup_steps, size_t total_steps, size_t step);

/* ---- data in, weights out ------------------------------------------------------------------- */

/* BinaryDataLoader (src/data/dataloader.rs:84-203), without fill-in-the-middle: a file of
 * little-endian u16 token ids cut into windows of seq_len+1 tokens.  next_batch fills x (token ids as
 * f32, [batch*seq]) and targets (the next token, [batch*seq]) and sets *got to 1, or sets it to 0 when
 * the stream is exhausted (the reference returns None).  The refill pattern of the reference's 4 MiB
 * BufReader is reproduced, so the two hand out the same batches and stop at the same one. */
typedef struct eisen_data_loader eisen_data_loader;
int eisen_data_loader_open(const char* path, size_t seq_len, size_t batch_size, eisen_data_loader** out);
int eisen_data_loader_close(eisen_data_loader* dl);
int eisen_data_loader_total_batches(eisen_data_loader* dl, size_t* out);
int eisen_data_loader_next_batch(eisen_data_loader* dl, float* x, int64_t* targets, int* got);
int eisen_data_loader_reset(eisen_data_loader* dl);
/* Message of the last failed eisen_data_loader_* / eisen_write_llama_config call of this thread. */
const char* eisen_io_last_error(void);

/* save_weights (examples/train_llm.rs:93-105): parameter tensors in id order, raw f32 LE. */
int eisen_graph_save_weights(eisen_graph* g, const char* path);
/* load_weights (examples/chat_cli.rs:161-180): consecutive f32 runs, one per id; floats_out may be NULL. */
int eisen_graph_load_weights(eisen_graph* g, const size_t* params, size_t n_params, const char* path, size_t* floats_out);
/* write_safetensors over TransformerLM::named_params (src/tools/huggingface.rs:88-146,
 * src/nn/transformer.rs:119-172): F32, linear weights transposed to [out, in]. */
int eisen_lm_write_safetensors(eisen_graph* g, eisen_lm* lm, const char* path);
/* write_llama_config (src/tools/huggingface.rs:38-84); num_key_value_heads is written as given
 * (the reference repeats num_attention_heads there). */
int eisen_write_llama_config(const char* path, size_t vocab, size_t hidden, size_t ffn, size_t layers, size_t heads, size_t kv_heads,
                             size_t max_position_embeddings, float rms_norm_eps, float rope_theta, int tie_word_embeddings);

#ifdef __cplusplus
}
#endif
#endif /* EISEN_GRAPH_H */
