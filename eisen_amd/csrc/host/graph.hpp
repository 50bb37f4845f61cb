// Host side of the Device::Gpu backend: Graph / Tensor / Tape with the reference's operator
// interface (src/graph/mod.rs, src/graph/ops/*.rs, src/tensor.rs, src/tape.rs), written against
// the public C-ABI of include/eisen_hip.h only -- every device action below is one eisen_hip_* call.
//
// Differences from the reference that a caller can observe are limited to what its GPU arm
// could not do: attention and SwiGLU have fused ops with gradients, activation gradients are
// bf16 in mixed mode, parameters keep f32 master weights next to a bf16 copy, and nothing
// synchronises the stream unless the caller reads a value back.
#pragma once
#include <utility>
#include <cstdint>
#include <functional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "eisen_hip.h"

namespace eisen {

// src/graph/mod.rs:48-53
enum class PrecisionMode { Fp32 = 0, Bf16Mixed = 1 };

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// src/tensor.rs:35-44 `Storage`: one device allocation and its element type.
struct Storage {
    void* ptr = nullptr;
    size_t numel = 0;
    int dtype = EISEN_F32;
    bool valid() const { return ptr != nullptr; }
};

// src/tensor.rs:132-142 `Tensor` (public fields are API: shape/strides/data/grad/name/is_pooled).
struct Tensor {
    size_t id = 0;
    std::vector<size_t> shape, strides;
    Storage data;            // activations: f32 or bf16; parameters: f32 master
    Storage grad;            // parameters: f32, allocated with the tensor; activations: lazily, activation dtype
    Storage shadow;          // parameters in Bf16Mixed: bf16 copy of `data` the kernels read
    std::string name;
    bool is_pooled = false;
    bool is_param = false;        // allocated through alloc()/alloc_param_bf16(): owns an f32 grad
    bool grad_written = false;    // this backward pass already stored into grad (next store accumulates)
    bool grad_borrowed = false;   // grad's buffer now belongs to another tensor's grad (see matmul_residual): not freed with this one
    bool grad_zero_pending = false;  // zero_grad() was requested; materialised on first use
    std::vector<float> host_copy;    // kept for small host-loaded tensors (token ids)
    size_t size() const {
        size_t n = 1;
        for (size_t s : shape) n *= s;
        return n;
    }
};

class Graph;

// src/tape.rs:3-7
struct TapeNode {
    std::vector<size_t> inputs;
    size_t output;
    std::function<void(Graph&)> backward_fn;
};
struct Tape {
    std::vector<TapeNode> nodes;
};

class Graph {
   public:
    std::vector<Tensor> tensors;
    Tape tape;
    size_t num_params = 0;
    bool no_grad = false;
    // Like no_grad for the tape only: ops record nothing but still choose the kernels of a training forward pass (no_grad
    // also switches attention to the inference path, src/nn/attention.rs:335-336, whose bits differ from the chain's).
    bool tape_paused = false;
    PrecisionMode precision_mode;

    Graph(eisen_ctx* ctx, PrecisionMode mode);
    ~Graph();
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;

    eisen_ctx* ctx() const { return ctx_; }
    int act_dtype() const { return precision_mode == PrecisionMode::Bf16Mixed ? EISEN_BF16 : EISEN_F32; }
    bool uses_bf16_mixed_precision() const { return precision_mode == PrecisionMode::Bf16Mixed; }

    // ---- runtime (src/graph/mod.rs:317-598) ------------------------------------------------
    void name_tensor(size_t id, const std::string& name) { at(id).name = name; }
    void mark_params() { num_params = tensors.size(); }
    size_t mark_save_point() const { return tensors.size(); }
    void restore_save_point(size_t save_point);
    // restore_save_point that lets one of the dropped tensors live on: `keep` (>= save_point) becomes tensor
    // `save_point`, everything else above the save point is released.  Returns the new id.  (The reference's test of the
    // primitives, tests/gpu_kernels.rs:560-610, copies the value out instead; a block-by-block recompute needs it on the
    // device.)
    size_t restore_save_point_keep(size_t save_point, size_t keep);
    void clear_activations();
    size_t alloc(const std::vector<size_t>& shape, const std::vector<float>& data);
    size_t alloc(const std::vector<size_t>& shape, const float* data, size_t n);
    size_t alloc_pooled(const std::vector<size_t>& shape);
    size_t alloc_pooled_dtype(const std::vector<size_t>& shape, int dtype);   // pooled buffer of an explicit element type
    size_t alloc_param_bf16(const std::vector<size_t>& shape, const std::vector<float>& data) { return alloc(shape, data); }
    void load_tensor_data(size_t id, const float* host, size_t n);
    std::vector<float> sync_to_cpu(size_t id);
    std::vector<float> sync_grad_to_cpu(size_t id);
    std::vector<float> sync_compute_copy_to_cpu(size_t id);   // the bf16 copy kernels read (mixed-mode parameters), widened
    void reinterpret_shape(size_t id, const std::vector<size_t>& shape);
    void synchronize();

    // ---- ops (src/graph/ops/*.rs); all return the output tensor id ------------------------------
    size_t add(size_t a, size_t b);
    size_t mul(size_t a, size_t b);
    size_t silu(size_t a);
    size_t swiglu(size_t gate, size_t up);                      // fused silu(gate) * up
    size_t matmul(size_t a, size_t b);
    // r + a b in one kernel.  defer_dw: the weight gradient is left for the matmul_group whose `collect_dw` names b (it
    // runs later in backward and puts b's gradient GEMM into the same launch as its own); backward() fails loudly if
    // nobody collects it
    size_t matmul_residual(size_t a, size_t b, size_t r, bool defer_dw = false);
    // r + (silu(gate) * up) b; backward forms dgate, dup in the dX GEMM.  h: silu(gate) * up where a matmul_group has
    // already formed it.
    size_t swiglu_matmul_residual(size_t gate, size_t up, size_t b, size_t r, size_t h = (size_t)-1);
    // matmuls of one input against 2-3 weights with fewer launches (bf16 graphs; otherwise plain matmuls).
    // collect_dw: weights whose deferred gradient GEMMs join this group's dW launch; defer_dw: this group's own weight
    // gradients are left for a later group that names them; swiglu_h: receives the id of silu(out0) * out1 when the
    // kernel that forms it with the two products ran, (size_t)-1 otherwise
    // rope_members / rope_head_dim / rotated: the first rope_members outputs may leave rotary-embedded (`rope` applied to
    // a [batch, seq, hidden] product by the kernel that forms it); *rotated says whether they did.  Such an output stands for
    // rope(a w): its consumer (attention_gqa_rope with prerotated) leaves the gradient of the un-rotated product a w in its
    // gradient buffer, which is what this group's backward multiplies.
    std::vector<size_t> matmul_group(size_t a, const std::vector<size_t>& weights, const std::vector<size_t>& collect_dw = {}, size_t* swiglu_h = nullptr,
                                     bool defer_dw = false, size_t rope_members = 0, size_t rope_head_dim = 0, bool* rotated = nullptr);
    size_t matmul_bf16(size_t a, size_t b) { return matmul(a, b); }
    size_t matmul_trans_b(size_t a, size_t b);
    size_t bmm(size_t a, size_t b, bool trans_b);
    size_t softmax(size_t a);
    size_t cross_entropy(size_t logits, const std::vector<int64_t>& targets);
    size_t cross_entropy_masked(size_t logits, const std::vector<int64_t>& targets);
    size_t transpose_0213(size_t a);
    size_t gather(size_t weights, size_t indices);
    size_t reshape(size_t a, const std::vector<size_t>& shape);
    size_t rope(size_t a, size_t head_dim);
    size_t rms_norm(size_t x, size_t w, float eps);
    size_t repeat_kv(size_t x, size_t repeats);
    // Reference signature (src/graph/ops/attention.rs:7-14): q [B,M,D], k/v [B,N,D], M == N here.
    // Unlike the reference it also records a backward.
    size_t flash_attention(size_t q, size_t k, size_t v, float scale, bool causal);
    // q [B,S,Hq*hd], k/v [B,S,Hkv*hd] straight from the projections -> [B,S,Hq*hd].
    size_t attention_gqa(size_t q, size_t k, size_t v, size_t heads, size_t kv_heads, float scale, bool causal);
    // the same with the rotary embedding of q and k inside: rope(q), rope(k) -> attention; backward stores d q, d k un-rotated
    // prerotated: q and k already are rope(q0), rope(k0) (matmul_group with *rotated); d q0, d k0 are stored all the same
    size_t attention_gqa_rope(size_t q, size_t k, size_t v, size_t heads, size_t kv_heads, float scale, bool causal, bool prerotated = false);

    // src/graph/mod.rs:670-796
    void backward(size_t loss_id);
    // Replays tape nodes [first_node, end) in reverse, as backward() does for the whole tape: for a backward closure that
    // recorded more nodes (a recomputed block) and now differentiates through them.
    void backward_nodes_from(size_t first_node);

    // ---- helpers for optimisers and backward closures -----------------------------------------
    Tensor& at(size_t id);
    // Gradient buffer of `id` for a store; *accumulate tells the kernel whether to add.  add_from: a caller that can read
    // what it adds to from another buffer than the one it writes passes this; it receives that buffer (the returned one
    // itself unless the gradient's present content has to stay as it is for a weight-gradient GEMM that has not run yet,
    // see set_weight_gradient_window: then the store goes to a fresh buffer, and a caller without add_from gets the old
    // content copied there first).
    Storage& grad_for_write(size_t id, int* accumulate, const void** add_from = nullptr);
    // Gradient as an input (must have been written).
    const Storage& grad_for_read(size_t id);
    void materialize_grad(size_t id);      // before a gradient is read: run what the weight-gradient window holds, apply a pending zero_grad
    void apply_pending_zero(size_t id);    // the pending zero_grad alone (for a store that touches part of the buffer)
    void request_zero_grad(size_t id);     // AdamW::zero_grad, lazily
    const Storage& compute_data(size_t id);   // what kernels read: bf16 shadow for mixed-mode params
    void refresh_shadow(size_t id);           // re-cast the master weight into the bf16 copy
    void check(int rc, const char* what) const;
    size_t backward_root() const { return backward_root_; }
    size_t backward_epoch() const { return backward_epoch_; }  // counts backward() calls
    bool has_grad(size_t id) { const Tensor& t = at(id); return t.is_param || (t.grad.valid() && t.grad_written); }
    // A weight-gradient GEMM dW (+)= x^T dy left for a later node of the same backward pass (see matmul_residual)
    struct PendingDW {
        size_t weight;
        const void* x;    // [rows, in] activations the weight multiplied
        const void* dy;   // [rows, out] gradient of the product
        size_t rows, in, out;
    };
    std::vector<PendingDW> pending_dw;
    // buffers that GEMMs on the context's side stream are still reading: the first node that asks to write one of them waits
    // for those GEMMs
    std::vector<const void*> side_guards;
    // gain gradients of RMSNorm nodes left as partial rows during a backward pass; one launch finishes them all at its end
    struct PendingNormDW {
        Storage partial;
        size_t weight, nrows, dim;
        bool assign;   // the gain's gradient was waiting to be cleared: the finishing launch overwrites it instead
    };
    std::vector<PendingNormDW> pending_norm_dw;
    void flush_norm_dw(bool compute);
    void side_join();

    // ---- weight gradients over a window of micro-batches ---------------------------------------------------
    // The reference forms a Linear layer's weight gradient in the backward pass of every micro-batch and adds it to the
    // f32 gradient (src/graph/ops/linear.rs:279-287; examples/train_llm.rs:386-477 runs 8 such passes per optimizer step).
    // With a window of n > 1 backward passes the product is left for later instead (bf16 graphs, weights of whole
    // 256 x 256 tiles): the activations and the output gradient stay where the passes left them -- their buffers outlive
    // clear_activations, and a gradient buffer that a later node would add to in place is replaced by a fresh one -- and
    // one launch per group of equally shaped weights contracts over all the micro-batches of the window
    // (eisen_hip_gemm_grouped_ksegments): each gradient is read and written once per window.  The launches run when
    // the n-th pass ends, and before anything reads, clears or scales a parameter's gradient; what a caller can observe
    // is the reference's sum in a different rounding order (one f32 accumulation over all tokens of the window).
    // The price is memory: the operands of every windowed product of every pass in the window stay allocated.
    // Without a window, the weight-gradient GEMMs of narrow layers (each too small to fill the chip) run on the context's
    // side stream beside the chain of input gradients, which never waits for them: their operands are kept as above
    // (a gradient buffer that a later node adds to in place is replaced by a fresh one) until the backward pass ends
    // and the main stream has waited for the side stream.  Same kernels, same bits.  On by default.
    void set_weight_gradients_beside(bool on) { beside_ = on; }
    void set_weight_gradient_window(size_t backward_passes);
    size_t weight_gradient_window() const { return window_; }
    void flush_weight_gradients(size_t only_weight = (size_t)-1);
    struct WindowDW {
        size_t weight, rows, in, out;
        std::vector<const void*> x, dy;  // one pair per piece, in the order the passes ran
    };
    std::vector<WindowDW> window_dw;

   private:
    eisen_ctx* ctx_;
    size_t backward_root_ = (size_t)-1;
    size_t backward_epoch_ = 0;
    size_t window_ = 0, window_passes_ = 0;
    bool beside_ = true, in_beside_ = false;
    std::vector<size_t> side_written_;  // parameters whose gradients the side stream is writing: the main stream waits before it touches them
    // Runs `launch` (weight-gradient GEMMs reading `reads`, writing the gradients of `weights`) on the side stream when
    // the products are small and no window is set, on the current stream otherwise.
    bool beside_fits(size_t in, size_t out) const;
    void run_beside(bool beside, const std::vector<const void*>& reads, const std::vector<size_t>& weights, const std::function<int()>& launch, const char* what);
    void release_retained();
    // buffers a windowed weight-gradient GEMM will read -> whether their owner has released them (then the flush frees them)
    std::unordered_map<const void*, bool> retained_;
    // the product x^T dy joins the window when it can; false: the caller forms it now
    bool window_take(size_t weight, const void* x, const void* dy, int dtype, size_t rows, size_t in, size_t out);
    bool window_fits(size_t weight, int dtype, size_t rows, size_t in, size_t out);
    void free_buffer(void* ptr);  // eisen_hip_free unless the buffer is retained
    size_t push_tensor(const std::vector<size_t>& shape, int dtype, bool pooled);
    Storage device_alloc(size_t numel, int dtype, bool zero);
    void device_free(Storage& s);
    void release(Tensor& t);
    void record(std::vector<size_t> inputs, size_t output, std::function<void(Graph&)> fn);
    size_t elementwise_binary(size_t a, size_t b, bool is_mul);
    size_t attention_impl(size_t q, size_t k, size_t v, size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd, const long long* qs,
                          const long long* ks, float scale, bool causal, const std::vector<size_t>& out_shape);
};

std::vector<size_t> compute_strides(const std::vector<size_t>& shape);                      // src/tensor.rs:225-233
std::vector<size_t> broadcasted_shape(const std::vector<size_t>& a, const std::vector<size_t>& b);  // :235-244
std::vector<size_t> broadcasted_strides(const std::vector<size_t>& shape, const std::vector<size_t>& base,
                                        const std::vector<size_t>& out_shape);              // :246-260

}  // namespace eisen
