// nn modules and the optimiser over Graph, with the reference's interface (src/nn/*.rs).
#pragma once
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "graph.hpp"

namespace eisen {

// src/nn/mod.rs:12-18
struct Module {
    virtual ~Module() = default;
    virtual size_t forward(Graph& g, size_t x_id) const = 0;
    virtual std::vector<size_t> params() const = 0;
};

// src/nn/linear.rs: weight [in, out], Y = X W (+ b); N(0, 0.02) from a fixed LCG + Box-Muller.
struct Linear : Module {
    size_t weight_id = 0;
    bool has_bias = false;
    size_t bias_id = 0;
    Linear() = default;
    Linear(Graph& g, size_t in_features, size_t out_features, bool use_bias);
    size_t forward(Graph& g, size_t x_id) const override;
    std::vector<size_t> params() const override;
};

// src/nn/embedding.rs: uniform(-0.02, 0.02) from a fixed LCG.
struct Embedding : Module {
    size_t weight_id = 0;
    Embedding() = default;
    Embedding(Graph& g, size_t vocab_size, size_t hidden_dim);
    size_t forward(Graph& g, size_t x_id) const override { return g.gather(weight_id, x_id); }
    std::vector<size_t> params() const override { return {weight_id}; }
};

// src/nn/rmsnorm.rs
struct RMSNorm : Module {
    size_t weight_id = 0;
    float eps = 1e-5f;
    RMSNorm() = default;
    RMSNorm(Graph& g, size_t dim, float eps);
    size_t forward(Graph& g, size_t x_id) const override { return g.rms_norm(x_id, weight_id, eps); }
    std::vector<size_t> params() const override { return {weight_id}; }
};

// src/nn/attention.rs:251-404.  MultiHeadAttention (:100-249) is the num_kv_heads == num_heads case.
struct GroupedQueryAttention : Module {
    size_t num_heads = 0, num_kv_heads = 0, head_dim = 0, hidden_dim = 0;
    Linear q_proj, k_proj, v_proj, out_proj;
    // false: the reference's materialised chain (reshape/transpose/repeat_kv/bmm/mul/add/softmax/bmm),
    // true (default): the fused attention op.  Both give the same function and gradients.
    bool fused = true;
    GroupedQueryAttention() = default;
    GroupedQueryAttention(Graph& g, size_t hidden_dim, size_t num_heads, size_t num_kv_heads);
    // residual != npos (fused path only): the output projection also adds this tensor, i.e. the result is
    // residual + attention(x) as the transformer block computes it
    // residual: added by the output projection's kernel.  collect_dw: weights of later layers of the same block whose
    // deferred gradient GEMMs join the Q/K/V group's launch; collects() says whether this call would take them.
    size_t forward_with_mask(Graph& g, size_t x_id, bool causal, size_t residual = (size_t)-1, const std::vector<size_t>& collect_dw = {}) const;
    bool collects() const { return fused && !q_proj.has_bias && !k_proj.has_bias && !v_proj.has_bias; }
    size_t forward(Graph& g, size_t x_id) const override { return forward_with_mask(g, x_id, true); }
    std::vector<size_t> params() const override;
};

// src/nn/transformer.rs:8-68
struct TransformerBlock : Module {
    RMSNorm norm1;
    GroupedQueryAttention attn;
    RMSNorm norm2;
    Linear ffn1, ffn2, ffn_gate;
    TransformerBlock() = default;
    TransformerBlock(Graph& g, size_t hidden_dim, size_t num_heads, size_t num_kv_heads, size_t ffn_dim);
    size_t forward_with_mask(Graph& g, size_t x_id, bool causal) const;
    size_t forward(Graph& g, size_t x_id) const override { return forward_with_mask(g, x_id, true); }
    std::vector<size_t> params() const override;
};

// src/nn/transformer.rs:70-211
struct TransformerLM : Module {
    Embedding token_emb;
    std::vector<TransformerBlock> blocks;
    RMSNorm norm_f;
    Linear lm_head;
    bool tie_weights = false;
    size_t vocab_size = 0;
    TransformerLM(Graph& g, size_t vocab_size, size_t hidden_dim, size_t num_heads, size_t num_kv_heads, size_t ffn_dim, size_t num_layers,
                  bool tie_weights);
    std::vector<std::pair<std::string, size_t>> named_params() const;
    void tag_parameters(Graph& g) const;
    void set_fused(bool fused);
    // Per-block recompute on the save-point primitives (src/graph/mod.rs:332-365, exercised block-wise by
    // tests/gpu_kernels.rs:560-610): forward() runs each block without a tape and keeps only its output; backward re-runs
    // the block from its input, differentiates it and drops its activations again.  Same gradients, bit for bit.
    bool checkpointing = false;
    void set_checkpointing(bool on) { checkpointing = on; }
    size_t forward(Graph& g, size_t x_id) const override;
    std::vector<size_t> params() const override;
};

// src/nn/optim.rs
class AdamW {
   public:
    std::vector<size_t> params;
    float lr, beta1 = 0.9f, beta2 = 0.999f, eps = 1e-8f, weight_decay = 0.01f;
    AdamW(Graph& g, std::vector<size_t> params, float lr);
    ~AdamW();
    void set_grad_clip_norm(float max_norm) {
        if (max_norm > 0.0f) grad_clip_norm_ = max_norm;
    }
    float last_grad_norm();   // reads the value back from the device
    float last_grad_scale();
    size_t step_count() const { return t_; }
    void init_moments();
    void zero_grad();
    std::pair<float, float> clip_grad_norm(float max_norm);
    void step();
    const Storage& moment_m(size_t i) const { return m_[i]; }
    const Storage& moment_v(size_t i) const { return v_[i]; }

   private:
    Graph& g_;
    size_t t_ = 0;
    std::vector<Storage> m_, v_;
    float grad_clip_norm_ = 0.0f;
    float* norm_dev_ = nullptr;  // [norm, clip coefficient] on the device
    bool norm_valid_ = false;
    std::vector<eisen_param_slot> slots();
};

// src/nn/scheduler.rs
struct CosineScheduler {
    float lr_max, lr_min;
    size_t warmup_steps, total_steps;
    float get_lr(size_t step) const;
};

// One micro-step of examples/train_llm.rs:433-458: ids -> forward -> cross entropy -> backward ->
// clear_activations.  Returns the id-free loss value only when `loss_out` is given (forces a sync).
void lm_micro_step(Graph& g, const TransformerLM& lm, const float* ids, const int64_t* targets, size_t micro_batch, size_t seq_len,
                   float* loss_out);

}  // namespace eisen
