#include "nn.hpp"

#include <cmath>
#include <cstring>

namespace eisen {

namespace {
// f32::powi -> compiler-rt __powisf2 (square and multiply), as AdamW::step uses it (src/nn/optim.rs:337-338).
float powi_f32(float a, int b) {
    const bool recip = b < 0;
    float r = 1.0f;
    while (true) {
        if (b & 1) r *= a;
        b /= 2;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0f / r : r;
}
}  // namespace

// Linear::new (src/nn/linear.rs:10-50): the same seed-42 LCG for every layer.
Linear::Linear(Graph& g, size_t in_features, size_t out_features, bool use_bias) {
    const size_t n = in_features * out_features;
    std::vector<float> w(n);
    const float stdv = 0.02f;
    uint32_t seed = 42;
    const float umax = (float)UINT32_MAX;
    for (size_t i = 0; i < n; i++) {
        const float u1 = std::fmin((float)seed / umax + 1e-7f, 1.0f - 1e-7f);
        seed = seed * 1664525u + 1013904223u;
        const float u2 = std::fmin(std::fmax((float)seed / umax, 1e-7f), 1.0f - 1e-7f);
        seed = seed * 1664525u + 1013904223u;
        const float mag = std::sqrt(-2.0f * std::log(u1));
        w[i] = mag * std::cos(2.0f * 3.14159274101257324f * u2) * stdv;
    }
    weight_id = g.alloc({in_features, out_features}, w);
    has_bias = use_bias;
    if (use_bias) bias_id = g.alloc({out_features}, std::vector<float>(out_features, 0.0f));
}

// Linear::forward (src/nn/linear.rs:53-95): matmul over flattened rows, 3-D shape restored.
size_t Linear::forward(Graph& g, size_t x_id) const {
    const std::vector<size_t> xs = g.at(x_id).shape;
    size_t out = g.matmul(x_id, weight_id);
    if (has_bias) out = g.add(out, bias_id);
    if (xs.size() == 3) g.reinterpret_shape(out, {xs[0], xs[1], g.at(weight_id).shape[1]});
    return out;
}
std::vector<size_t> Linear::params() const {
    std::vector<size_t> p{weight_id};
    if (has_bias) p.push_back(bias_id);
    return p;
}

// Embedding::new (src/nn/embedding.rs:9-31)
Embedding::Embedding(Graph& g, size_t vocab_size, size_t hidden_dim) {
    const size_t n = vocab_size * hidden_dim;
    std::vector<float> w(n);
    uint32_t seed = 84;
    const float umax = (float)UINT32_MAX;
    for (size_t i = 0; i < n; i++) {
        seed = seed * 1664525u + 1013904223u;
        w[i] = ((float)seed / umax * 2.0f - 1.0f) * 0.02f;
    }
    weight_id = g.alloc({vocab_size, hidden_dim}, w);
}

RMSNorm::RMSNorm(Graph& g, size_t dim, float eps_) : eps(eps_) { weight_id = g.alloc({dim}, std::vector<float>(dim, 1.0f)); }

GroupedQueryAttention::GroupedQueryAttention(Graph& g, size_t hidden, size_t heads, size_t kv_heads) {
    if (hidden % heads) throw Error("hidden_dim must be cleanly divisible by num_heads");
    if (heads % kv_heads) throw Error("num_heads must be divisible by num_kv_heads");
    num_heads = heads;
    num_kv_heads = kv_heads;
    head_dim = hidden / heads;
    hidden_dim = hidden;
    const size_t kv_dim = kv_heads * head_dim;
    q_proj = Linear(g, hidden, hidden, false);
    k_proj = Linear(g, hidden, kv_dim, false);
    v_proj = Linear(g, hidden, kv_dim, false);
    out_proj = Linear(g, hidden, hidden, false);
}

// GroupedQueryAttention::forward_with_mask (src/nn/attention.rs:289-388).
size_t GroupedQueryAttention::forward_with_mask(Graph& g, size_t x_id, bool causal, size_t residual, const std::vector<size_t>& collect_dw) const {
    const std::vector<size_t> xs = g.at(x_id).shape;
    if (xs.size() != 3) throw Error("GQA requires [Batch, Seq, Dim]");
    const size_t batch = xs[0], seq = xs[1];
    size_t q, k, v;
    bool rotated = false;  // q and k left their projection kernels rotary-embedded
    if (collects()) {
        // the three projections read the same input: K and V as one launch, one input-gradient GEMM for all
        // (the group also collects the output projection's weight gradient when that projection defers it: four dW GEMMs, one launch)
        const bool defer_out = residual != (size_t)-1 && !out_proj.has_bias;
        std::vector<size_t> collect = collect_dw;
        if (defer_out) collect.insert(collect.begin(), out_proj.weight_id);
        const bool kernel_attention = fused && (!g.uses_bf16_mixed_precision() || head_dim == 32 || head_dim == 64 || head_dim == 128);
        const std::vector<size_t> qkv = g.matmul_group(x_id, {q_proj.weight_id, k_proj.weight_id, v_proj.weight_id}, collect, nullptr, false,
                                                       kernel_attention ? 2 : 0, head_dim, &rotated);
        q = qkv[0]; k = qkv[1]; v = qkv[2];
        for (size_t t : qkv) g.reinterpret_shape(t, {batch, seq, g.at(t).shape.back()});
    } else {
        q = q_proj.forward(g, x_id);
        k = k_proj.forward(g, x_id);
        v = v_proj.forward(g, x_id);
    }
    const float scale = 1.0f / std::sqrt((float)head_dim);
    // the bf16 MFMA attention kernels exist for head_dim 32, 64 and 128; other head dims in mixed precision take the
    // reference's materialised chain below (any head_dim), like every f32 graph may
    const bool kernel_head_dim = !g.uses_bf16_mixed_precision() || head_dim == 32 || head_dim == 64 || head_dim == 128;
    const bool fused_attention = fused && kernel_head_dim;
    size_t ctx_flat;
    if (fused_attention) {
        // one op for the rotary embedding and steps 3-11: head split, GQA repeat, scores, scale, mask, softmax, P V, merge
        ctx_flat = g.attention_gqa_rope(q, k, v, num_heads, num_kv_heads, scale, causal, rotated);
    } else {
        const size_t q_rope = g.rope(q, head_dim), k_rope = g.rope(k, head_dim);
        const size_t q4 = g.reshape(q_rope, {batch, seq, num_heads, head_dim});
        const size_t k4 = g.reshape(k_rope, {batch, seq, num_kv_heads, head_dim});
        const size_t v4 = g.reshape(v, {batch, seq, num_kv_heads, head_dim});
        const size_t qt = g.transpose_0213(q4), kt = g.transpose_0213(k4), vt = g.transpose_0213(v4);
        const size_t repeats = num_heads / num_kv_heads;
        const size_t kr = g.repeat_kv(kt, repeats), vr = g.repeat_kv(vt, repeats);
        const size_t bh = batch * num_heads;
        g.reinterpret_shape(qt, {bh, seq, head_dim});
        g.reinterpret_shape(kr, {bh, seq, head_dim});
        g.reinterpret_shape(vr, {bh, seq, head_dim});
        size_t ctx;
        if (g.no_grad && kernel_head_dim) {
            ctx = g.flash_attention(qt, kr, vr, scale, causal);
        } else {
            const size_t scores = g.bmm(qt, kr, true);
            // the reference uploads a full [bh, seq, seq] tensor of `scale`; a broadcast scalar is the same product
            const size_t scale_id = g.alloc_pooled({1});
            g.load_tensor_data(scale_id, &scale, 1);
            size_t scaled = g.mul(scores, scale_id);
            if (causal) {
                std::vector<float> mask(seq * seq, 0.0f);
                for (size_t r = 0; r < seq; r++)
                    for (size_t c = r + 1; c < seq; c++) mask[r * seq + c] = -1e20f;
                const size_t mask_id = g.alloc_pooled({1, seq, seq});
                g.load_tensor_data(mask_id, mask.data(), mask.size());
                scaled = g.add(scaled, mask_id);
            }
            ctx = g.bmm(g.softmax(scaled), vr, false);
        }
        g.reinterpret_shape(ctx, {batch, num_heads, seq, head_dim});
        const size_t ctx_t = g.transpose_0213(ctx);
        ctx_flat = g.reshape(ctx_t, {batch, seq, hidden_dim});
    }
    if (fused && residual != (size_t)-1 && !out_proj.has_bias)
        return g.matmul_residual(ctx_flat, out_proj.weight_id, residual, /*defer_dw=*/collects());
    return out_proj.forward(g, ctx_flat);
}
std::vector<size_t> GroupedQueryAttention::params() const {
    return {q_proj.weight_id, k_proj.weight_id, v_proj.weight_id, out_proj.weight_id};
}

// TransformerBlock::new (src/nn/transformer.rs:19-28): allocation order norm1, attn, norm2, gate, ffn1, ffn2.
TransformerBlock::TransformerBlock(Graph& g, size_t hidden, size_t heads, size_t kv_heads, size_t ffn_dim) {
    norm1 = RMSNorm(g, hidden, 1e-5f);
    attn = GroupedQueryAttention(g, hidden, heads, kv_heads);
    norm2 = RMSNorm(g, hidden, 1e-5f);
    ffn_gate = Linear(g, hidden, ffn_dim, false);
    ffn1 = Linear(g, hidden, ffn_dim, false);
    ffn2 = Linear(g, ffn_dim, hidden, false);
}

// TransformerBlock::forward_with_mask (src/nn/transformer.rs:31-49).
size_t TransformerBlock::forward_with_mask(Graph& g, size_t x_id, bool causal) const {
    const size_t norm1_out = norm1.forward(g, x_id);
    size_t res1;
    bool defer_ffn = false;
    if (attn.fused && !attn.out_proj.has_bias) {
        // the output projection adds the residual itself; the weight gradients of gate and up wait for the Q/K/V group
        defer_ffn = attn.collects() && !ffn_gate.has_bias && !ffn1.has_bias;
        res1 = attn.forward_with_mask(g, norm1_out, causal, x_id, defer_ffn ? std::vector<size_t>{ffn_gate.weight_id, ffn1.weight_id} : std::vector<size_t>{});
    } else {
        const size_t attn_out = attn.forward_with_mask(g, norm1_out, causal);
        res1 = g.add(x_id, attn_out);
    }
    const size_t norm2_out = norm2.forward(g, res1);
    size_t gated;
    size_t gate_id = (size_t)-1, up_id = (size_t)-1, h_id = (size_t)-1;  // set when gate and up are available unfused-multiplied (SwiGLU folded into the down projection node)
    if (attn.fused && !ffn_gate.has_bias && !ffn1.has_bias) {
        // gate and up projections as one launch that also forms silu(gate) * up where the down projection consumes it
        const std::vector<size_t> guv = g.matmul_group(norm2_out, {ffn_gate.weight_id, ffn1.weight_id}, {}, !ffn2.has_bias ? &h_id : nullptr, defer_ffn);
        const std::pair<size_t, size_t> gu{guv[0], guv[1]};
        const std::vector<size_t> ns = g.at(norm2_out).shape;
        if (ns.size() == 3) {
            const size_t f = g.at(ffn_gate.weight_id).shape[1];
            g.reinterpret_shape(gu.first, {ns[0], ns[1], f});
            g.reinterpret_shape(gu.second, {ns[0], ns[1], f});
        }
        if (!ffn2.has_bias) {
            gate_id = gu.first;
            up_id = gu.second;
            gated = (size_t)-1;
        } else {
            gated = g.swiglu(gu.first, gu.second);
        }
    } else if (attn.fused) {
        const size_t gate_out = ffn_gate.forward(g, norm2_out);
        const size_t up = ffn1.forward(g, norm2_out);
        gated = g.swiglu(gate_out, up);
    } else {
        const size_t gate_out = ffn_gate.forward(g, norm2_out);
        const size_t gate = g.silu(gate_out);
        const size_t up = ffn1.forward(g, norm2_out);
        gated = g.mul(gate, up);
    }
    if (gate_id != (size_t)-1) return g.swiglu_matmul_residual(gate_id, up_id, ffn2.weight_id, res1, h_id);  // SwiGLU + down projection + residual
    if (attn.fused && !ffn2.has_bias) return g.matmul_residual(gated, ffn2.weight_id, res1);  // down projection + residual
    const size_t ffn2_out = ffn2.forward(g, gated);
    return g.add(res1, ffn2_out);
}
// params order (src/nn/transformer.rs:57-66): norm1, attn, norm2, ffn1, ffn2, ffn_gate
std::vector<size_t> TransformerBlock::params() const {
    std::vector<size_t> p{norm1.weight_id};
    for (size_t id : attn.params()) p.push_back(id);
    p.push_back(norm2.weight_id);
    p.push_back(ffn1.weight_id);
    p.push_back(ffn2.weight_id);
    p.push_back(ffn_gate.weight_id);
    return p;
}

// TransformerLM::new (src/nn/transformer.rs:78-117); nothing is demoted to the host here.
TransformerLM::TransformerLM(Graph& g, size_t vocab, size_t hidden, size_t heads, size_t kv_heads, size_t ffn_dim, size_t layers, bool tie)
    : tie_weights(tie), vocab_size(vocab) {
    token_emb = Embedding(g, vocab, hidden);
    blocks.reserve(layers);
    for (size_t l = 0; l < layers; l++) blocks.emplace_back(g, hidden, heads, kv_heads, ffn_dim);
    norm_f = RMSNorm(g, hidden, 1e-5f);
    if (tie) {
        lm_head.weight_id = token_emb.weight_id;
        lm_head.has_bias = false;
    } else {
        lm_head = Linear(g, hidden, vocab, false);
    }
}

std::vector<std::pair<std::string, size_t>> TransformerLM::named_params() const {
    std::vector<std::pair<std::string, size_t>> out;
    out.emplace_back("model.embed_tokens.weight", token_emb.weight_id);
    for (size_t i = 0; i < blocks.size(); i++) {
        const TransformerBlock& b = blocks[i];
        const std::string p = "model.layers." + std::to_string(i) + ".";
        out.emplace_back(p + "input_layernorm.weight", b.norm1.weight_id);
        out.emplace_back(p + "self_attn.q_proj.weight", b.attn.q_proj.weight_id);
        out.emplace_back(p + "self_attn.k_proj.weight", b.attn.k_proj.weight_id);
        out.emplace_back(p + "self_attn.v_proj.weight", b.attn.v_proj.weight_id);
        out.emplace_back(p + "self_attn.o_proj.weight", b.attn.out_proj.weight_id);
        out.emplace_back(p + "post_attention_layernorm.weight", b.norm2.weight_id);
        out.emplace_back(p + "mlp.gate_proj.weight", b.ffn_gate.weight_id);
        out.emplace_back(p + "mlp.up_proj.weight", b.ffn1.weight_id);
        out.emplace_back(p + "mlp.down_proj.weight", b.ffn2.weight_id);
    }
    out.emplace_back("model.norm.weight", norm_f.weight_id);
    if (!tie_weights) out.emplace_back("lm_head.weight", lm_head.weight_id);
    return out;
}
void TransformerLM::tag_parameters(Graph& g) const {
    for (auto& kv : named_params()) g.name_tensor(kv.second, kv.first);
}
void TransformerLM::set_fused(bool fused) {
    for (auto& b : blocks) b.attn.fused = fused;
}

// One block under per-block recompute.  Forward: the block runs with the tape paused (the kernels of a training forward
// pass, no tape nodes), then everything it allocated
// except its output goes back to the pool.  The one tape node recorded for it re-runs the block from its input when the
// backward pass reaches it, seeds the recomputed output's gradient with the gradient that arrived at the kept output,
// replays the new nodes and drops them again.  The kernels are deterministic, so the recomputed activations and the
// gradients equal those of the plain step bit for bit.
static size_t checkpointed_block(Graph& g, const TransformerBlock& block, size_t x_id) {
    const size_t sp = g.mark_save_point();
    g.tape_paused = true;
    size_t y;
    try {
        y = block.forward_with_mask(g, x_id, true);
    } catch (...) {
        g.tape_paused = false;
        throw;
    }
    g.tape_paused = false;
    y = g.restore_save_point_keep(sp, y);
    const TransformerBlock* b = &block;  // blocks live as long as the model, which outlives the tape
    g.tape.nodes.push_back(TapeNode{{x_id}, y, [b, x_id, y](Graph& G) {
        const size_t sp2 = G.mark_save_point(), first = G.tape.nodes.size();
        const size_t y2 = b->forward_with_mask(G, x_id, true);
        {   // the gradient buffer moves over: the recomputed output owns it from here on (it travels on to the residual)
            Tensor& ty = G.at(y);
            Tensor& t2 = G.at(y2);
            t2.grad = ty.grad;
            t2.grad_written = true;
            ty.grad = Storage();
            ty.grad_written = false;
        }
        G.backward_nodes_from(first);
        G.tape.nodes.erase(G.tape.nodes.begin() + first, G.tape.nodes.end());
        G.flush_norm_dw(true);  // the gain gradients' partial rows belong to this block
        G.restore_save_point(sp2);
    }});
    return y;
}

// TransformerLM::forward (src/nn/transformer.rs:184-196).
size_t TransformerLM::forward(Graph& g, size_t x_id) const {
    size_t h = token_emb.forward(g, x_id);
    for (const TransformerBlock& b : blocks) h = checkpointing && !g.no_grad ? checkpointed_block(g, b, h) : b.forward_with_mask(g, h, true);
    h = norm_f.forward(g, h);
    if (tie_weights) return g.matmul_trans_b(h, lm_head.weight_id);
    return lm_head.forward(g, h);
}
std::vector<size_t> TransformerLM::params() const {
    std::vector<size_t> p = token_emb.params();
    for (const TransformerBlock& b : blocks)
        for (size_t id : b.params()) p.push_back(id);
    p.push_back(norm_f.weight_id);
    if (!tie_weights) p.push_back(lm_head.weight_id);
    return p;
}

// ---- AdamW (src/nn/optim.rs) -----------------------------------------------------------------------

AdamW::AdamW(Graph& g, std::vector<size_t> params_, float lr_) : params(std::move(params_)), lr(lr_), g_(g) {
    void* p = nullptr;
    g_.check(eisen_hip_malloc_zeroed(g_.ctx(), 2 * sizeof(float), &p), "AdamW");
    norm_dev_ = (float*)p;
}
AdamW::~AdamW() {
    for (auto& s : m_)
        if (s.ptr) eisen_hip_free(g_.ctx(), s.ptr);
    for (auto& s : v_)
        if (s.ptr) eisen_hip_free(g_.ctx(), s.ptr);
    if (norm_dev_) eisen_hip_free(g_.ctx(), norm_dev_);
}

// AdamW::init_moments (src/nn/optim.rs:70-112): f32 first and second moments, zero.
void AdamW::init_moments() {
    if (!m_.empty()) return;
    for (size_t id : params) {
        const size_t n = g_.at(id).size();
        Storage m, v;
        m.numel = v.numel = n;
        g_.check(eisen_hip_malloc_zeroed(g_.ctx(), std::max<size_t>(n, 1) * sizeof(float), &m.ptr), "AdamW moments");
        g_.check(eisen_hip_malloc_zeroed(g_.ctx(), std::max<size_t>(n, 1) * sizeof(float), &v.ptr), "AdamW moments");
        m_.push_back(m);
        v_.push_back(v);
    }
}

std::vector<eisen_param_slot> AdamW::slots() {
    init_moments();
    std::vector<eisen_param_slot> out;
    for (size_t i = 0; i < params.size(); i++) {
        Tensor& t = g_.at(params[i]);
        if (!t.is_param || t.data.dtype != EISEN_F32) throw Error("AdamW: tensor " + std::to_string(params[i]) + " is not an f32 parameter");
        eisen_param_slot s;
        s.w = (float*)t.data.ptr;
        s.g = (const float*)t.grad.ptr;
        s.m = (float*)m_[i].ptr;
        s.v = (float*)v_[i].ptr;
        s.w_bf16 = t.shadow.ptr;
        s.n = t.size();
        if (s.n) out.push_back(s);
    }
    return out;
}

// AdamW::zero_grad (src/nn/optim.rs:207-245).  Deferred: the first gradient store of the next
// backward overwrites instead of adding, so the buffers are not swept twice.
void AdamW::zero_grad() {
    for (size_t id : params) g_.request_zero_grad(id);
}

// AdamW::clip_grad_norm (src/nn/optim.rs:250-321): norm and coefficient are computed on the device
// (f64 accumulation), gradients scaled in place when the coefficient is below 1.
std::pair<float, float> AdamW::clip_grad_norm(float max_norm) {
    for (size_t id : params) g_.materialize_grad(id);
    std::vector<eisen_param_slot> s = slots();
    g_.check(eisen_hip_grad_norm(g_.ctx(), s.data(), s.size(), max_norm, norm_dev_), "clip_grad_norm");
    float host[2] = {0.f, 1.f};
    g_.check(eisen_hip_dtoh(g_.ctx(), host, norm_dev_, sizeof(host)), "clip_grad_norm");
    if (host[1] < 1.0f)
        for (auto& slot : s) g_.check(eisen_hip_scale_by_device_scalar(g_.ctx(), (void*)slot.g, EISEN_F32, norm_dev_ + 1, slot.n), "clip_grad_norm scale");
    norm_valid_ = true;
    return {host[0], host[1]};
}

float AdamW::last_grad_norm() {
    if (!norm_valid_) return 0.0f;
    float host[2];
    g_.check(eisen_hip_dtoh(g_.ctx(), host, norm_dev_, sizeof(host)), "last_grad_norm");
    return host[0];
}
float AdamW::last_grad_scale() {
    if (!norm_valid_) return 1.0f;
    float host[2];
    g_.check(eisen_hip_dtoh(g_.ctx(), host, norm_dev_, sizeof(host)), "last_grad_scale");
    return host[1];
}

// AdamW::step (src/nn/optim.rs:334-562): optional clip (maybe_clip_gradients, :114-200), t += 1,
// bias corrections by f32 powi, then one fused launch over every parameter.  With a clip norm
// configured the coefficient stays on the device and is applied inside the update kernel.
void AdamW::step() {
    for (size_t id : params) g_.materialize_grad(id);
    std::vector<eisen_param_slot> s = slots();
    const float* scale_dev = nullptr;
    if (grad_clip_norm_ > 0.0f) {
        g_.check(eisen_hip_grad_norm(g_.ctx(), s.data(), s.size(), grad_clip_norm_, norm_dev_), "AdamW clip");
        scale_dev = norm_dev_ + 1;
        norm_valid_ = true;
    }
    t_ += 1;
    const float bc1 = 1.0f / (1.0f - powi_f32(beta1, (int)t_));
    const float bc2 = 1.0f / (1.0f - powi_f32(beta2, (int)t_));
    g_.check(eisen_hip_adamw_step(g_.ctx(), s.data(), s.size(), lr, beta1, beta2, eps, weight_decay, bc1, bc2, scale_dev), "AdamW step");
}

// CosineScheduler::get_lr (src/nn/scheduler.rs:45-55)
float CosineScheduler::get_lr(size_t step) const {
    if (step < warmup_steps) return lr_max * (float)(step + 1) / (float)warmup_steps;
    const size_t decay = std::max<size_t>(total_steps - warmup_steps, 1);
    float progress = (float)(step - warmup_steps) / (float)decay;
    progress = std::fmin(std::fmax(progress, 0.0f), 1.0f);
    return lr_min + 0.5f * (lr_max - lr_min) * (1.0f + std::cos(3.14159274101257324f * progress));
}

void lm_micro_step(Graph& g, const TransformerLM& lm, const float* ids, const int64_t* targets, size_t mb, size_t seq, float* loss_out) {
    const size_t x_id = g.alloc_pooled({mb, seq});
    g.name_tensor(x_id, "input");
    g.load_tensor_data(x_id, ids, mb * seq);
    const size_t logits = lm.forward(g, x_id);
    g.reinterpret_shape(logits, {mb * seq, lm.vocab_size});  // train_llm.rs:440 reshapes (a copy); the view is equivalent
    const std::vector<int64_t> t(targets, targets + mb * seq);
    const size_t loss = g.cross_entropy_masked(logits, t);
    // the loss is read back every micro-batch (train_llm.rs:450); the copy is queued here and collected after the backward
    // pass has been queued behind it, so the device never runs dry while the host waits
    int ticket = -1;
    if (loss_out) g.check(eisen_hip_dtoh_begin(g.ctx(), g.at(loss).data.ptr, sizeof(float), &ticket), "loss read-back");
    try {
        g.backward(loss);
    } catch (...) {
        float dropped;
        if (ticket >= 0) (void)eisen_hip_dtoh_finish(g.ctx(), ticket, &dropped, sizeof(float));
        throw;
    }
    if (loss_out) g.check(eisen_hip_dtoh_finish(g.ctx(), ticket, loss_out, sizeof(float)), "loss read-back");
    g.clear_activations();
}

}  // namespace eisen
