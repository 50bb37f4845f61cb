// extern "C" surface of the host Graph / nn / AdamW layer (include/eisen_graph.h).
// C++ exceptions stop here: every entry point returns an int and stores a message.
#include <cstring>
#include <memory>
#include <string>

#include "eisen_graph.h"
#include "io.hpp"
#include "nn.hpp"

using namespace eisen;

struct eisen_graph {
    std::unique_ptr<Graph> g;
    std::string last_error;
};
struct eisen_lm {
    eisen_graph* owner;
    std::unique_ptr<TransformerLM> lm;
};
struct eisen_adamw {
    eisen_graph* owner;
    std::unique_ptr<AdamW> opt;
};

namespace {
template <typename F>
int guarded(eisen_graph* h, F&& f) {
    if (!h || !h->g) return -1;
    try {
        f(*h->g);
        return 0;
    } catch (const std::exception& e) {
        h->last_error = e.what();
        return 1;
    }
}
std::vector<size_t> shape_of(const size_t* shape, int rank) {
    if (rank < 0 || rank > EISEN_MAX_RANK || (rank > 0 && !shape)) throw Error("bad shape argument");
    return std::vector<size_t>(shape, shape + rank);
}
void need(const void* p, const char* what) {
    if (!p) throw Error(std::string("null argument: ") + what);
}
}  // namespace

extern "C" {

int eisen_graph_new(eisen_ctx* ctx, int precision, eisen_graph** out) {
    if (!out) return -1;
    *out = nullptr;
    if (precision != EISEN_PRECISION_FP32 && precision != EISEN_PRECISION_BF16_MIXED) return -1;
    try {
        auto h = std::make_unique<eisen_graph>();
        h->g = std::make_unique<Graph>(ctx, precision == EISEN_PRECISION_BF16_MIXED ? PrecisionMode::Bf16Mixed : PrecisionMode::Fp32);
        *out = h.release();
        return 0;
    } catch (const std::exception&) {
        return 1;
    }
}
int eisen_graph_free(eisen_graph* g) {
    delete g;
    return 0;
}
const char* eisen_graph_last_error(eisen_graph* g) { return g ? g->last_error.c_str() : "null graph"; }

int eisen_graph_alloc(eisen_graph* g, const size_t* shape, int rank, const float* data, size_t* id_out) {
    return guarded(g, [&](Graph& G) {
        need(id_out, "id_out");
        const std::vector<size_t> s = shape_of(shape, rank);
        size_t n = 1;
        for (size_t d : s) n *= d;
        if (n) need(data, "data");
        *id_out = G.alloc(s, data, n);
    });
}
int eisen_graph_alloc_pooled(eisen_graph* g, const size_t* shape, int rank, size_t* id_out) {
    return guarded(g, [&](Graph& G) { need(id_out, "id_out"); *id_out = G.alloc_pooled(shape_of(shape, rank)); });
}
int eisen_graph_load_tensor_data(eisen_graph* g, size_t id, const float* host, size_t n) {
    return guarded(g, [&](Graph& G) { if (n) need(host, "host"); G.load_tensor_data(id, host, n); });
}
int eisen_graph_mark_params(eisen_graph* g) { return guarded(g, [&](Graph& G) { G.mark_params(); }); }
int eisen_graph_mark_save_point(eisen_graph* g, size_t* out) { return guarded(g, [&](Graph& G) { need(out, "out"); *out = G.mark_save_point(); }); }
int eisen_graph_restore_save_point(eisen_graph* g, size_t sp) { return guarded(g, [&](Graph& G) { G.restore_save_point(sp); }); }
int eisen_graph_restore_save_point_keep(eisen_graph* g, size_t sp, size_t keep, size_t* out) {
    return guarded(g, [&](Graph& G) { need(out, "out"); *out = G.restore_save_point_keep(sp, keep); });
}
int eisen_graph_clear_activations(eisen_graph* g) { return guarded(g, [&](Graph& G) { G.clear_activations(); }); }
int eisen_graph_reinterpret_shape(eisen_graph* g, size_t id, const size_t* shape, int rank) {
    return guarded(g, [&](Graph& G) { G.reinterpret_shape(id, shape_of(shape, rank)); });
}
int eisen_graph_set_weight_gradient_window(eisen_graph* g, size_t backward_passes) {
    return guarded(g, [&](Graph& G) { G.set_weight_gradient_window(backward_passes); });
}
int eisen_graph_set_weight_gradients_beside(eisen_graph* g, int on) {
    return guarded(g, [&](Graph& G) { G.set_weight_gradients_beside(on != 0); });
}
int eisen_graph_flush_weight_gradients(eisen_graph* g) {
    return guarded(g, [&](Graph& G) { G.flush_weight_gradients(); });
}
int eisen_graph_set_no_grad(eisen_graph* g, int v) { return guarded(g, [&](Graph& G) { G.no_grad = v != 0; }); }
int eisen_graph_num_tensors(eisen_graph* g, size_t* out) { return guarded(g, [&](Graph& G) { need(out, "out"); *out = G.tensors.size(); }); }
int eisen_graph_num_params(eisen_graph* g, size_t* out) { return guarded(g, [&](Graph& G) { need(out, "out"); *out = G.num_params; }); }
int eisen_graph_tape_len(eisen_graph* g, size_t* out) { return guarded(g, [&](Graph& G) { need(out, "out"); *out = G.tape.nodes.size(); }); }
int eisen_graph_tensor_shape(eisen_graph* g, size_t id, size_t* shape_out, int* rank_out) {
    return guarded(g, [&](Graph& G) {
        need(shape_out, "shape_out");
        need(rank_out, "rank_out");
        const Tensor& t = G.at(id);
        if (t.shape.size() > EISEN_MAX_RANK) throw Error("rank above EISEN_MAX_RANK");
        *rank_out = (int)t.shape.size();
        for (size_t i = 0; i < t.shape.size(); i++) shape_out[i] = t.shape[i];
    });
}
int eisen_graph_sync_to_cpu(eisen_graph* g, size_t id, float* out, size_t n) {
    return guarded(g, [&](Graph& G) {
        if (n != G.at(id).size()) throw Error("sync_to_cpu: element count mismatch");
        if (n) need(out, "out");
        const std::vector<float> v = G.sync_to_cpu(id);
        std::memcpy(out, v.data(), n * sizeof(float));
    });
}
int eisen_graph_sync_grad_to_cpu(eisen_graph* g, size_t id, float* out, size_t n) {
    return guarded(g, [&](Graph& G) {
        if (n != G.at(id).size()) throw Error("sync_grad_to_cpu: element count mismatch");
        if (n) need(out, "out");
        const std::vector<float> v = G.sync_grad_to_cpu(id);
        std::memcpy(out, v.data(), n * sizeof(float));
    });
}
int eisen_graph_sync_compute_copy_to_cpu(eisen_graph* g, size_t id, float* out, size_t n) {
    return guarded(g, [&](Graph& G) {
        if (n != G.at(id).size()) throw Error("sync_compute_copy_to_cpu: element count mismatch");
        if (n) need(out, "out");
        const std::vector<float> v = G.sync_compute_copy_to_cpu(id);
        std::memcpy(out, v.data(), n * sizeof(float));
    });
}
int eisen_graph_synchronize(eisen_graph* g) { return guarded(g, [&](Graph& G) { G.synchronize(); }); }

#define OP_OUT(expr) return guarded(g, [&](Graph& G) { need(out, "out"); *out = (expr); })
int eisen_graph_add(eisen_graph* g, size_t a, size_t b, size_t* out) { OP_OUT(G.add(a, b)); }
int eisen_graph_mul(eisen_graph* g, size_t a, size_t b, size_t* out) { OP_OUT(G.mul(a, b)); }
int eisen_graph_silu(eisen_graph* g, size_t a, size_t* out) { OP_OUT(G.silu(a)); }
int eisen_graph_swiglu(eisen_graph* g, size_t gate, size_t up, size_t* out) { OP_OUT(G.swiglu(gate, up)); }
int eisen_graph_matmul(eisen_graph* g, size_t a, size_t b, size_t* out) { OP_OUT(G.matmul(a, b)); }
int eisen_graph_matmul_trans_b(eisen_graph* g, size_t a, size_t b, size_t* out) { OP_OUT(G.matmul_trans_b(a, b)); }
int eisen_graph_bmm(eisen_graph* g, size_t a, size_t b, int trans_b, size_t* out) { OP_OUT(G.bmm(a, b, trans_b != 0)); }
int eisen_graph_softmax(eisen_graph* g, size_t a, size_t* out) { OP_OUT(G.softmax(a)); }
int eisen_graph_cross_entropy(eisen_graph* g, size_t logits, const int64_t* targets, size_t n, size_t* out) {
    return guarded(g, [&](Graph& G) { need(out, "out"); need(targets, "targets"); *out = G.cross_entropy(logits, std::vector<int64_t>(targets, targets + n)); });
}
int eisen_graph_cross_entropy_masked(eisen_graph* g, size_t logits, const int64_t* targets, size_t n, size_t* out) {
    return guarded(g, [&](Graph& G) { need(out, "out"); need(targets, "targets"); *out = G.cross_entropy_masked(logits, std::vector<int64_t>(targets, targets + n)); });
}
int eisen_graph_transpose_0213(eisen_graph* g, size_t a, size_t* out) { OP_OUT(G.transpose_0213(a)); }
int eisen_graph_gather(eisen_graph* g, size_t w, size_t idx, size_t* out) { OP_OUT(G.gather(w, idx)); }
int eisen_graph_reshape(eisen_graph* g, size_t a, const size_t* shape, int rank, size_t* out) { OP_OUT(G.reshape(a, shape_of(shape, rank))); }
int eisen_graph_rope(eisen_graph* g, size_t a, size_t head_dim, size_t* out) { OP_OUT(G.rope(a, head_dim)); }
int eisen_graph_rms_norm(eisen_graph* g, size_t x, size_t w, float eps, size_t* out) { OP_OUT(G.rms_norm(x, w, eps)); }
int eisen_graph_repeat_kv(eisen_graph* g, size_t x, size_t repeats, size_t* out) { OP_OUT(G.repeat_kv(x, repeats)); }
int eisen_graph_flash_attention(eisen_graph* g, size_t q, size_t k, size_t v, float scale, int causal, size_t* out) {
    OP_OUT(G.flash_attention(q, k, v, scale, causal != 0));
}
int eisen_graph_attention_gqa(eisen_graph* g, size_t q, size_t k, size_t v, size_t heads, size_t kv_heads, float scale, int causal, size_t* out) {
    OP_OUT(G.attention_gqa(q, k, v, heads, kv_heads, scale, causal != 0));
}
int eisen_graph_backward(eisen_graph* g, size_t loss_id) { return guarded(g, [&](Graph& G) { G.backward(loss_id); }); }

int eisen_lm_new(eisen_graph* g, size_t vocab, size_t hidden, size_t heads, size_t kv_heads, size_t ffn, size_t layers, int tie, eisen_lm** out) {
    return guarded(g, [&](Graph& G) {
        need(out, "out");
        if (!vocab || !hidden || !heads || !kv_heads || !ffn) throw Error("TransformerLM: zero-sized dimension");
        auto h = std::make_unique<eisen_lm>();
        h->owner = g;
        h->lm = std::make_unique<TransformerLM>(G, vocab, hidden, heads, kv_heads, ffn, layers, tie != 0);
        *out = h.release();
    });
}
int eisen_lm_free(eisen_lm* lm) {
    delete lm;
    return 0;
}
int eisen_lm_params(eisen_lm* lm, size_t* ids_out, size_t capacity, size_t* count_out) {
    if (!lm) return -1;
    return guarded(lm->owner, [&](Graph&) {
        need(count_out, "count_out");
        const std::vector<size_t> p = lm->lm->params();
        *count_out = p.size();
        if (ids_out) {
            if (capacity < p.size()) throw Error("eisen_lm_params: capacity too small");
            for (size_t i = 0; i < p.size(); i++) ids_out[i] = p[i];
        }
    });
}
int eisen_lm_forward(eisen_graph* g, eisen_lm* lm, size_t x_id, size_t* out) {
    return guarded(g, [&](Graph& G) { need(lm, "lm"); need(out, "out"); *out = lm->lm->forward(G, x_id); });
}
int eisen_lm_set_fused(eisen_lm* lm, int fused) {
    if (!lm) return -1;
    lm->lm->set_fused(fused != 0);
    return 0;
}
int eisen_lm_set_checkpointing(eisen_lm* lm, int on) {
    if (!lm) return -1;
    lm->lm->set_checkpointing(on != 0);
    return 0;
}
int eisen_lm_micro_step(eisen_graph* g, eisen_lm* lm, const float* ids, const int64_t* targets, size_t mb, size_t seq, float* loss_out) {
    return guarded(g, [&](Graph& G) { need(lm, "lm"); need(ids, "ids"); need(targets, "targets"); lm_micro_step(G, *lm->lm, ids, targets, mb, seq, loss_out); });
}

int eisen_adamw_new(eisen_graph* g, const size_t* params, size_t n, float lr, eisen_adamw** out) {
    return guarded(g, [&](Graph& G) {
        need(out, "out");
        if (n) need(params, "params");
        auto h = std::make_unique<eisen_adamw>();
        h->owner = g;
        h->opt = std::make_unique<AdamW>(G, std::vector<size_t>(params, params + n), lr);
        *out = h.release();
    });
}
int eisen_adamw_free(eisen_adamw* opt) {
    delete opt;
    return 0;
}
#define OPT_GUARD(body) if (!opt) return -1; return guarded(opt->owner, [&](Graph&) { body; })
int eisen_adamw_config(eisen_adamw* opt, float lr, float beta1, float beta2, float eps, float wd, float clip) {
    OPT_GUARD(opt->opt->lr = lr; opt->opt->beta1 = beta1; opt->opt->beta2 = beta2; opt->opt->eps = eps; opt->opt->weight_decay = wd; opt->opt->set_grad_clip_norm(clip));
}
int eisen_adamw_init_moments(eisen_adamw* opt) { OPT_GUARD(opt->opt->init_moments()); }
int eisen_adamw_zero_grad(eisen_adamw* opt) { OPT_GUARD(opt->opt->zero_grad()); }
int eisen_adamw_clip_grad_norm(eisen_adamw* opt, float max_norm, float* norm_out, float* coef_out) {
    OPT_GUARD(auto r = opt->opt->clip_grad_norm(max_norm); if (norm_out) *norm_out = r.first; if (coef_out) *coef_out = r.second);
}
int eisen_adamw_step(eisen_adamw* opt) { OPT_GUARD(opt->opt->step()); }
int eisen_adamw_last_grad_norm(eisen_adamw* opt, float* norm_out, float* scale_out) {
    OPT_GUARD(if (norm_out) *norm_out = opt->opt->last_grad_norm(); if (scale_out) *scale_out = opt->opt->last_grad_scale());
}
int eisen_adamw_moments_to_cpu(eisen_adamw* opt, size_t i, float* m_out, float* v_out, size_t n) {
    if (!opt) return -1;
    return guarded(opt->owner, [&](Graph& G) {
        opt->opt->init_moments();
        if (i >= opt->opt->params.size()) throw Error("moments: parameter index out of range");
        const Storage& m = opt->opt->moment_m(i);
        const Storage& v = opt->opt->moment_v(i);
        if (n != m.numel) throw Error("moments: element count mismatch");
        if (m_out) G.check(eisen_hip_dtoh(G.ctx(), m_out, m.ptr, n * sizeof(float)), "moments");
        if (v_out) G.check(eisen_hip_dtoh(G.ctx(), v_out, v.ptr, n * sizeof(float)), "moments");
    });
}
float eisen_cosine_lr(float lr_max, float lr_min, size_t warmup, size_t total, size_t step) {
    return CosineScheduler{lr_max, lr_min, warmup, total}.get_lr(step);
}


// ---- data loader / checkpoints -----------------------------------------------------------------
}  // extern "C"

struct eisen_data_loader {
    std::unique_ptr<BinaryDataLoader> dl;
};
namespace {
thread_local std::string io_error;
template <typename F>
int io_guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        io_error = e.what();
        return 1;
    }
}
}  // namespace

extern "C" {

const char* eisen_io_last_error(void) { return io_error.c_str(); }

int eisen_data_loader_open(const char* path, size_t seq_len, size_t batch_size, eisen_data_loader** out) {
    if (!out) return -1;
    *out = nullptr;
    return io_guarded([&] {
        need(path, "path");
        auto h = std::make_unique<eisen_data_loader>();
        h->dl = std::make_unique<BinaryDataLoader>(path, seq_len, batch_size);
        *out = h.release();
    });
}
int eisen_data_loader_close(eisen_data_loader* dl) {
    delete dl;
    return 0;
}
int eisen_data_loader_total_batches(eisen_data_loader* dl, size_t* out) {
    if (!dl || !out) return -1;
    *out = dl->dl->total_batches();
    return 0;
}
int eisen_data_loader_next_batch(eisen_data_loader* dl, float* x, int64_t* targets, int* got) {
    if (!dl) return -1;
    return io_guarded([&] {
        need(x, "x"); need(targets, "targets"); need(got, "got");
        *got = dl->dl->next_batch(x, targets) ? 1 : 0;
    });
}
int eisen_data_loader_reset(eisen_data_loader* dl) {
    if (!dl) return -1;
    dl->dl->reset();
    return 0;
}
int eisen_graph_save_weights(eisen_graph* g, const char* path) {
    return guarded(g, [&](Graph& G) { need(path, "path"); save_weights(G, path); });
}
int eisen_graph_load_weights(eisen_graph* g, const size_t* params, size_t n_params, const char* path, size_t* floats_out) {
    return guarded(g, [&](Graph& G) {
        need(path, "path");
        if (n_params) need(params, "params");
        const size_t n = load_weights(G, std::vector<size_t>(params, params + n_params), path);
        if (floats_out) *floats_out = n;
    });
}
int eisen_lm_write_safetensors(eisen_graph* g, eisen_lm* lm, const char* path) {
    return guarded(g, [&](Graph& G) {
        need(path, "path");
        if (!lm || !lm->lm) throw Error("null model");
        write_safetensors(G, lm->lm->named_params(), path);
    });
}
int eisen_write_llama_config(const char* path, size_t vocab, size_t hidden, size_t ffn, size_t layers, size_t heads, size_t kv_heads,
                             size_t max_position_embeddings, float rms_norm_eps, float rope_theta, int tie_word_embeddings) {
    return io_guarded([&] {
        need(path, "path");
        write_llama_config(path, LlamaConfig{vocab, hidden, ffn, layers, heads, kv_heads, max_position_embeddings, rms_norm_eps, rope_theta,
                                             tie_word_embeddings != 0});
    });
}

}  // extern "C"
