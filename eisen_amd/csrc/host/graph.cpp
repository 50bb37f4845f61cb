// Graph / Tensor / Tape for Device::Gpu over the eisen_hip C-ABI.  See graph.hpp.
#include "graph.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <numeric>

namespace eisen {

namespace {
size_t numel_of(const std::vector<size_t>& shape) {
    size_t n = 1;
    for (size_t s : shape) n *= s;
    return n;
}
std::string shape_str(const std::vector<size_t>& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}
constexpr size_t kHostCopyLimit = size_t(1) << 22;  // elements; token-id tensors are far below
}  // namespace

std::vector<size_t> compute_strides(const std::vector<size_t>& shape) {
    std::vector<size_t> st(shape.size(), 0);
    size_t cur = 1;
    for (size_t i = shape.size(); i-- > 0;) {
        st[i] = cur;
        cur *= shape[i];
    }
    return st;
}
std::vector<size_t> broadcasted_shape(const std::vector<size_t>& a, const std::vector<size_t>& b) {
    const size_t ml = std::max(a.size(), b.size());
    std::vector<size_t> out(ml);
    for (size_t i = 0; i < ml; i++) {
        const size_t da = i < ml - a.size() ? 1 : a[i - (ml - a.size())];
        const size_t db = i < ml - b.size() ? 1 : b[i - (ml - b.size())];
        out[i] = std::max(da, db);
    }
    return out;
}
std::vector<size_t> broadcasted_strides(const std::vector<size_t>& shape, const std::vector<size_t>& base,
                                        const std::vector<size_t>& out_shape) {
    std::vector<size_t> st(out_shape.size(), 0);
    const size_t pad = out_shape.size() - shape.size();
    for (size_t i = 0; i < shape.size(); i++)
        if (shape[i] == out_shape[pad + i]) st[pad + i] = base[i];
    return st;
}

Graph::Graph(eisen_ctx* ctx, PrecisionMode mode) : precision_mode(mode), ctx_(ctx) {
    if (!ctx) throw Error("Graph: null device context (Device::Gpu needs eisen_hip_init)");
}

Graph::~Graph() {
    (void)eisen_hip_side_wait(ctx_);
    for (auto& t : tensors) release(t);
    for (auto& kv : retained_)
        if (kv.second) eisen_hip_free(ctx_, const_cast<void*>(kv.first));
}

void Graph::check(int rc, const char* what) const {
    if (rc != 0) throw Error(std::string(what) + ": " + eisen_hip_last_error(ctx_) + " (code " + std::to_string(rc) + ")");
}

Tensor& Graph::at(size_t id) {
    if (id >= tensors.size()) throw Error("tensor id " + std::to_string(id) + " out of range");
    return tensors[id];
}

Storage Graph::device_alloc(size_t numel, int dtype, bool zero) {
    Storage s;
    s.numel = numel;
    s.dtype = dtype;
    const size_t bytes = std::max<size_t>(numel, 1) * (dtype == EISEN_BF16 ? 2 : 4);
    check(zero ? eisen_hip_malloc_zeroed(ctx_, bytes, &s.ptr) : eisen_hip_malloc(ctx_, bytes, &s.ptr), "device allocation");
    return s;
}
void Graph::free_buffer(void* ptr) {
    if (!ptr) return;
    if (!retained_.empty()) {
        auto it = retained_.find(ptr);
        if (it != retained_.end()) {  // a windowed weight-gradient GEMM still has to read it: flush_weight_gradients frees it
            it->second = true;
            return;
        }
    }
    check(eisen_hip_free(ctx_, ptr), "device free");
}
void Graph::device_free(Storage& s) {
    free_buffer(s.ptr);
    s = Storage();
}
void Graph::release(Tensor& t) {
    void* const bufs[3] = {t.data.ptr, t.grad_borrowed ? nullptr : t.grad.ptr, t.shadow.ptr};
    t.data = t.grad = t.shadow = Storage();
    for (void* p : bufs) free_buffer(p);
}

size_t Graph::push_tensor(const std::vector<size_t>& shape, int dtype, bool pooled) {
    Tensor t;
    t.id = tensors.size();
    t.shape = shape;
    t.strides = compute_strides(shape);
    t.is_pooled = pooled;
    t.data = device_alloc(numel_of(shape), dtype, false);
    tensors.push_back(std::move(t));
    return tensors.size() - 1;
}

// Graph::alloc (src/graph/mod.rs:558-564) + Tensor::new (src/tensor.rs:145-175): data uploaded,
// gradient zero-filled.  In mixed mode the kernels read a bf16 copy; `data` stays the f32 master.
size_t Graph::alloc(const std::vector<size_t>& shape, const float* data, size_t n) {
    if (n != numel_of(shape)) throw Error("alloc: shape " + shape_str(shape) + " does not hold " + std::to_string(n) + " values");
    const size_t id = push_tensor(shape, EISEN_F32, false);
    Tensor& t = tensors[id];
    t.is_param = true;
    if (n) check(eisen_hip_htod(ctx_, t.data.ptr, data, n * sizeof(float)), "alloc upload");
    t.grad = device_alloc(n, EISEN_F32, true);
    if (n <= kHostCopyLimit) t.host_copy.assign(data, data + n);
    if (uses_bf16_mixed_precision()) {
        t.shadow = device_alloc(n, EISEN_BF16, false);
        refresh_shadow(id);
    }
    return id;
}
size_t Graph::alloc(const std::vector<size_t>& shape, const std::vector<float>& data) { return alloc(shape, data.data(), data.size()); }

// Graph::alloc_pooled (src/graph/mod.rs:437-556): an activation-typed buffer from the pool;
// the gradient is allocated on first use in backward (src/graph/memory.rs:401-417).
size_t Graph::alloc_pooled(const std::vector<size_t>& shape) { return push_tensor(shape, act_dtype(), true); }
size_t Graph::alloc_pooled_dtype(const std::vector<size_t>& shape, int dtype) { return push_tensor(shape, dtype, true); }

void Graph::refresh_shadow(size_t id) {
    Tensor& t = at(id);
    if (!t.shadow.valid()) return;
    check(eisen_hip_cast(ctx_, t.data.ptr, EISEN_F32, t.shadow.ptr, EISEN_BF16, t.data.numel), "bf16 weight copy");
}

const Storage& Graph::compute_data(size_t id) {
    Tensor& t = at(id);
    return t.shadow.valid() ? t.shadow : t.data;
}

// Graph::load_tensor_data (src/graph/mod.rs:368-430).  bf16 storage is filled with
// round-to-nearest-even values (the device cast), not the reference's host-side truncation.
void Graph::load_tensor_data(size_t id, const float* host, size_t n) {
    Tensor& t = at(id);
    if (n != t.size()) throw Error("Shape mismatch: Tensor " + std::to_string(id) + " expects " + std::to_string(t.size()) + " elements, but got " + std::to_string(n) + ".");
    if (n <= kHostCopyLimit) t.host_copy.assign(host, host + n);
    else t.host_copy.clear();
    if (t.data.dtype == EISEN_F32) {
        check(eisen_hip_htod(ctx_, t.data.ptr, host, n * sizeof(float)), "load_tensor_data");
        refresh_shadow(id);
    } else {
        Storage tmp = device_alloc(n, EISEN_F32, false);
        check(eisen_hip_htod(ctx_, tmp.ptr, host, n * sizeof(float)), "load_tensor_data");
        check(eisen_hip_cast(ctx_, tmp.ptr, EISEN_F32, t.data.ptr, EISEN_BF16, n), "load_tensor_data cast");
        device_free(tmp);
    }
}

static std::vector<float> download(Graph& g, const Storage& s) {
    std::vector<float> out(s.numel);
    if (!s.numel) return out;
    if (s.dtype == EISEN_F32) {
        g.check(eisen_hip_dtoh(g.ctx(), out.data(), s.ptr, s.numel * sizeof(float)), "sync_to_cpu");
    } else {
        std::vector<uint16_t> raw(s.numel);
        g.check(eisen_hip_dtoh(g.ctx(), raw.data(), s.ptr, s.numel * 2), "sync_to_cpu");
        for (size_t i = 0; i < s.numel; i++) {
            const uint32_t bits = (uint32_t)raw[i] << 16;
            std::memcpy(&out[i], &bits, 4);
        }
    }
    return out;
}

// Tensor::sync_to_cpu / Graph::sync_grad_to_cpu (src/tensor.rs:177-223, src/graph/mod.rs:629-668).
std::vector<float> Graph::sync_to_cpu(size_t id) { return download(*this, at(id).data); }
std::vector<float> Graph::sync_compute_copy_to_cpu(size_t id) { return download(*this, compute_data(id)); }
std::vector<float> Graph::sync_grad_to_cpu(size_t id) {
    Tensor& t = at(id);
    materialize_grad(id);
    if (!t.grad.valid()) return std::vector<float>(t.size(), 0.0f);  // never touched by backward: zero
    return download(*this, t.grad);
}

void Graph::synchronize() { check(eisen_hip_stream_sync(ctx_), "synchronize"); }

// Graph::reinterpret_shape (src/graph/ops/transform.rs:413-426).
void Graph::reinterpret_shape(size_t id, const std::vector<size_t>& shape) {
    Tensor& t = at(id);
    if (numel_of(shape) != t.size()) throw Error("reinterpret_shape: element count mismatch");
    t.shape = shape;
    t.strides = compute_strides(shape);
}

// Graph::restore_save_point / clear_activations (src/graph/mod.rs:336-365, :432-435): buffers go
// back to the size-keyed pool inside the runtime.
void Graph::restore_save_point(size_t save_point) {
    if (!side_guards.empty()) side_join();  // a backward pass that threw may have left side-stream work reading these buffers
    // buffers kept for side-stream GEMMs (no window): given back now, so that a block-by-block recompute keeps its low
    // high-water mark (the main stream waits for the side stream here; after a whole backward pass it already has)
    if (window_dw.empty() && !retained_.empty()) side_join();
    flush_norm_dw(false);                   // ... and partial rows nobody will finish
    while (tensors.size() > save_point) {
        release(tensors.back());
        tensors.pop_back();
    }
}
size_t Graph::restore_save_point_keep(size_t save_point, size_t keep) {
    if (keep < save_point || keep >= tensors.size()) throw Error("restore_save_point_keep: the tensor to keep is not above the save point");
    Tensor kept = std::move(tensors[keep]);
    tensors[keep] = Tensor();  // nothing left to release there
    restore_save_point(save_point);
    kept.id = tensors.size();
    tensors.push_back(std::move(kept));
    return tensors.size() - 1;
}
void Graph::clear_activations() {
    tape.nodes.clear();
    restore_save_point(num_params);
}

void Graph::record(std::vector<size_t> inputs, size_t output, std::function<void(Graph&)> fn) {
    if (no_grad || tape_paused) return;  // e.g. src/graph/ops/linear.rs:288
    tape.nodes.push_back(TapeNode{std::move(inputs), output, std::move(fn)});
}

Storage& Graph::grad_for_write(size_t id, int* accumulate, const void** add_from) {
    Tensor& t = at(id);
    if (t.is_param) {
        if (!in_beside_ && !side_written_.empty() && std::find(side_written_.begin(), side_written_.end(), id) != side_written_.end()) side_join();
        *accumulate = t.grad_zero_pending ? 0 : 1;
        t.grad_zero_pending = false;
        if (add_from) *add_from = t.grad.ptr;
        return t.grad;
    }
    if (!t.grad.valid()) {
        t.grad = device_alloc(t.size(), t.data.dtype, false);
        *accumulate = 0;
    } else {
        *accumulate = t.grad_written ? 1 : 0;
    }
    t.grad_written = true;
    if (!side_guards.empty() && std::find(side_guards.begin(), side_guards.end(), t.grad.ptr) != side_guards.end()) side_join();
    if (add_from) *add_from = t.grad.ptr;
    if (!retained_.empty() && retained_.count(t.grad.ptr)) {
        // The buffer's present content is an operand of a weight-gradient GEMM of the window: the store goes elsewhere.
        // Whoever else points at the old buffer (the tensor it was handed over from) only keeps it from being freed twice.
        Storage old = t.grad;
        t.grad = device_alloc(old.numel, old.dtype, false);
        if (*accumulate && !add_from)
            check(eisen_hip_dtod(ctx_, t.grad.ptr, old.ptr, old.numel * (old.dtype == EISEN_BF16 ? 2 : 4)), "gradient copy");
        if (t.grad_borrowed) t.grad_borrowed = false;  // the fresh buffer is this tensor's own
        else retained_[old.ptr] = true;                // the tensor owned the old one: the flush frees it
    }
    return t.grad;
}

void Graph::flush_norm_dw(bool compute) {
    if (pending_norm_dw.empty()) return;
    std::vector<PendingNormDW> list;
    list.swap(pending_norm_dw);
    int rc = 0;
    if (compute) {
        std::vector<const float*> parts;
        std::vector<float*> gws;
        std::vector<size_t> nrows;
        std::vector<int> assign;
        for (const PendingNormDW& e : list) {
            if (e.nrows == 0) {
                if (e.assign) at(e.weight).grad_zero_pending = true;  // nothing was added: the clearing is still owed
                continue;
            }
            parts.push_back((const float*)e.partial.ptr);
            gws.push_back((float*)at(e.weight).grad.ptr);
            nrows.push_back(e.nrows);
            assign.push_back(e.assign ? 1 : 0);
        }
        if (!parts.empty()) rc = eisen_hip_rms_norm_dw_finish(ctx_, parts.size(), parts.data(), gws.data(), nrows.data(), list[0].dim, assign.data());
    } else {
        for (const PendingNormDW& e : list)
            if (e.assign) at(e.weight).grad_zero_pending = true;
    }
    for (PendingNormDW& e : list) device_free(e.partial);
    check(rc, "rms_norm gain gradients");
}

// ---- weight gradients over a window of micro-batches (see graph.hpp) -----------------------------------------

void Graph::set_weight_gradient_window(size_t backward_passes) {
    if (backward_passes > (size_t)EISEN_GEMM_MAX_KSEGMENTS) throw Error("set_weight_gradient_window: at most " + std::to_string(EISEN_GEMM_MAX_KSEGMENTS) + " backward passes");
    flush_weight_gradients();
    window_ = backward_passes;
}

// Products the one-launch form of eisen_hip_gemm_grouped_ksegments takes and that are big enough to be worth keeping their
// operands for: bf16 operands, an f32 parameter gradient of at least 16 whole 256 x 256 tiles, pieces of whole 128 rows.
bool Graph::window_fits(size_t weight, int dtype, size_t rows, size_t in, size_t out) {
    if (window_ < 2 || dtype != EISEN_BF16 || rows == 0 || rows % 128 || in % 256 || out % 256 || (in / 256) * (out / 256) < 16) return false;
    const Tensor& tw = at(weight);
    return tw.is_param && tw.grad.dtype == EISEN_F32 && tw.size() == in * out;
}

bool Graph::window_take(size_t weight, const void* x, const void* dy, int dtype, size_t rows, size_t in, size_t out) {
    if (!window_fits(weight, dtype, rows, in, out)) return false;
    WindowDW* e = nullptr;
    for (WindowDW& c : window_dw)
        if (c.weight == weight) e = &c;
    if (e && (e->rows != rows || e->x.size() >= (size_t)EISEN_GEMM_MAX_KSEGMENTS)) {  // a piece of another length, or one too many:
        flush_weight_gradients(weight);  // this weight's pieces are contracted now, the other weights and the pass count stay
        e = nullptr;
    }
    if (!e) {
        window_dw.push_back(WindowDW{weight, rows, in, out, {}, {}});
        e = &window_dw.back();
    }
    e->x.push_back(x);
    e->dy.push_back(dy);
    retained_.emplace(x, false);
    retained_.emplace(dy, false);
    return true;
}

// only_weight: contract the pieces held for that one weight and leave the window as it is otherwise (the kept operands
// stay allocated until the whole window is flushed: other weights' pieces may be the same buffers)
void Graph::flush_weight_gradients(size_t only_weight) {
    const bool all = only_weight == (size_t)-1;
    if (all) window_passes_ = 0;
    if (window_dw.empty()) {
        // nothing waits for a launch; buffers kept for side-stream GEMMs go back once the main stream has waited for them
        if (all && !retained_.empty()) side_join();
        return;
    }
    std::vector<WindowDW> list;
    if (all) {
        list.swap(window_dw);
    } else {
        for (size_t i = 0; i < window_dw.size(); i++)
            if (window_dw[i].weight == only_weight) {
                list.push_back(std::move(window_dw[i]));
                window_dw.erase(window_dw.begin() + (ptrdiff_t)i);
                break;
            }
        if (list.empty()) return;
    }
    // One launch per set of products with the same shape, number of pieces and accumulate state (equal tiles, and for a
    // model of equal blocks a whole number of rounds of the chip); sets of fewer tiles than the chip has CUs share one.
    struct Launch {
        size_t in, out, rows, pieces;
        int acc;
        std::vector<const WindowDW*> members;
    };
    std::vector<Launch> launches;
    for (const WindowDW& e : list) {
        int acc = 0;
        grad_for_write(e.weight, &acc);
        Launch* l = nullptr;
        for (Launch& c : launches)
            if (c.in == e.in && c.out == e.out && c.rows == e.rows && c.pieces == e.x.size() && c.acc == acc) l = &c;
        if (!l) {
            launches.push_back(Launch{e.in, e.out, e.rows, e.x.size(), acc, {}});
            l = &launches.back();
        }
        l->members.push_back(&e);
    }
    for (size_t i = 0; i < launches.size(); i++) {  // small sets join the first small set they can run with
        Launch& a = launches[i];
        if ((a.in / 256) * (a.out / 256) * a.members.size() >= 256) continue;
        for (size_t j = i + 1; j < launches.size();) {
            Launch& b = launches[j];
            if ((b.in / 256) * (b.out / 256) * b.members.size() < 256 && b.rows == a.rows && b.pieces == a.pieces && b.acc == a.acc) {
                a.members.insert(a.members.end(), b.members.begin(), b.members.end());
                launches.erase(launches.begin() + (ptrdiff_t)j);
            } else {
                j++;
            }
        }
    }
    int rc = 0;
    for (const Launch& l : launches) {
        std::vector<const void*> As, Bs;
        std::vector<void*> Cs;
        std::vector<size_t> Ms, Ns;
        for (const WindowDW* e : l.members) {
            As.insert(As.end(), e->x.begin(), e->x.end());
            Bs.insert(Bs.end(), e->dy.begin(), e->dy.end());
            Cs.push_back(at(e->weight).grad.ptr);
            Ms.push_back(e->in);
            Ns.push_back(e->out);
        }
        rc = eisen_hip_gemm_grouped_ksegments(ctx_, Cs.size(), l.pieces, As.data(), Bs.data(), Cs.data(), Ms.data(), Ns.data(), l.rows, l.acc);
        if (rc) break;
    }
    // the operands go back to the pool (stream order keeps them intact until the launches above have read them)
    if (all) release_retained();
    check(rc, "weight gradients of the window");
}

void Graph::side_join() {
    check(eisen_hip_side_wait(ctx_), "side stream join");
    side_guards.clear();
    side_written_.clear();
    if (window_dw.empty()) release_retained();  // operands of side-stream GEMMs: what the main stream does next is ordered after them
}

void Graph::release_retained() {
    if (retained_.empty()) return;
    std::unordered_map<const void*, bool> held;
    held.swap(retained_);
    for (auto& kv : held)
        if (kv.second) (void)eisen_hip_free(ctx_, const_cast<void*>(kv.first));
}

// a weight gradient of fewer 128 x 128 tiles than the chip has CUs, formed by its own backward pass (no window)
bool Graph::beside_fits(size_t in, size_t out) const {
    return beside_ && window_ < 2 && precision_mode == PrecisionMode::Bf16Mixed && ((in + 127) / 128) * ((out + 127) / 128) < 256;
}

void Graph::run_beside(bool beside, const std::vector<const void*>& reads, const std::vector<size_t>& weights, const std::function<int()>& launch,
                       const char* what) {
    if (!beside) {
        check(launch(), what);
        return;
    }
    check(eisen_hip_side_begin(ctx_), "side stream");
    in_beside_ = true;
    int rc = 0;
    try {
        rc = launch();
    } catch (...) {
        in_beside_ = false;
        (void)eisen_hip_side_end(ctx_);
        throw;
    }
    in_beside_ = false;
    const int rc_end = eisen_hip_side_end(ctx_);  // back on the main stream whatever the launch returned
    for (const void* p : reads) retained_.emplace(p, false);
    for (size_t w : weights)
        if (std::find(side_written_.begin(), side_written_.end(), w) == side_written_.end()) side_written_.push_back(w);
    check(rc, what);
    check(rc_end, "side stream");
}

const Storage& Graph::grad_for_read(size_t id) {
    Tensor& t = at(id);
    materialize_grad(id);
    if (!t.grad.valid()) throw Error("backward: tensor " + std::to_string(id) + " has no gradient to read");
    return t.grad;
}

void Graph::request_zero_grad(size_t id) {
    if (!window_dw.empty() && at(id).is_param) flush_weight_gradients();  // what the window holds is added first, then cleared with the rest
    Tensor& t = at(id);
    if (t.is_param) t.grad_zero_pending = true;
    else if (t.grad.valid()) check(eisen_hip_memset_zero(ctx_, t.grad.ptr, t.grad.numel * (t.grad.dtype == EISEN_BF16 ? 2 : 4)), "zero_grad");
}

void Graph::materialize_grad(size_t id) {
    if (!window_dw.empty() && at(id).is_param) flush_weight_gradients();  // a parameter's gradient is about to be read
    apply_pending_zero(id);
}

void Graph::apply_pending_zero(size_t id) {
    if (!side_written_.empty() && std::find(side_written_.begin(), side_written_.end(), id) != side_written_.end()) side_join();
    Tensor& t = at(id);
    if (t.grad_zero_pending) {
        check(eisen_hip_memset_zero(ctx_, t.grad.ptr, t.grad.numel * sizeof(float)), "zero_grad");
        t.grad_zero_pending = false;
    }
}

// Graph::backward (src/graph/mod.rs:670-796): seed every element of the loss gradient with 1,
// replay the tape in reverse insertion order, keep the tape.  No per-node synchronisation:
// everything is ordered by the one stream.
void Graph::backward(size_t loss_id) {
    if (no_grad) return;
    backward_root_ = loss_id;
    backward_epoch_++;
    int acc = 0;
    Storage& lg = grad_for_write(loss_id, &acc);
    check(eisen_hip_fill(ctx_, lg.ptr, lg.dtype, 1.0f, lg.numel), "backward seed");
    backward_nodes_from(0);
    backward_root_ = (size_t)-1;
    flush_norm_dw(true);
    side_join();
    if (!pending_dw.empty()) {
        pending_dw.clear();
        throw Error("backward: a deferred weight gradient was not collected by a matmul_group");
    }
    if (!window_dw.empty() && ++window_passes_ >= window_) flush_weight_gradients();
}

void Graph::backward_nodes_from(size_t first_node) {
    for (size_t i = tape.nodes.size(); i-- > first_node;) {
        const Tensor& out = at(tape.nodes[i].output);
        // an output nobody differentiated through has a zero gradient: nothing to propagate
        if (!out.is_param && !(out.grad.valid() && out.grad_written)) continue;
        // a copy: the closure may record further nodes (a recomputed block), which can move the tape's storage
        const std::function<void(Graph&)> fn = tape.nodes[i].backward_fn;
        fn(*this);
    }
}

// ---- elementwise ---------------------------------------------------------------------------------

// Graph::add / Graph::mul (src/graph/ops/elementwise.rs:15-183, :188-331).
size_t Graph::elementwise_binary(size_t a, size_t b, bool is_mul) {
    const std::vector<size_t> sa = at(a).shape, sb = at(b).shape;
    const Storage da = compute_data(a), db = compute_data(b);
    if (da.dtype != db.dtype) throw Error(std::string(is_mul ? "mul" : "add") + ": operands have different element types");
    const int dtype = da.dtype;
    const std::vector<size_t> os = broadcasted_shape(sa, sb);
    if (os.size() > 4) throw Error("add/mul: rank above 4 is not supported");
    const size_t n = numel_of(os);
    const size_t out = push_tensor(os, dtype, true);
    const bool same = sa == os && sb == os;
    const std::vector<size_t> sta = broadcasted_strides(sa, compute_strides(sa), os), stb = broadcasted_strides(sb, compute_strides(sb), os);
    if (same) {
        check(is_mul ? eisen_hip_mul(ctx_, da.ptr, db.ptr, at(out).data.ptr, dtype, n) : eisen_hip_add(ctx_, da.ptr, db.ptr, at(out).data.ptr, dtype, n),
              is_mul ? "mul" : "add");
    } else {
        const std::vector<size_t> osv = os.empty() ? std::vector<size_t>{1} : os;
        std::vector<size_t> xa = sta, xb = stb;
        if (os.empty()) { xa = {0}; xb = {0}; }
        check(is_mul ? eisen_hip_mul_bcast(ctx_, da.ptr, db.ptr, at(out).data.ptr, dtype, (int)osv.size(), osv.data(), xa.data(), xb.data())
                     : eisen_hip_add_bcast(ctx_, da.ptr, db.ptr, at(out).data.ptr, dtype, (int)osv.size(), osv.data(), xa.data(), xb.data()),
              is_mul ? "mul (broadcast)" : "add (broadcast)");
    }
    record({a, b}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        auto one_side = [&](size_t self, size_t other, const std::vector<size_t>& self_shape, const std::vector<size_t>& self_st,
                            const std::vector<size_t>& other_st) {
            int acc = 0;
            Storage& gs = g.grad_for_write(self, &acc);
            const Storage od = g.compute_data(other);
            if (gs.dtype != go.dtype) {
                // a parameter operand in mixed precision (a Linear bias): bf16 dOut, f32 parameter gradient
                if (gs.dtype != EISEN_F32) throw Error("add/mul backward: gradient element types differ");
                const std::vector<size_t> osv = os.empty() ? std::vector<size_t>{1} : os;
                std::vector<size_t> st_self = self_st, st_other = other_st;
                if (os.empty()) { st_self = {1}; st_other = {0}; }
                g.check(eisen_hip_bcast_backward_f32(g.ctx(), (float*)gs.ptr, go.ptr, is_mul ? od.ptr : nullptr, dtype, (int)osv.size(), osv.data(), st_self.data(),
                                                     is_mul ? st_other.data() : nullptr, numel_of(self_shape), acc),
                        "add/mul backward (f32 parameter gradient)");
                return;
            }
            if (self_shape == os) {
                if (is_mul) {
                    // ga (+)= other * go, expressed through mul_backward with the other side disabled
                    if (other_st == compute_strides(os)) {
                        g.check(eisen_hip_mul_backward(g.ctx(), od.ptr, od.ptr, go.ptr, gs.ptr, nullptr, dtype, n, acc, 0), "mul backward");
                    } else {
                        const std::vector<size_t> full = compute_strides(os);
                        g.check(eisen_hip_bcast_backward(g.ctx(), gs.ptr, go.ptr, od.ptr, dtype, (int)os.size(), os.data(), full.data(), other_st.data(), n, acc), "mul backward");
                    }
                } else {
                    g.check(eisen_hip_accumulate(g.ctx(), gs.ptr, go.ptr, dtype, n, acc), "add backward");
                }
            } else {
                const std::vector<size_t> osv = os.empty() ? std::vector<size_t>{1} : os;
                g.check(eisen_hip_bcast_backward(g.ctx(), gs.ptr, go.ptr, is_mul ? od.ptr : nullptr, dtype, (int)osv.size(), osv.data(), self_st.data(),
                                                 is_mul ? other_st.data() : nullptr, numel_of(self_shape), acc),
                        "broadcast backward");
            }
        };
        one_side(a, b, sa, sta, stb);  // when a == b both contributions land on the same buffer
        one_side(b, a, sb, stb, sta);
    });
    return out;
}
size_t Graph::add(size_t a, size_t b) { return elementwise_binary(a, b, false); }
size_t Graph::mul(size_t a, size_t b) { return elementwise_binary(a, b, true); }

// Graph::silu (src/graph/ops/elementwise.rs:337-465).
size_t Graph::silu(size_t a) {
    const Storage da = compute_data(a);
    const size_t out = push_tensor(at(a).shape, da.dtype, true);
    check(eisen_hip_silu(ctx_, da.ptr, at(out).data.ptr, da.dtype, da.numel), "silu");
    record({a}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_silu_backward(g.ctx(), g.compute_data(a).ptr, go.ptr, ga.ptr, go.dtype, go.numel, acc), "silu backward");
    });
    return out;
}

// silu(gate) * up in one pass each way: the gate/silu/up/mul part of
// TransformerBlock::forward_with_mask (src/nn/transformer.rs:40-43).
size_t Graph::swiglu(size_t gate, size_t up) {
    const Storage dg = compute_data(gate), du = compute_data(up);
    if (at(gate).shape != at(up).shape || dg.dtype != du.dtype) throw Error("swiglu: gate and up must have the same shape and type");
    const size_t out = push_tensor(at(gate).shape, dg.dtype, true);
    check(eisen_hip_swiglu(ctx_, dg.ptr, du.ptr, at(out).data.ptr, dg.dtype, dg.numel), "swiglu");
    record({gate, up}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int ag = 0, au = 0;
        Storage& gg = g.grad_for_write(gate, &ag);
        Storage& gu = g.grad_for_write(up, &au);
        g.check(eisen_hip_swiglu_backward(g.ctx(), g.compute_data(gate).ptr, g.compute_data(up).ptr, go.ptr, gg.ptr, gu.ptr, go.dtype, go.numel, ag, au),
                "swiglu backward");
    });
    return out;
}

// ---- contractions --------------------------------------------------------------------------------

// Graph::matmul / matmul_bf16 (src/graph/ops/linear.rs:8-297, :526-656): a [..., K] flattened to
// [M, K], b [K, N] -> [M, N].  dA += dC B^T, dB += A^T dC.
size_t Graph::matmul(size_t a, size_t b) {
    const std::vector<size_t> sa = at(a).shape, sb = at(b).shape;
    if (sb.size() != 2 || sa.empty()) throw Error("matmul: expects a [..,K] and b [K,N], got " + shape_str(sa) + " x " + shape_str(sb));
    const size_t K = sa.back(), M = numel_of(sa) / std::max<size_t>(K, 1), N = sb[1];
    if (sb[0] != K) throw Error("matmul: inner dimensions differ: " + shape_str(sa) + " x " + shape_str(sb));
    const Storage da = compute_data(a), db = compute_data(b);
    if (da.dtype != db.dtype) throw Error("matmul: operands have different element types");
    const size_t out = push_tensor({M, N}, da.dtype, true);
    check(eisen_hip_gemm(ctx_, da.ptr, db.ptr, at(out).data.ptr, da.dtype, da.dtype, 0, 0, M, N, K, 0), "matmul");
    record({a, b}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_gemm(g.ctx(), go.ptr, g.compute_data(b).ptr, ga.ptr, go.dtype, ga.dtype, 0, 1, M, K, N, acc), "matmul backward dA");
        if (g.window_take(b, g.compute_data(a).ptr, go.ptr, go.dtype, M, K, N)) return;
        const void* xa = g.compute_data(a).ptr;
        g.run_beside(g.at(b).is_param && g.beside_fits(K, N), {xa, go.ptr}, {b}, [&]() {
            int accb = 0;
            Storage& gb = g.grad_for_write(b, &accb);
            return eisen_hip_gemm(g.ctx(), xa, go.ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, K, N, M, accb);
        }, "matmul backward dB");
    });
    return out;
}

// Graph::matmul followed by Graph::add of a residual (src/nn/transformer.rs:36, :47) as one kernel:
// out = r + a b, with r and out [.., N].  Backward is that of the two ops: dR += dOut, dA += dOut B^T,
// dB += A^T dOut.
size_t Graph::matmul_residual(size_t a, size_t b, size_t r, bool defer_dw) {
    const std::vector<size_t> sa = at(a).shape, sb = at(b).shape, sr = at(r).shape;
    if (sb.size() != 2 || sa.empty() || sr.empty()) throw Error("matmul_residual: expects a [..,K], b [K,N], r [..,N]");
    const size_t K = sa.back(), M = numel_of(sa) / std::max<size_t>(K, 1), N = sb[1];
    if (sb[0] != K || sr.back() != N || numel_of(sr) != M * N) throw Error("matmul_residual: shapes do not match: " + shape_str(sa) + " x " + shape_str(sb) + " + " + shape_str(sr));
    const Storage da = compute_data(a), db = compute_data(b), dr = compute_data(r);
    if (da.dtype != db.dtype || dr.dtype != da.dtype) throw Error("matmul_residual: operands have different element types");
    const size_t out = push_tensor(sr, da.dtype, true);
    check(eisen_hip_gemm_residual(ctx_, da.ptr, db.ptr, dr.ptr, at(out).data.ptr, da.dtype, da.dtype, 0, 0, M, N, K), "matmul_residual");
    record({a, b, r}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Tensor& tr = g.at(r);
        Tensor& to = g.at(out);
        if (!tr.is_param && !tr.grad.valid() && !to.is_param && !to.grad_borrowed && tr.data.dtype == go.dtype) {
            // The first gradient to reach the residual is dOut itself: hand the buffer over instead of copying it.
            // Nothing reads dOut after this node (its consumers ran before it), and later contributions to dR
            // accumulate into the buffer in place.
            tr.grad = to.grad;
            tr.grad_written = true;
            to.grad_borrowed = true;
        } else {
            Storage& gr = g.grad_for_write(r, &acc);
            if (gr.dtype != go.dtype) throw Error("matmul_residual backward: gradient element types differ");
            if (gr.ptr == go.ptr) throw Error("matmul_residual backward: a second backward pass over the same activations is not supported");
            g.check(eisen_hip_accumulate(g.ctx(), gr.ptr, go.ptr, go.dtype, M * N, acc), "matmul_residual backward dR");
        }
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_gemm(g.ctx(), go.ptr, g.compute_data(b).ptr, ga.ptr, go.dtype, ga.dtype, 0, 1, M, K, N, acc), "matmul_residual backward dA");
        if (g.window_take(b, g.compute_data(a).ptr, go.ptr, go.dtype, M, K, N)) {
            // left for the window's launch; whoever adds to dOut's buffer (now dR's) next gets a fresh one
        } else if (defer_dw && go.dtype == EISEN_BF16 && g.at(b).is_param) {
            // dOut's buffer (now also dR's) is only added to by nodes that run after the collecting group
            g.pending_dw.push_back(PendingDW{b, g.compute_data(a).ptr, go.ptr, M, K, N});
        } else {
            const void* xa = g.compute_data(a).ptr;
            g.run_beside(g.at(b).is_param && g.beside_fits(K, N), {xa, go.ptr}, {b}, [&]() {
                int accb = 0;
                Storage& gb = g.grad_for_write(b, &accb);
                return eisen_hip_gemm(g.ctx(), xa, go.ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, K, N, M, accb);
            }, "matmul_residual backward dB");
        }
    });
    return out;
}

// The feed-forward tail of the transformer block, `ffn2(g.mul(g.silu(gate), up)) + res1` (src/nn/transformer.rs:44-47),
// as one node: forward = the SwiGLU kernel + the residual GEMM; backward = dR (buffer hand-over as in
// matmul_residual), dW += h^T dOut, and one GEMM whose epilogue turns dH = dOut W^T straight into dgate and dup
// (dH itself is never stored).
size_t Graph::swiglu_matmul_residual(size_t gate, size_t up, size_t b, size_t r, size_t h_in) {
    const std::vector<size_t> sg = at(gate).shape, sb = at(b).shape, sr = at(r).shape;
    if (sb.size() != 2 || sg.empty() || sr.empty() || at(up).shape != sg) throw Error("swiglu_matmul_residual: expects gate/up [..,K], b [K,N], r [..,N]");
    const size_t K = sg.back(), M = numel_of(sg) / std::max<size_t>(K, 1), N = sb[1];
    if (sb[0] != K || sr.back() != N || numel_of(sr) != M * N) throw Error("swiglu_matmul_residual: shapes do not match: " + shape_str(sg) + " x " + shape_str(sb) + " + " + shape_str(sr));
    const Storage dg = compute_data(gate), du = compute_data(up), db = compute_data(b), dr = compute_data(r);
    if (dg.dtype != du.dtype || dg.dtype != db.dtype || dr.dtype != dg.dtype) throw Error("swiglu_matmul_residual: operands have different element types");
    size_t h = h_in;  // kept for dW
    if (h == (size_t)-1) {
        h = push_tensor(sg, dg.dtype, true);
        check(eisen_hip_swiglu(ctx_, dg.ptr, du.ptr, at(h).data.ptr, dg.dtype, dg.numel), "swiglu");
    } else if (numel_of(at(h).shape) != dg.numel || at(h).data.dtype != dg.dtype) {
        throw Error("swiglu_matmul_residual: h does not match gate and up");
    }
    const size_t out = push_tensor(sr, dg.dtype, true);
    check(eisen_hip_gemm_residual(ctx_, at(h).data.ptr, db.ptr, dr.ptr, at(out).data.ptr, dg.dtype, dg.dtype, 0, 0, M, N, K), "swiglu_matmul_residual");
    record({gate, up, b, r}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Tensor& tr = g.at(r);
        Tensor& to = g.at(out);
        if (!tr.is_param && !tr.grad.valid() && !to.is_param && !to.grad_borrowed && tr.data.dtype == go.dtype) {
            tr.grad = to.grad;  // see matmul_residual
            tr.grad_written = true;
            to.grad_borrowed = true;
        } else {
            Storage& gr = g.grad_for_write(r, &acc);
            if (gr.dtype != go.dtype) throw Error("swiglu_matmul_residual backward: gradient element types differ");
            if (gr.ptr == go.ptr) throw Error("swiglu_matmul_residual backward: a second backward pass over the same activations is not supported");
            g.check(eisen_hip_accumulate(g.ctx(), gr.ptr, go.ptr, go.dtype, M * N, acc), "swiglu_matmul_residual backward dR");
        }
        // large products only: a small one gains nothing from running beside the chain
        const bool windowed = g.window_take(b, g.at(h).data.ptr, go.ptr, go.dtype, M, K, N);
        const bool side = !windowed && go.dtype == EISEN_BF16 && g.at(b).is_param && K % 256 == 0 && N % 128 == 0 && M % 64 == 0 && (K / 256) * (N / 128) >= 128;
        if (side) {
            // dB beside the input-gradient chain: it reads h and dOut; dOut's buffer (now dR's) is next written by whoever
            // accumulates into dR, and that write waits (grad_for_write)
            Storage& gb = g.grad_for_write(b, &acc);
            g.check(eisen_hip_side_begin(g.ctx()), "side stream");
            const int rc = eisen_hip_gemm(g.ctx(), g.at(h).data.ptr, go.ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, K, N, M, acc);
            const int rc_end = eisen_hip_side_end(g.ctx());  // back on the main stream whatever the GEMM returned
            g.side_guards.push_back(go.ptr);
            g.check(rc, "swiglu_matmul_residual backward dB");
            g.check(rc_end, "side stream");
        }
        int ag = 0, au = 0;
        Storage& gg = g.grad_for_write(gate, &ag);
        Storage& gu = g.grad_for_write(up, &au);
        const Storage wb = g.compute_data(b);
        if (!ag && !au && gg.dtype == go.dtype && gu.dtype == go.dtype) {
            g.check(eisen_hip_gemm_swiglu_backward(g.ctx(), go.ptr, wb.ptr, g.compute_data(gate).ptr, g.compute_data(up).ptr, gg.ptr, gu.ptr, go.dtype, 0, 1, M,
                                                   K, N),
                    "swiglu_matmul_residual backward dgate/dup");
        } else {  // gate or up already carries a gradient: dH through a temporary, then the accumulating element-wise kernel
            Storage dh = g.device_alloc(M * K, go.dtype, false);
            g.check(eisen_hip_gemm(g.ctx(), go.ptr, wb.ptr, dh.ptr, go.dtype, go.dtype, 0, 1, M, K, N, 0), "swiglu_matmul_residual backward dH");
            g.check(eisen_hip_swiglu_backward(g.ctx(), g.compute_data(gate).ptr, g.compute_data(up).ptr, dh.ptr, gg.ptr, gu.ptr, go.dtype, M * K, ag, au),
                    "swiglu_matmul_residual backward");
            g.device_free(dh);
        }
        if (!side && !windowed) {
            const void* xh = g.at(h).data.ptr;
            g.run_beside(g.at(b).is_param && g.beside_fits(K, N), {xh, go.ptr}, {b}, [&]() {
                int accb = 0;
                Storage& gb = g.grad_for_write(b, &accb);
                return eisen_hip_gemm(g.ctx(), xh, go.ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, K, N, M, accb);
            }, "swiglu_matmul_residual backward dB");
        }
    });
    return out;
}

// Several Graph::matmul calls that share their left operand (Q/K/V projections, gate and up projections:
// src/nn/attention.rs:300-302, src/nn/transformer.rs:41-44), with the results of the separate matmuls but
// fewer launches: equally shaped neighbours (K and V, gate and up) run as a batch of two whose "stride" is the
// distance between the two tensors, forward and for dW; the input gradient of the whole group is one GEMM
// whose contraction runs over the outputs of all members, written once.
std::vector<size_t> Graph::matmul_group(size_t a, const std::vector<size_t>& ws, const std::vector<size_t>& collect_dw, size_t* swiglu_h, bool defer_dw,
                                        size_t rope_members, size_t rope_head_dim, bool* rotated) {
    const std::vector<size_t> sa = at(a).shape;
    const size_t n = ws.size();
    if (rotated) *rotated = false;
    const Storage da = compute_data(a);
    bool ok = n >= 2 && n <= 3 && !sa.empty() && da.dtype == EISEN_BF16;
    for (size_t i = 0; i < n && ok; i++)
        ok = at(ws[i]).shape.size() == 2 && at(ws[i]).shape[0] == sa.back() && compute_data(ws[i]).dtype == da.dtype &&
             std::count(ws.begin(), ws.end(), ws[i]) == 1;
    if (!ok) {
        std::vector<size_t> outs;
        for (size_t w : ws) outs.push_back(matmul(a, w));
        if (swiglu_h) *swiglu_h = (size_t)-1;
        return outs;
    }
    const size_t K = sa.back(), M = numel_of(sa) / std::max<size_t>(K, 1);
    std::vector<size_t> outs(n), N(n);
    for (size_t i = 0; i < n; i++) {
        N[i] = at(ws[i]).shape[1];
        outs[i] = push_tensor({M, N[i]}, da.dtype, true);
    }
    // pair[i]: member i runs batched with member i+1
    std::vector<char> pair(n, 0);
    auto congruent = [](const void* p, const void* q, size_t elem) { return ((const char*)q - (const char*)p) % (ptrdiff_t)(8 * elem) == 0; };
    for (size_t i = 0; i + 1 < n; i++)
        if (!(i > 0 && pair[i - 1]) && at(ws[i]).shape == at(ws[i + 1]).shape &&
            congruent(compute_data(ws[i]).ptr, compute_data(ws[i + 1]).ptr, 2) && congruent(at(outs[i]).data.ptr, at(outs[i + 1]).data.ptr, 2))
            pair[i] = 1;
    // shapes whose gate|up + SwiGLU kernel exists (eisen_hip_gemm_swiglu_forward would otherwise run three launches
    // where the batched pair below and the SwiGLU kernel are two)
    const bool with_h = swiglu_h && n == 2 && N[0] == N[1] && M % 256 == 0 && N[0] % 128 == 0 && K % 32 == 0 && (M / 256) * (N[0] / 128) >= 256;
    if (swiglu_h) *swiglu_h = with_h ? push_tensor({M, N[0]}, da.dtype, true) : (size_t)-1;
    if (with_h)
        check(eisen_hip_gemm_swiglu_forward(ctx_, da.ptr, compute_data(ws[0]).ptr, compute_data(ws[1]).ptr, at(outs[0]).data.ptr, at(outs[1]).data.ptr,
                                            at(*swiglu_h).data.ptr, da.dtype, M, N[0], K),
              "matmul_group");
    // rotary embedding of the first outputs by the kernel that forms them ([batch, seq, hidden] inputs, whole heads)
    size_t rope_n = (rotated && !swiglu_h && sa.size() == 3 && sa[1] > 0 && rope_head_dim >= 8 && rope_head_dim % 8 == 0) ? std::min(rope_members, n) : 0;
    for (size_t i = 0; i < rope_n; i++)
        if (N[i] % rope_head_dim) rope_n = 0;
    if (rope_n > 0) *rotated = true;
    const size_t seq = sa.size() == 3 ? sa[1] : 0;
    for (size_t i = 0; i < n && !with_h; i++) {
        const Storage w = compute_data(ws[i]);
        if (pair[i]) {
            const ptrdiff_t wd = ((const char*)compute_data(ws[i + 1]).ptr - (const char*)w.ptr) / 2;
            const ptrdiff_t od = ((const char*)at(outs[i + 1]).data.ptr - (const char*)at(outs[i]).data.ptr) / 2;
            const size_t members = (i < rope_n ? 1 : 0) + (i + 1 < rope_n ? 1 : 0);
            if (members > 0)
                check(eisen_hip_gemm_rope(ctx_, da.ptr, w.ptr, at(outs[i]).data.ptr, da.dtype, 2, M, N[i], K, wd, od, members, seq, rope_head_dim), "matmul_group");
            else
                check(eisen_hip_gemm_strided_batched(ctx_, da.ptr, w.ptr, at(outs[i]).data.ptr, da.dtype, da.dtype, 0, 0, 2, M, N[i], K, 0, wd, od, 0), "matmul_group");
            i++;
        } else if (i < rope_n) {
            check(eisen_hip_gemm_rope(ctx_, da.ptr, w.ptr, at(outs[i]).data.ptr, da.dtype, 1, M, N[i], K, 0, 0, 1, seq, rope_head_dim), "matmul_group");
        } else {
            check(eisen_hip_gemm(ctx_, da.ptr, w.ptr, at(outs[i]).data.ptr, da.dtype, da.dtype, 0, 0, M, N[i], K, 0), "matmul_group");
        }
    }
    auto epoch = std::make_shared<size_t>((size_t)-1);
    auto fn = [=](Graph& g) {
        if (*epoch == g.backward_epoch()) return;  // the node is on the tape once per output; it runs once per backward
        *epoch = g.backward_epoch();
        std::vector<char> has(n);
        bool all = true;
        for (size_t i = 0; i < n; i++) {
            has[i] = g.has_grad(outs[i]);
            all = all && has[i];
        }
        // dA (+)= sum_i dY_i W_i^T, the last member first as the reversed tape of separate matmuls would
        {
            int acc = 0;
            Storage& ga = g.grad_for_write(a, &acc);
            const void* As[3];
            const void* Bs[3];
            size_t Ks[3];
            size_t m = 0;
            for (size_t i = n; i-- > 0;) {
                if (!has[i]) continue;
                As[m] = g.grad_for_read(outs[i]).ptr;
                Bs[m] = g.compute_data(ws[i]).ptr;
                Ks[m] = N[i];
                m++;
            }
            if (m > 0)
                g.check(eisen_hip_gemm_ksegments(g.ctx(), m, As, Bs, Ks, ga.ptr, EISEN_BF16, ga.dtype, 0, 1, M, K, acc), "matmul_group backward dA");
        }
        // dW_i (+)= A^T dY_i.  First choice: every member, and the deferred gradients this group collects, as one grouped
        // launch (same rows, same input width, same accumulate state, f32 gradients).
        const Storage xa = g.compute_data(a);
        if (all) {
            // every member joins the window or none: a group split between the window and this pass gains nothing
            bool fits = true;
            for (size_t i = 0; i < n; i++) fits = fits && g.window_fits(ws[i], EISEN_BF16, M, K, N[i]);
            if (fits) {
                for (size_t i = 0; i < n; i++) g.window_take(ws[i], xa.ptr, g.grad_for_read(outs[i]).ptr, EISEN_BF16, M, K, N[i]);
                for (size_t e = 0; e < g.pending_dw.size();) {  // gradients this group was to collect (none in a model whose layers all join the window)
                    const PendingDW p = g.pending_dw[e];
                    if (std::find(collect_dw.begin(), collect_dw.end(), p.weight) == collect_dw.end()) {
                        e++;
                        continue;
                    }
                    g.pending_dw.erase(g.pending_dw.begin() + (ptrdiff_t)e);
                    int acc = 0;
                    Storage& gw = g.grad_for_write(p.weight, &acc);
                    g.check(eisen_hip_gemm(g.ctx(), p.x, p.dy, gw.ptr, EISEN_BF16, gw.dtype, 1, 0, p.in, p.out, p.rows, acc), "deferred dW");
                }
                return;
            }
        }
        if (defer_dw && all && collect_dw.empty()) {
            // only products that the grouped launch takes as wide tiles are worth the wait: small ones are served better by
            // the batched pair below
            bool params = K % 256 == 0 && M % 64 == 0;
            size_t wide_tiles = 0;
            for (size_t i = 0; i < n; i++) {
                params = params && g.at(ws[i]).is_param && N[i] % 128 == 0 && g.at(ws[i]).grad.dtype == EISEN_F32;
                wide_tiles += (K / 256) * (N[i] / 128);
            }
            // (a narrow model's gate and up gradients stay here as well: joining the Q/K/V group's split-contraction launch
            // measured 8 % slower on the config-4 step than the batched pair)
            if (params && wide_tiles >= 300) {
                for (size_t i = 0; i < n; i++) g.pending_dw.push_back(PendingDW{ws[i], xa.ptr, g.grad_for_read(outs[i]).ptr, M, K, N[i]});
                return;
            }
        }
        std::vector<PendingDW> extras;
        for (size_t e = 0; e < g.pending_dw.size();) {
            if (std::find(collect_dw.begin(), collect_dw.end(), g.pending_dw[e].weight) != collect_dw.end()) {
                extras.push_back(g.pending_dw[e]);
                g.pending_dw.erase(g.pending_dw.begin() + (ptrdiff_t)e);
            } else {
                e++;
            }
        }
        bool done = false;
        bool fits = all && n + extras.size() >= 3 && n + extras.size() <= 8;
        for (const PendingDW& e : extras) fits = fits && e.rows == M && e.in == K;
        // (a plain pair of equal shapes stays with the batched launch below: the 256x128 tile serves it better)
        if (fits) {
            const void* As[8];
            const void* Bs[8];
            void* Cs[8];
            size_t Ns[8];
            int accs[8];
            int dts[8];
            size_t m = 0;
            bool same = true;
            for (size_t i = 0; i < n + extras.size(); i++) {
                const bool own = i < n;
                const size_t w = own ? ws[i] : extras[i - n].weight;
                As[m] = own ? xa.ptr : extras[i - n].x;
                Bs[m] = own ? g.grad_for_read(outs[i]).ptr : extras[i - n].dy;
                Storage& gw = g.grad_for_write(w, &accs[m]);
                same = same && gw.dtype == EISEN_F32;
                dts[m] = gw.dtype;
                Cs[m] = gw.ptr;
                Ns[m] = own ? N[i] : extras[i - n].out;
                m++;
            }
            for (size_t i = 1; i < m; i++) same = same && accs[i] == accs[0];
            // narrow products: beside the chain (the gradients were fetched above: a weight the side stream is still writing
            // has made the main stream wait there, which is safe and rare)
            std::vector<const void*> reads(As, As + m);
            reads.insert(reads.end(), Bs, Bs + m);
            std::vector<size_t> written;
            size_t tiles = 0;
            for (size_t i = 0; i < m; i++) {
                written.push_back(i < n ? ws[i] : extras[i - n].weight);
                tiles += ((K + 127) / 128) * ((Ns[i] + 127) / 128);
            }
            g.run_beside(tiles < 256 && g.beside_fits(K, 128), reads, written, [&]() {
                if (same) return eisen_hip_gemm_grouped(g.ctx(), m, As, Bs, Cs, Ns, EISEN_BF16, EISEN_F32, 1, 0, K, M, accs[0]);
                int rc = 0;  // same work, one launch per product (grad_for_write has already been consumed above)
                for (size_t i = 0; i < m && !rc; i++) rc = eisen_hip_gemm(g.ctx(), As[i], Bs[i], Cs[i], EISEN_BF16, dts[i], 1, 0, K, Ns[i], M, accs[i]);
                return rc;
            }, "matmul_group backward dW");
            done = true;
        } else {
            for (const PendingDW& e : extras) {
                int acc = 0;
                Storage& gw = g.grad_for_write(e.weight, &acc);
                g.run_beside(g.beside_fits(e.in, e.out), {e.x, e.dy}, {e.weight}, [&]() {
                    return eisen_hip_gemm(g.ctx(), e.x, e.dy, gw.ptr, EISEN_BF16, gw.dtype, 1, 0, e.in, e.out, e.rows, acc);
                }, "deferred dW");
            }
        }
        for (size_t i = 0; i < n && !done; i++) {
            if (pair[i] && has[i] && has[i + 1]) {
                const Storage& go1 = g.grad_for_read(outs[i]);
                const Storage& go2 = g.grad_for_read(outs[i + 1]);
                int acc1 = 0, acc2 = 0;
                Storage& g1 = g.grad_for_write(ws[i], &acc1);
                Storage& g2 = g.grad_for_write(ws[i + 1], &acc2);
                const size_t gs = g1.dtype == EISEN_BF16 ? 2 : 4;
                const ptrdiff_t gd = (const char*)g2.ptr - (const char*)g1.ptr, od = (const char*)go2.ptr - (const char*)go1.ptr;
                const bool beside = g.at(ws[i]).is_param && g.at(ws[i + 1]).is_param && g.beside_fits(K, 2 * N[i]);
                g.run_beside(beside, {xa.ptr, go1.ptr, go2.ptr}, {ws[i], ws[i + 1]}, [&]() {
                    if (acc1 == acc2 && g1.dtype == g2.dtype && gd % 16 == 0 && od % 16 == 0)
                        return eisen_hip_gemm_strided_batched(g.ctx(), xa.ptr, go1.ptr, g1.ptr, go1.dtype, g1.dtype, 1, 0, 2, K, N[i], M, 0, od / 2,
                                                              gd / (ptrdiff_t)gs, acc1);
                    const int rc = eisen_hip_gemm(g.ctx(), xa.ptr, go1.ptr, g1.ptr, go1.dtype, g1.dtype, 1, 0, K, N[i], M, acc1);
                    return rc ? rc : eisen_hip_gemm(g.ctx(), xa.ptr, go2.ptr, g2.ptr, go2.dtype, g2.dtype, 1, 0, K, N[i + 1], M, acc2);
                }, "matmul_group backward dW");
                i++;
            } else if (has[i]) {
                const Storage& go = g.grad_for_read(outs[i]);
                int acc = 0;
                Storage& gb = g.grad_for_write(ws[i], &acc);
                g.run_beside(g.at(ws[i]).is_param && g.beside_fits(K, N[i]), {xa.ptr, go.ptr}, {ws[i]}, [&]() {
                    return eisen_hip_gemm(g.ctx(), xa.ptr, go.ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, K, N[i], M, acc);
                }, "matmul_group backward dW");
            }
        }
        (void)all;
    };
    for (size_t i = 0; i < n; i++) record(std::vector<size_t>(ws.begin(), ws.end()), outs[i], fn);
    return outs;
}

// Graph::matmul_trans_b (src/graph/ops/linear.rs:301-523; GPU arm semantics): C = A B^T with
// b stored [N, K]; dA += dC B, dB += dC^T A.  Leading dims of a are kept.
size_t Graph::matmul_trans_b(size_t a, size_t b) {
    const std::vector<size_t> sa = at(a).shape, sb = at(b).shape;
    if (sb.size() != 2 || sa.empty()) throw Error("matmul_trans_b: expects a [..,K] and b [N,K]");
    const size_t K = sa.back(), M = numel_of(sa) / std::max<size_t>(K, 1), N = sb[0];
    if (sb[1] != K) throw Error("matmul_trans_b: inner dimensions differ: " + shape_str(sa) + " x " + shape_str(sb) + "^T");
    const Storage da = compute_data(a), db = compute_data(b);
    if (da.dtype != db.dtype) throw Error("matmul_trans_b: operands have different element types");
    std::vector<size_t> os = sa;
    os.back() = N;
    const size_t out = push_tensor(os, da.dtype, true);
    check(eisen_hip_gemm(ctx_, da.ptr, db.ptr, at(out).data.ptr, da.dtype, da.dtype, 0, 1, M, N, K, 0), "matmul_trans_b");
    record({a, b}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_gemm(g.ctx(), go.ptr, g.compute_data(b).ptr, ga.ptr, go.dtype, ga.dtype, 0, 0, M, K, N, acc), "matmul_trans_b backward dA");
        const void* xa = g.compute_data(a).ptr;
        g.run_beside(g.at(b).is_param && g.beside_fits(N, K), {go.ptr, xa}, {b}, [&]() {
            int accb = 0;
            Storage& gb = g.grad_for_write(b, &accb);
            return eisen_hip_gemm(g.ctx(), go.ptr, xa, gb.ptr, go.dtype, gb.dtype, 1, 0, N, K, M, accb);
        }, "matmul_trans_b backward dB");
    });
    return out;
}

// Graph::bmm (src/graph/ops/linear.rs:1198-1511): a [B,M,K]; b [B,N,K] if trans_b else [B,K,N].
size_t Graph::bmm(size_t a, size_t b, bool trans_b) {
    const std::vector<size_t> sa = at(a).shape, sb = at(b).shape;
    if (sa.size() != 3 || sb.size() != 3 || sa[0] != sb[0]) throw Error("bmm: expects [B,M,K] and [B,N,K]/[B,K,N]");
    const size_t B = sa[0], M = sa[1], K = sa[2], N = trans_b ? sb[1] : sb[2];
    if ((trans_b ? sb[2] : sb[1]) != K) throw Error("bmm: inner dimensions differ");
    const Storage da = compute_data(a), db = compute_data(b);
    if (da.dtype != db.dtype) throw Error("bmm: operands have different element types");
    const size_t out = push_tensor({B, M, N}, da.dtype, true);
    check(eisen_hip_bmm(ctx_, da.ptr, db.ptr, at(out).data.ptr, da.dtype, da.dtype, 0, trans_b ? 1 : 0, B, M, N, K, 0), "bmm");
    record({a, b}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        // dA = dC * B (trans_b: B is [N,K]) or dC * B^T (B is [K,N])
        g.check(eisen_hip_bmm(g.ctx(), go.ptr, g.compute_data(b).ptr, ga.ptr, go.dtype, ga.dtype, 0, trans_b ? 0 : 1, B, M, K, N, acc), "bmm backward dA");
        Storage& gb = g.grad_for_write(b, &acc);
        if (trans_b)  // dB [N,K] = dC^T * A
            g.check(eisen_hip_bmm(g.ctx(), go.ptr, g.compute_data(a).ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, B, N, K, M, acc), "bmm backward dB");
        else          // dB [K,N] = A^T * dC
            g.check(eisen_hip_bmm(g.ctx(), g.compute_data(a).ptr, go.ptr, gb.ptr, go.dtype, gb.dtype, 1, 0, B, K, N, M, acc), "bmm backward dB");
    });
    return out;
}

// ---- reductions / loss ---------------------------------------------------------------------------

// Graph::softmax (src/graph/ops/reduction.rs:397-523), over the last dim.
size_t Graph::softmax(size_t a) {
    const std::vector<size_t> sa = at(a).shape;
    if (sa.empty()) throw Error("softmax: scalar input");
    const size_t n = sa.back(), rows = numel_of(sa) / std::max<size_t>(n, 1);
    const Storage da = compute_data(a);
    const size_t out = push_tensor(sa, da.dtype, true);
    check(eisen_hip_softmax(ctx_, da.ptr, at(out).data.ptr, da.dtype, rows, n), "softmax");
    record({a}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_softmax_backward(g.ctx(), g.at(out).data.ptr, go.ptr, ga.ptr, go.dtype, rows, n, acc), "softmax backward");
    });
    return out;
}

// Graph::cross_entropy_masked (src/graph/ops/reduction.rs:724-944); Graph::cross_entropy is the
// case without masked rows (:529-716).  The gradient of the logits is produced by the forward
// kernel in the same pass; the recorded backward only rescales it when the loss is not the root.
size_t Graph::cross_entropy_masked(size_t logits, const std::vector<int64_t>& targets) {
    const std::vector<size_t> sl = at(logits).shape;
    if (sl.size() != 2) throw Error("cross_entropy: logits must be [rows, classes], got " + shape_str(sl));
    const size_t rows = sl[0], classes = sl[1];
    if (targets.size() != rows) throw Error("cross_entropy: " + std::to_string(targets.size()) + " targets for " + std::to_string(rows) + " rows");
    std::vector<int32_t> t32(rows);
    size_t valid = 0;
    for (size_t i = 0; i < rows; i++) {
        if (targets[i] == (int64_t)-1) {
            t32[i] = EISEN_IGNORE_INDEX;
        } else {
            if (targets[i] < 0 || (size_t)targets[i] >= classes)
                throw Error("cross_entropy: target " + std::to_string(targets[i]) + " at row " + std::to_string(i) + " outside [0, " + std::to_string(classes) + ")");
            t32[i] = (int32_t)targets[i];
            valid++;
        }
    }
    const size_t out = push_tensor({}, EISEN_F32, true);
    if (valid == 0) {  // src/graph/ops/reduction.rs:737-741: zero loss, no tape node
        check(eisen_hip_fill(ctx_, at(out).data.ptr, EISEN_F32, 0.0f, 1), "cross_entropy");
        return out;
    }
    const float normalizer = 1.0f / (float)valid;
    const Storage dl = compute_data(logits);
    Storage tgt = device_alloc(rows, EISEN_F32, false);  // int32 payload
    check(eisen_hip_htod(ctx_, tgt.ptr, t32.data(), rows * sizeof(int32_t)), "cross_entropy targets");
    Storage row_loss = device_alloc(rows, EISEN_F32, false);
    // Fast path: the logits are a fresh activation, so their gradient buffer is created here and the
    // kernel writes straight into it.  Otherwise (a leaf that already owns a gradient, or no_grad) the
    // gradient goes to a pooled side tensor and is added in backward.
    Tensor& tl = at(logits);
    const bool direct = !no_grad && !tl.is_param && !tl.grad.valid();
    size_t side = (size_t)-1;
    void* dlogits = nullptr;
    if (direct) {
        int acc = 0;
        dlogits = grad_for_write(logits, &acc).ptr;
    } else {
        side = push_tensor(sl, dl.dtype, true);
        dlogits = at(side).data.ptr;
    }
    check(eisen_hip_cross_entropy(ctx_, dl.ptr, (const int32_t*)tgt.ptr, dlogits, (float*)row_loss.ptr, (float*)at(out).data.ptr, nullptr, nullptr,
                                  dl.dtype, rows, classes, normalizer, 1.0f),
          "cross_entropy");
    device_free(tgt);  // stream-ordered: reused only by later work
    device_free(row_loss);
    record({logits}, out, [=](Graph& g) {
        const bool scale = g.backward_root() != out;  // seed 1: the stored gradient is already final
        if (direct) {
            if (!scale) return;
            Storage& gl = g.at(logits).grad;
            g.check(eisen_hip_scale_by_device_scalar(g.ctx(), gl.ptr, gl.dtype, (const float*)g.grad_for_read(out).ptr, gl.numel), "cross_entropy backward");
            return;
        }
        Storage& sd = g.at(side).data;
        if (scale) g.check(eisen_hip_scale_by_device_scalar(g.ctx(), sd.ptr, sd.dtype, (const float*)g.grad_for_read(out).ptr, sd.numel), "cross_entropy backward");
        int acc = 0;
        Storage& gl = g.grad_for_write(logits, &acc);
        if (gl.dtype == sd.dtype) {
            g.check(eisen_hip_accumulate(g.ctx(), gl.ptr, sd.ptr, sd.dtype, sd.numel, acc), "cross_entropy backward");
        } else {  // f32 leaf gradient, bf16 logits
            Storage tmp = g.device_alloc(sd.numel, gl.dtype, false);
            g.check(eisen_hip_cast(g.ctx(), sd.ptr, sd.dtype, tmp.ptr, gl.dtype, sd.numel), "cross_entropy backward");
            g.check(eisen_hip_accumulate(g.ctx(), gl.ptr, tmp.ptr, gl.dtype, sd.numel, acc), "cross_entropy backward");
            g.device_free(tmp);
        }
    });
    return out;
}
size_t Graph::cross_entropy(size_t logits, const std::vector<int64_t>& targets) {
    for (int64_t t : targets)
        if (t == (int64_t)-1) throw Error("cross_entropy: IGNORE_INDEX target; use cross_entropy_masked");
    return cross_entropy_masked(logits, targets);
}

// ---- layout --------------------------------------------------------------------------------------

// Graph::transpose_0213 (src/graph/ops/transform.rs:7-127).
size_t Graph::transpose_0213(size_t a) {
    const std::vector<size_t> sa = at(a).shape;
    if (sa.size() != 4) throw Error("transpose_0213 requires a 4-D tensor");
    const size_t b = sa[0], s = sa[1], h = sa[2], d = sa[3];
    const Storage da = compute_data(a);
    const size_t out = push_tensor({b, h, s, d}, da.dtype, true);
    check(eisen_hip_transpose_0213(ctx_, da.ptr, at(out).data.ptr, da.dtype, b, s, h, d, 0), "transpose_0213");
    record({a}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_transpose_0213(g.ctx(), go.ptr, ga.ptr, go.dtype, b, h, s, d, acc), "transpose_0213 backward");
    });
    return out;
}

// Graph::gather (src/graph/ops/transform.rs:132-324).  Indices are a tensor of f32 ids loaded from
// the host (`as usize` truncation, :294); the host copy is checked against the vocabulary here, the int32 copy on the
// device feeds the gather and the deterministic backward scatter.
size_t Graph::gather(size_t weights, size_t indices) {
    const std::vector<size_t> sw = at(weights).shape;
    if (sw.size() != 2) throw Error("gather: weights must be [vocab, hidden]");
    const size_t vocab = sw[0], hidden = sw[1];
    Tensor& ti = at(indices);
    const size_t n = ti.size();
    if (ti.host_copy.size() != n) {
        std::vector<float> host = sync_to_cpu(indices);  // ids that never came from the host: read them back
        at(indices).host_copy = host;
    }
    std::vector<int32_t> ids(n);
    const std::vector<float>& hc = at(indices).host_copy;
    for (size_t i = 0; i < n; i++) {
        const float f = hc[i];
        if (!(f >= 0.0f) || (size_t)f >= vocab) throw Error("gather: index " + std::to_string(f) + " at position " + std::to_string(i) + " outside [0, " + std::to_string(vocab) + ")");
        ids[i] = (int32_t)f;
    }
    const Storage dw = compute_data(weights);
    std::vector<size_t> os = at(indices).shape;
    os.push_back(hidden);
    // the ids as int32 on the device: a pooled tensor, so that the backward pass finds them there and they leave with
    // the activations
    const size_t dids = push_tensor({n}, EISEN_F32, true);  // int32 payload
    const size_t out = push_tensor(os, dw.dtype, true);
    check(eisen_hip_htod(ctx_, at(dids).data.ptr, ids.data(), n * sizeof(int32_t)), "gather ids");
    check(eisen_hip_gather(ctx_, dw.ptr, (const int32_t*)at(dids).data.ptr, at(out).data.ptr, dw.dtype, n, vocab, hidden), "gather");
    // The position index of the backward scatter depends on the ids alone: it is built now, on the side stream beside the
    // forward pass (one workgroup sorting for tens of microseconds), instead of in front of the last kernel of the backward pass.
    size_t didx = (size_t)-1;
    if (!no_grad && !tape_paused && beside_) {
        didx = push_tensor({3 * n}, EISEN_F32, true);  // int32 payload
        check(eisen_hip_side_begin(ctx_), "side stream");
        const int rc = eisen_hip_gather_index_dev(ctx_, (const int32_t*)at(dids).data.ptr, n, vocab, (int32_t*)at(didx).data.ptr);
        const int rc_end = eisen_hip_side_end(ctx_);  // back on the main stream whatever the call returned
        side_guards.push_back(at(didx).data.ptr);     // a restore_save_point before any backward pass waits for the sort
        if (rc == EISEN_E_SHAPE) didx = (size_t)-1;   // a batch the device-side index does not take: backward builds it its own way
        else check(rc, "gather index");
        check(rc_end, "side stream");
    }
    record({weights, indices}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        g.apply_pending_zero(weights);  // the scatter touches only the rows that occur
        Tensor& w = g.at(weights);
        if (!w.is_param) {
            int acc = 0;
            Storage& gw0 = g.grad_for_write(weights, &acc);
            if (!acc) g.check(eisen_hip_memset_zero(g.ctx(), gw0.ptr, gw0.numel * (gw0.dtype == EISEN_BF16 ? 2 : 4)), "gather backward");
        }
        if (w.grad.dtype != EISEN_F32) throw Error("gather backward: the embedding gradient must be f32");
        int rc = EISEN_E_SHAPE;
        if (didx != (size_t)-1) {
            g.side_join();  // the index (and whatever else the side stream was given) is complete
            rc = eisen_hip_gather_backward_indexed(g.ctx(), (const int32_t*)g.at(didx).data.ptr, go.ptr, (float*)w.grad.ptr, go.dtype, n, vocab, hidden);
        }
        if (rc == EISEN_E_SHAPE)  // no index, or rows the indexed kernel does not take
            rc = eisen_hip_gather_backward_dev(g.ctx(), (const int32_t*)g.at(dids).data.ptr, go.ptr, (float*)w.grad.ptr, go.dtype, n, vocab, hidden);
        g.check(rc, "gather backward");
    });
    return out;
}

// Graph::reshape (src/graph/ops/transform.rs:329-406): a copy with a new shape.
size_t Graph::reshape(size_t a, const std::vector<size_t>& shape) {
    if (numel_of(shape) != at(a).size()) throw Error("reshape: element count mismatch");
    const Storage da = compute_data(a);
    const size_t out = push_tensor(shape, da.dtype, true);
    check(eisen_hip_dtod(ctx_, at(out).data.ptr, da.ptr, da.numel * (da.dtype == EISEN_BF16 ? 2 : 4)), "reshape");
    record({a}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        if (ga.dtype != go.dtype) throw Error("reshape backward: gradient element types differ");
        g.check(eisen_hip_accumulate(g.ctx(), ga.ptr, go.ptr, go.dtype, go.numel, acc), "reshape backward");
    });
    return out;
}

// Graph::rope (src/graph/ops/transform.rs:467-610): a [batch, seq, hidden].
size_t Graph::rope(size_t a, size_t head_dim) {
    const std::vector<size_t> sa = at(a).shape;
    if (sa.size() != 3) throw Error("rope: expects [batch, seq, hidden]");
    const Storage da = compute_data(a);
    const size_t out = push_tensor(sa, da.dtype, true);
    check(eisen_hip_rope(ctx_, da.ptr, at(out).data.ptr, da.dtype, sa[0], sa[1], sa[2], head_dim), "rope");
    record({a}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& ga = g.grad_for_write(a, &acc);
        g.check(eisen_hip_rope_backward(g.ctx(), go.ptr, ga.ptr, go.dtype, sa[0], sa[1], sa[2], head_dim, acc), "rope backward");
    });
    return out;
}

// Graph::rms_norm (src/graph/ops/normalization.rs:8-184): the gain is an f32 parameter.
size_t Graph::rms_norm(size_t x, size_t w, float eps) {
    const std::vector<size_t> sx = at(x).shape;
    if (sx.empty()) throw Error("rms_norm: scalar input");
    const size_t dim = sx.back(), rows = numel_of(sx) / std::max<size_t>(dim, 1);
    if (at(w).size() != dim || at(w).data.dtype != EISEN_F32) throw Error("rms_norm: weight must be an f32 vector of the last dimension");
    const Storage dx = compute_data(x);
    const size_t out = push_tensor(sx, dx.dtype, true);
    const size_t rr = push_tensor({rows}, EISEN_F32, true);  // reciprocal RMS per row, kept for backward
    check(eisen_hip_rms_norm(ctx_, dx.ptr, (const float*)at(w).data.ptr, at(out).data.ptr, (float*)at(rr).data.ptr, dx.dtype, rows, dim, eps), "rms_norm");
    record({x, w}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        const void* add_to = nullptr;  // where the gradient so far is read from: the buffer written, or one that has to stay as it is
        Storage& gx = g.grad_for_write(x, &acc, &add_to);
        Tensor& tw = g.at(w);
        if (!tw.is_param) g.apply_pending_zero(w);
        if (!tw.grad.valid() || tw.grad.dtype != EISEN_F32) throw Error("rms_norm backward: the gain needs an f32 gradient buffer");
        if (tw.is_param) {
            // the gain gradient stays in partial rows until the end of the backward pass (flush_norm_dw)
            bool clash = g.pending_norm_dw.size() >= 64;
            for (const PendingNormDW& e : g.pending_norm_dw) clash = clash || e.weight == w || e.dim != dim;
            if (clash) g.flush_norm_dw(true);
            // a gradient still waiting to be cleared (zero_grad is lazy) is overwritten by the finishing launch
            PendingNormDW e{g.device_alloc((size_t)EISEN_RMS_NORM_PARTIAL_ROWS * dim, EISEN_F32, false), w, 0, dim, tw.grad_zero_pending};
            tw.grad_zero_pending = false;
            const int rc = acc ? eisen_hip_rms_norm_backward_partial_add(g.ctx(), g.compute_data(x).ptr, (const float*)tw.data.ptr,
                                                                         (const float*)g.at(rr).data.ptr, go.ptr, add_to, gx.ptr, (float*)e.partial.ptr,
                                                                         &e.nrows, go.dtype, rows, dim)
                               : eisen_hip_rms_norm_backward_partial(g.ctx(), g.compute_data(x).ptr, (const float*)tw.data.ptr,
                                                                     (const float*)g.at(rr).data.ptr, go.ptr, gx.ptr, (float*)e.partial.ptr, &e.nrows,
                                                                     go.dtype, rows, dim, 0);
            g.pending_norm_dw.push_back(e);  // before the check: the buffer is released with the list
            g.check(rc, "rms_norm backward");
        } else {
            if (acc && add_to != gx.ptr) g.check(eisen_hip_dtod(g.ctx(), gx.ptr, add_to, gx.numel * (gx.dtype == EISEN_BF16 ? 2 : 4)), "gradient copy");
            g.check(eisen_hip_rms_norm_backward(g.ctx(), g.compute_data(x).ptr, (const float*)tw.data.ptr, (const float*)g.at(rr).data.ptr, go.ptr, gx.ptr,
                                                (float*)tw.grad.ptr, go.dtype, rows, dim, acc),
                    "rms_norm backward");
        }
    });
    return out;
}

// Graph::repeat_kv (src/graph/ops/gqa.rs:13-194).
size_t Graph::repeat_kv(size_t x, size_t repeats) {
    const std::vector<size_t> sx = at(x).shape;
    if (sx.size() != 4) throw Error("repeat_kv requires [Batch, KVHeads, SeqLen, HeadDim]");
    if (repeats == 1) return x;
    const Storage dx = compute_data(x);
    const size_t out = push_tensor({sx[0], sx[1] * repeats, sx[2], sx[3]}, dx.dtype, true);
    check(eisen_hip_repeat_kv(ctx_, dx.ptr, at(out).data.ptr, dx.dtype, sx[0], sx[1], sx[2], sx[3], repeats), "repeat_kv");
    record({x}, out, [=](Graph& g) {
        const Storage& go = g.grad_for_read(out);
        int acc = 0;
        Storage& gx = g.grad_for_write(x, &acc);
        g.check(eisen_hip_repeat_kv_backward(g.ctx(), go.ptr, gx.ptr, go.dtype, sx[0], sx[1], sx[2], sx[3], repeats, acc), "repeat_kv backward");
    });
    return out;
}

// ---- attention -----------------------------------------------------------------------------------

size_t Graph::attention_impl(size_t q, size_t k, size_t v, size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd, const long long* qs,
                             const long long* ks, float scale, bool causal, const std::vector<size_t>& out_shape) {
    Graph& g = *this;
    const Storage dq = g.compute_data(q), dk = g.compute_data(k), dv = g.compute_data(v);
    if (dq.dtype != dk.dtype || dq.dtype != dv.dtype) throw Error("attention: q, k, v must share an element type");
    const size_t out = g.alloc_pooled_dtype(out_shape, dq.dtype);
    const size_t lse = g.alloc_pooled_dtype({B, Hq, S}, EISEN_F32);  // log-sum-exp per query row, kept for backward
    std::vector<long long> qsv, ksv;
    if (qs) qsv.assign(qs, qs + 3);
    if (ks) ksv.assign(ks, ks + 3);
    g.check(eisen_hip_attention_forward(g.ctx(), dq.ptr, dk.ptr, dv.ptr, g.at(out).data.ptr, (float*)g.at(lse).data.ptr, dq.dtype, B, S, Hq, Hkv, hd,
                                        qs ? qsv.data() : nullptr, ks ? ksv.data() : nullptr, scale, causal ? 1 : 0),
            "attention forward");
    record({q, k, v}, out, [=](Graph& gg) {
        const Storage& go = gg.grad_for_read(out);
        int aq = 0, ak = 0, av = 0;
        // the kernels overwrite: route through temporaries when a gradient is already there
        Storage& gq = gg.grad_for_write(q, &aq);
        Storage& gk = gg.grad_for_write(k, &ak);
        Storage& gv = gg.grad_for_write(v, &av);
        if (aq || ak || av) throw Error("attention backward: q, k, v must not have other consumers");
        gg.check(eisen_hip_attention_backward(gg.ctx(), gg.compute_data(q).ptr, gg.compute_data(k).ptr, gg.compute_data(v).ptr, gg.at(out).data.ptr, go.ptr,
                                              (const float*)gg.at(lse).data.ptr, gq.ptr, gk.ptr, gv.ptr, go.dtype, B, S, Hq, Hkv, hd,
                                              qsv.empty() ? nullptr : qsv.data(), ksv.empty() ? nullptr : ksv.data(), scale, causal ? 1 : 0),
                 "attention backward");
    });
    return out;
}

size_t Graph::attention_gqa(size_t q, size_t k, size_t v, size_t heads, size_t kv_heads, float scale, bool causal) {
    const std::vector<size_t> sq = at(q).shape, sk = at(k).shape;
    if (sq.size() != 3 || sk.size() != 3 || at(v).shape != sk) throw Error("attention_gqa: expects q [B,S,Hq*hd], k/v [B,S,Hkv*hd]");
    if (heads == 0 || kv_heads == 0 || sq[2] % heads || heads % kv_heads) throw Error("attention_gqa: bad head counts");
    const size_t hd = sq[2] / heads;
    if (sk[2] != kv_heads * hd || sk[0] != sq[0] || sk[1] != sq[1]) throw Error("attention_gqa: k/v shape does not match q");
    return attention_impl(q, k, v, sq[0], sq[1], heads, kv_heads, hd, nullptr, nullptr, scale, causal, sq);
}

// `g.rope(q)`, `g.rope(k)` and the attention chain (src/nn/attention.rs:316-375) as one node.  Forward: the two
// rotary kernels into internal tensors, then the fused attention.  Backward: one attention backward whose
// kernels un-rotate dQ and dK as they store them, so the gradients land directly on the projections.
size_t Graph::attention_gqa_rope(size_t q, size_t k, size_t v, size_t heads, size_t kv_heads, float scale, bool causal, bool prerotated) {
    const std::vector<size_t> sq = at(q).shape, sk = at(k).shape;
    if (sq.size() != 3 || sk.size() != 3 || at(v).shape != sk) throw Error("attention_gqa_rope: expects q [B,S,Hq*hd], k/v [B,S,Hkv*hd]");
    if (heads == 0 || kv_heads == 0 || sq[2] % heads || heads % kv_heads) throw Error("attention_gqa_rope: bad head counts");
    const size_t hd = sq[2] / heads, B = sq[0], S = sq[1];
    if (sk[2] != kv_heads * hd || sk[0] != B || sk[1] != S) throw Error("attention_gqa_rope: k/v shape does not match q");
    const Storage dq = compute_data(q), dk = compute_data(k), dv = compute_data(v);
    if (dq.dtype != dk.dtype || dq.dtype != dv.dtype) throw Error("attention_gqa_rope: q, k, v must share an element type");
    size_t q_rot = q, k_rot = k;
    if (!prerotated) {
        q_rot = push_tensor(sq, dq.dtype, true);  // kept for backward
        k_rot = push_tensor(sk, dk.dtype, true);
        check(eisen_hip_rope_pair(ctx_, dq.ptr, at(q_rot).data.ptr, sq[2], dk.ptr, at(k_rot).data.ptr, sk[2], dq.dtype, B, S, hd), "rope");
    }
    const size_t out = alloc_pooled_dtype(sq, dq.dtype);
    const size_t lse = alloc_pooled_dtype({B, heads, S}, EISEN_F32);
    check(eisen_hip_attention_forward(ctx_, at(q_rot).data.ptr, at(k_rot).data.ptr, dv.ptr, at(out).data.ptr, (float*)at(lse).data.ptr, dq.dtype, B, S,
                                      heads, kv_heads, hd, nullptr, nullptr, scale, causal ? 1 : 0),
          "attention forward");
    record({q, k, v}, out, [=](Graph& gg) {
        const Storage& go = gg.grad_for_read(out);
        int aq = 0, ak = 0, av = 0;
        Storage& gq = gg.grad_for_write(q, &aq);
        Storage& gk = gg.grad_for_write(k, &ak);
        Storage& gv = gg.grad_for_write(v, &av);
        if (aq || ak || av) throw Error("attention backward: q, k, v must not have other consumers");
        gg.check(eisen_hip_attention_rope_backward(gg.ctx(), gg.at(q_rot).data.ptr, gg.at(k_rot).data.ptr, gg.compute_data(v).ptr, gg.at(out).data.ptr, go.ptr,
                                                   (const float*)gg.at(lse).data.ptr, gq.ptr, gk.ptr, gv.ptr, go.dtype, B, S, heads, kv_heads, hd, scale,
                                                   causal ? 1 : 0),
                 "attention backward");
    });
    return out;
}

size_t Graph::flash_attention(size_t q, size_t k, size_t v, float scale, bool causal) {
    const std::vector<size_t> sq = at(q).shape, sk = at(k).shape, sv = at(v).shape;
    if (sq.size() != 3) throw Error("flash_attention expects q=[B,M,D]");
    if (sk.size() != 3) throw Error("flash_attention expects k=[B,N,D]");
    if (sv.size() != 3) throw Error("flash_attention expects v=[B,N,D]");
    if (sk[0] != sq[0] || sv[0] != sq[0]) throw Error("flash_attention batch mismatch");
    if (sk[2] != sq[2] || sv[2] != sq[2]) throw Error("flash_attention head dim mismatch");
    if (sv[1] != sk[1]) throw Error("flash_attention sequence mismatch k/v");
    if (sq[2] > 256) throw Error("flash_attention kernel currently supports head_dim <= 256");
    if (sk[1] != sq[1]) throw Error("flash_attention: this backend needs M == N (self-attention)");
    const long long st[3] = {(long long)(sq[1] * sq[2]), (long long)sq[2], 0};
    return attention_impl(q, k, v, sq[0], sq[1], 1, 1, sq[2], st, st, scale, causal, sq);
}

}  // namespace eisen
