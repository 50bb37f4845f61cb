/*
 * eisen_cpu_ref.c -- CPU oracle for the eisen training step.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the GPU kernels are
 * compared against; nothing in the shipped library links, loads or calls it.
 *
 * It restates, in plain C, the f32 arithmetic of the reference's `Device::Cpu`
 * arms (single precision, no fused multiply-add, the same per-element order of
 * operations).  Every function cites the reference file:line it follows
 * (paths relative to the reference repository root).
 *
 * Two departures that do NOT change any result bit:
 *   - loops whose iterations write disjoint outputs may run under OpenMP
 *     (`ref_set_threads`, default 1 = the reference's single-threaded shape);
 *   - GEMM-like loops are interchanged so the innermost loop runs over the
 *     contiguous output index while each output element still receives its
 *     addends in the reference's order (k ascending, starting from 0.0f).
 *     `ref_matmul_fwd_literal` keeps the literal nesting; a test checks the two
 *     agree bit for bit.
 *
 * Three places where the reference cannot run at its snapshot and the intended
 * semantics are encoded instead:
 *   - `Graph::backward` on a CPU graph reaches a GPU-only grad allocator
 *     (src/graph/mod.rs:675, src/graph/memory.rs:401-412): treated as a no-op;
 *   - the attention scale tensor is `alloc_pooled` with an empty CPU grad
 *     (src/nn/attention.rs:342, src/graph/mod.rs:550): treated as a constant
 *     whose gradient is discarded;
 *   - `matmul_trans_b` has no CPU arm (src/graph/ops/linear.rs:519-521): the
 *     semantics of its GPU arm (src/graph/ops/linear.rs:456-481) are used:
 *     C = A*B^T, dA += dC*B, dB += dC^T*A.
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off -fno-fast-math).
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define REF_MAX_RANK 4
#define REF_IGNORE_INDEX ((int64_t)-1) /* usize::MAX, src/data/fim.rs:173 */

static int g_threads = 1;

void ref_set_threads(int n) {
    g_threads = n < 1 ? 1 : n;
#ifdef _OPENMP
    omp_set_num_threads(g_threads);
#endif
}
int ref_get_threads(void) { return g_threads; }

/* ------------------------------------------------------------------------- */
/* scalar helpers                                                            */
/* ------------------------------------------------------------------------- */

/* f32::powi lowers to compiler-rt's __powisf2: square-and-multiply. */
static float powi_f32(float a, int b) {
    const int recip = b < 0;
    float r = 1.0f;
    while (1) {
        if (b & 1) r *= a;
        b /= 2;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0f / r : r;
}
float ref_powi(float a, int b) { return powi_f32(a, b); }

/* ------------------------------------------------------------------------- */
/* stateless op kernels (raw arrays)                                         */
/* ------------------------------------------------------------------------- */

/* src/graph/ops/linear.rs:254-262, literal nesting. */
void ref_matmul_fwd_literal(const float* a, const float* b, float* out, size_t m, size_t k, size_t n) {
    for (size_t r = 0; r < m; r++)
        for (size_t c = 0; c < n; c++) {
            float sum = 0.0f;
            for (size_t i = 0; i < k; i++) sum += a[r * k + i] * b[i * n + c];
            out[r * n + c] = sum;
        }
}

/* src/graph/ops/linear.rs:254-262, interchanged (same per-element order). */
void ref_matmul_fwd(const float* a, const float* b, float* out, size_t m, size_t k, size_t n) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t r = 0; r < m; r++) {
        float* o = out + r * n;
        for (size_t c = 0; c < n; c++) o[c] = 0.0f;
        for (size_t i = 0; i < k; i++) {
            const float av = a[r * k + i];
            const float* br = b + i * n;
            for (size_t c = 0; c < n; c++) o[c] += av * br[c];
        }
    }
}

/* src/graph/ops/linear.rs:266-287.  dA[r,i] += sum_c go[r,c]*b[i,c] (c ascending);
 * dB[i,c] += sum_r a[r,i]*go[r,c] (r ascending, local sum from 0 then one add). */
void ref_matmul_bwd(const float* a, const float* b, const float* go, float* ga, float* gb,
                    size_t m, size_t k, size_t n) {
    if (ga) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
        for (size_t r = 0; r < m; r++)
            for (size_t i = 0; i < k; i++) {
                float sum = 0.0f;
                const float* g = go + r * n;
                const float* br = b + i * n;
                for (size_t c = 0; c < n; c++) sum += g[c] * br[c];
                ga[r * k + i] += sum;
            }
    }
    if (gb) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
        for (size_t i = 0; i < k; i++) {
            float* tmp = (float*)calloc(n, sizeof(float));
            for (size_t r = 0; r < m; r++) {
                const float av = a[r * k + i];
                const float* g = go + r * n;
                for (size_t c = 0; c < n; c++) tmp[c] += av * g[c];
            }
            for (size_t c = 0; c < n; c++) gb[i * n + c] += tmp[c];
            free(tmp);
        }
    }
}

/* Intended semantics of matmul_trans_b (GPU arm src/graph/ops/linear.rs:301-517,
 * kernels/ops_f32.cu:842-882): C[m,n] = sum_i A[m,i]*B[n,i]; dA += dC*B;
 * dB[n,i] += sum_m dC[m,n]*A[m,i].  Summation ascending in the contracted index. */
void ref_matmul_trans_b_fwd(const float* a, const float* b, float* out, size_t m, size_t k, size_t n) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t r = 0; r < m; r++)
        for (size_t c = 0; c < n; c++) {
            float sum = 0.0f;
            for (size_t i = 0; i < k; i++) sum += a[r * k + i] * b[c * k + i];
            out[r * n + c] = sum;
        }
}
void ref_matmul_trans_b_bwd(const float* a, const float* b, const float* go, float* ga, float* gb,
                            size_t m, size_t k, size_t n) {
    if (ga) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
        for (size_t r = 0; r < m; r++) {
            float* tmp = (float*)calloc(k, sizeof(float));
            for (size_t c = 0; c < n; c++) {
                const float g = go[r * n + c];
                for (size_t i = 0; i < k; i++) tmp[i] += g * b[c * k + i];
            }
            for (size_t i = 0; i < k; i++) ga[r * k + i] += tmp[i];
            free(tmp);
        }
    }
    if (gb) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
        for (size_t c = 0; c < n; c++) {
            float* tmp = (float*)calloc(k, sizeof(float));
            for (size_t r = 0; r < m; r++) {
                const float g = go[r * n + c];
                for (size_t i = 0; i < k; i++) tmp[i] += g * a[r * k + i];
            }
            for (size_t i = 0; i < k; i++) gb[c * k + i] += tmp[i];
            free(tmp);
        }
    }
}

/* src/graph/ops/linear.rs:1430-1446. */
void ref_bmm_fwd(const float* a, const float* b, float* out, size_t batch, size_t m, size_t k, size_t n,
                 int trans_b) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t bb = 0; bb < batch; bb++) {
        if (trans_b) {
            for (size_t i = 0; i < m; i++)
                for (size_t j = 0; j < n; j++) {
                    float acc = 0.0f;
                    const float* ar = a + (bb * m + i) * k;
                    const float* br = b + (bb * n + j) * k;
                    for (size_t kk = 0; kk < k; kk++) acc += ar[kk] * br[kk];
                    out[(bb * m + i) * n + j] = acc;
                }
        } else {
            for (size_t i = 0; i < m; i++) {
                float* o = out + (bb * m + i) * n;
                for (size_t j = 0; j < n; j++) o[j] = 0.0f;
                for (size_t kk = 0; kk < k; kk++) {
                    const float av = a[(bb * m + i) * k + kk];
                    const float* br = b + (bb * k + kk) * n;
                    for (size_t j = 0; j < n; j++) o[j] += av * br[j];
                }
            }
        }
    }
}

/* src/graph/ops/linear.rs:1452-1498.  No local sums: every product lands on the
 * gradient buffer directly, in (i, j, kk) order.  a_grad[i,kk] therefore receives
 * its addends in ascending j, b_grad in ascending i; the two streams touch
 * different buffers (a_id != b_id), so they are separated here and each keeps its
 * order.  The aliasing case a_id == b_id keeps the literal interleaving. */
void ref_bmm_bwd(const float* a, const float* b, const float* go, float* ga, float* gb, size_t batch,
                 size_t m, size_t k, size_t n, int trans_b) {
    if (ga == gb) {
        for (size_t bb = 0; bb < batch; bb++)
            for (size_t i = 0; i < m; i++)
                for (size_t j = 0; j < n; j++) {
                    const float g = go[(bb * m + i) * n + j];
                    for (size_t kk = 0; kk < k; kk++) {
                        size_t ai = (bb * m + i) * k + kk;
                        size_t bi = trans_b ? (bb * n + j) * k + kk : (bb * k + kk) * n + j;
                        ga[ai] += g * b[bi];
                        ga[bi] += g * a[ai];
                    }
                }
        return;
    }
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t bb = 0; bb < batch; bb++) {
        for (size_t i = 0; i < m; i++)
            for (size_t j = 0; j < n; j++) {
                const float g = go[(bb * m + i) * n + j];
                float* gar = ga + (bb * m + i) * k;
                if (trans_b) {
                    const float* br = b + (bb * n + j) * k;
                    for (size_t kk = 0; kk < k; kk++) gar[kk] += g * br[kk];
                } else {
                    for (size_t kk = 0; kk < k; kk++) gar[kk] += g * b[(bb * k + kk) * n + j];
                }
            }
        for (size_t i = 0; i < m; i++)
            for (size_t j = 0; j < n; j++) {
                const float g = go[(bb * m + i) * n + j];
                const float* ar = a + (bb * m + i) * k;
                if (trans_b) {
                    float* gbr = gb + (bb * n + j) * k;
                    for (size_t kk = 0; kk < k; kk++) gbr[kk] += g * ar[kk];
                } else {
                    for (size_t kk = 0; kk < k; kk++) gb[(bb * k + kk) * n + j] += g * ar[kk];
                }
            }
    }
}

/* src/graph/ops/elementwise.rs:442-455. */
void ref_silu_fwd(const float* x, float* out, size_t n) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t i = 0; i < n; i++) out[i] = x[i] * (1.0f / (1.0f + expf(-x[i])));
}
void ref_silu_bwd(const float* x, const float* go, float* gx, size_t n) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t i = 0; i < n; i++) {
        const float sig = 1.0f / (1.0f + expf(-x[i]));
        const float silu = x[i] * sig;
        gx[i] += go[i] * (silu + sig * (1.0f - silu));
    }
}

/* src/graph/ops/reduction.rs:483-496 (fwd), :504-512 (bwd). */
void ref_softmax_fwd(const float* x, float* out, size_t rows, size_t n) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t row = 0; row < rows; row++) {
        const float* xr = x + row * n;
        float* o = out + row * n;
        float mx = -INFINITY;
        for (size_t j = 0; j < n; j++) mx = fmaxf(mx, xr[j]);
        float sum = 0.0f;
        for (size_t j = 0; j < n; j++) {
            const float e = expf(xr[j] - mx);
            o[j] = e;
            sum += e;
        }
        for (size_t j = 0; j < n; j++) o[j] /= sum;
    }
}
void ref_softmax_bwd(const float* out, const float* go, float* gx, size_t rows, size_t n) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t row = 0; row < rows; row++) {
        const size_t off = row * n;
        float dot = 0.0f;
        for (size_t j = 0; j < n; j++) dot += go[off + j] * out[off + j];
        for (size_t j = 0; j < n; j++) gx[off + j] += out[off + j] * (go[off + j] - dot);
    }
}

/* src/graph/ops/reduction.rs:676-693.  probs must hold rows*classes floats.
 * Returns the mean loss; the per-row sum is sequential over rows as in the
 * reference, so the probability pass (parallel) and the loss pass are split. */
float ref_cross_entropy_fwd(const float* logits, const int64_t* targets, float* probs, size_t rows,
                            size_t classes) {
    ref_softmax_fwd(logits, probs, rows, classes);
    float out_loss = 0.0f;
    for (size_t b = 0; b < rows; b++) out_loss += -logf(probs[b * classes + (size_t)targets[b]] + 1e-8f);
    return out_loss / (float)rows;
}
/* src/graph/ops/reduction.rs:695-707. */
void ref_cross_entropy_bwd(const float* probs, const int64_t* targets, float o_grad, float* gl, size_t rows,
                           size_t classes) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t b = 0; b < rows; b++)
        for (size_t c = 0; c < classes; c++) {
            const size_t idx = b * classes + c;
            float g = probs[idx];
            if ((int64_t)c == targets[b]) g -= 1.0f;
            gl[idx] += (g / (float)rows) * o_grad;
        }
}

/* src/graph/ops/reduction.rs:724-760 (normalizer) and :888-916 (CPU arm).
 * normalizer = 1/valid_count (f32); rows whose target is IGNORE are skipped. */
float ref_cross_entropy_masked_fwd(const float* logits, const int64_t* targets, float* probs, size_t rows,
                                   size_t classes, float normalizer) {
    memset(probs, 0, rows * classes * sizeof(float));
    float out_loss = 0.0f;
    for (size_t b = 0; b < rows; b++) {
        if (targets[b] == REF_IGNORE_INDEX) continue;
        ref_softmax_fwd(logits + b * classes, probs + b * classes, 1, classes);
        const float p = probs[b * classes + (size_t)targets[b]];
        out_loss += -logf(p + 1e-8f) * normalizer;
    }
    return out_loss;
}
/* src/graph/ops/reduction.rs:921-932. */
void ref_cross_entropy_masked_bwd(const float* probs, const int64_t* targets, float o_grad, float* gl,
                                  size_t rows, size_t classes, float normalizer) {
    for (size_t b = 0; b < rows; b++) {
        if (targets[b] == REF_IGNORE_INDEX) continue;
        for (size_t c = 0; c < classes; c++) {
            const size_t idx = b * classes + c;
            float g = probs[idx];
            if ((int64_t)c == targets[b]) g -= 1.0f;
            gl[idx] += g * normalizer * o_grad;
        }
    }
}

/* src/graph/ops/transform.rs:87-97 (fwd) and :103-114 (bwd): [B,S,H,D] -> [B,H,S,D]. */
void ref_transpose_0213_fwd(const float* a, float* out, size_t b, size_t s, size_t h, size_t d) {
    for (size_t bb = 0; bb < b; bb++)
        for (size_t ss = 0; ss < s; ss++)
            for (size_t hh = 0; hh < h; hh++)
                for (size_t dd = 0; dd < d; dd++)
                    out[((bb * h + hh) * s + ss) * d + dd] = a[((bb * s + ss) * h + hh) * d + dd];
}
void ref_transpose_0213_bwd(const float* go, float* ga, size_t b, size_t s, size_t h, size_t d) {
    for (size_t bb = 0; bb < b; bb++)
        for (size_t ss = 0; ss < s; ss++)
            for (size_t hh = 0; hh < h; hh++)
                for (size_t dd = 0; dd < d; dd++)
                    ga[((bb * s + ss) * h + hh) * d + dd] += go[((bb * h + hh) * s + ss) * d + dd];
}

/* src/graph/ops/transform.rs:287-303 (fwd), :306-315 (bwd).  Indices are stored as
 * f32 and converted with `as usize` (truncation toward zero, saturating). */
void ref_gather_fwd(const float* w, const float* idx, float* out, size_t num_indices, size_t hidden) {
    for (size_t i = 0; i < num_indices; i++) {
        const size_t row = (size_t)idx[i];
        memcpy(out + i * hidden, w + row * hidden, hidden * sizeof(float));
    }
}
void ref_gather_bwd(const float* idx, const float* go, float* gw, size_t num_indices, size_t hidden) {
    for (size_t i = 0; i < num_indices; i++) {
        const size_t row = (size_t)idx[i];
        for (size_t d = 0; d < hidden; d++) gw[row * hidden + d] += go[i * hidden + d];
    }
}

/* src/graph/ops/transform.rs:546-571 (fwd), :575-599 (bwd).  x is [batch, seq, hidden]. */
void ref_rope_fwd(const float* a, float* out, size_t batch, size_t seq_len, size_t hidden, size_t head_dim) {
    memcpy(out, a, batch * seq_len * hidden * sizeof(float));
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t bb = 0; bb < batch; bb++)
        for (size_t pos = 0; pos < seq_len; pos++)
            for (size_t base = 0; base < hidden; base += head_dim)
                for (size_t pair = 0; pair < head_dim / 2; pair++) {
                    const size_t even = base + 2 * pair, odd = even + 1;
                    if (odd >= base + head_dim || odd >= hidden) continue;
                    const size_t i0 = (bb * seq_len + pos) * hidden + even, i1 = i0 + 1;
                    const float theta = (float)pos / powf(10000.0f, (2.0f * (float)pair) / (float)head_dim);
                    const float s = sinf(theta), c = cosf(theta);
                    const float x0 = a[i0], x1 = a[i1];
                    out[i0] = x0 * c - x1 * s;
                    out[i1] = x0 * s + x1 * c;
                }
}
void ref_rope_bwd(const float* go, float* ga, size_t batch, size_t seq_len, size_t hidden, size_t head_dim) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t bb = 0; bb < batch; bb++)
        for (size_t pos = 0; pos < seq_len; pos++)
            for (size_t base = 0; base < hidden; base += head_dim)
                for (size_t pair = 0; pair < head_dim / 2; pair++) {
                    const size_t even = base + 2 * pair, odd = even + 1;
                    if (odd >= base + head_dim || odd >= hidden) continue;
                    const size_t i0 = (bb * seq_len + pos) * hidden + even, i1 = i0 + 1;
                    const float theta = (float)pos / powf(10000.0f, (2.0f * (float)pair) / (float)head_dim);
                    const float s = sinf(theta), c = cosf(theta);
                    const float g0 = go[i0], g1 = go[i1];
                    ga[i0] += g0 * c + g1 * s;
                    ga[i1] += -g0 * s + g1 * c;
                }
}

/* src/graph/ops/normalization.rs:141-151.  rrms_cache holds num_vecs floats. */
void ref_rms_norm_fwd(const float* x, const float* w, float* out, float* rrms_cache, size_t num_vecs,
                      size_t dim, float eps) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t n = 0; n < num_vecs; n++) {
        const size_t off = n * dim;
        float ss = 0.0f;
        for (size_t d = 0; d < dim; d++) ss += x[off + d] * x[off + d];
        const float rrms = 1.0f / sqrtf(ss / (float)dim + eps);
        rrms_cache[n] = rrms;
        for (size_t d = 0; d < dim; d++) out[off + d] = x[off + d] * rrms * w[d];
    }
}
/* src/graph/ops/normalization.rs:157-171.  gw[d] receives rows in ascending order. */
void ref_rms_norm_bwd(const float* x, const float* w, const float* rrms_cache, const float* go, float* gx,
                      float* gw, size_t num_vecs, size_t dim) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t n = 0; n < num_vecs; n++) {
        const size_t off = n * dim;
        const float rrms = rrms_cache[n];
        float gdxw = 0.0f;
        for (size_t d = 0; d < dim; d++) gdxw += go[off + d] * x[off + d] * w[d];
        const float rrc_d = powi_f32(rrms, 3) / (float)dim;
        for (size_t d = 0; d < dim; d++)
            gx[off + d] += rrms * (go[off + d] * w[d]) - x[off + d] * rrc_d * gdxw;
    }
    for (size_t n = 0; n < num_vecs; n++) {
        const size_t off = n * dim;
        const float rrms = rrms_cache[n];
        for (size_t d = 0; d < dim; d++) gw[d] += go[off + d] * x[off + d] * rrms;
    }
}

/* src/graph/ops/gqa.rs:147-160 (fwd), :168-184 (bwd).  [B,KV,S,D] -> [B,KV*rep,S,D]. */
void ref_repeat_kv_fwd(const float* in, float* out, size_t batch, size_t kvh, size_t seq, size_t hd,
                       size_t repeats) {
    const size_t qh = kvh * repeats;
    for (size_t b = 0; b < batch; b++)
        for (size_t q = 0; q < qh; q++) {
            const size_t kv = q / repeats;
            memcpy(out + ((b * qh + q) * seq) * hd, in + ((b * kvh + kv) * seq) * hd, seq * hd * sizeof(float));
        }
}
void ref_repeat_kv_bwd(const float* go, float* gin, size_t batch, size_t kvh, size_t seq, size_t hd,
                       size_t repeats) {
    const size_t qh = kvh * repeats;
    for (size_t b = 0; b < batch; b++)
        for (size_t kv = 0; kv < kvh; kv++)
            for (size_t r = 0; r < repeats; r++) {
                const size_t q = kv * repeats + r;
                const float* g = go + ((b * qh + q) * seq) * hd;
                float* gi = gin + ((b * kvh + kv) * seq) * hd;
                for (size_t e = 0; e < seq * hd; e++) gi[e] += g[e];
            }
}

/* src/graph/ops/attention.rs:145-191: inference-only forward, q [B,M,D], k/v [B,N,D]. */
void ref_flash_attention_fwd(const float* q, const float* k, const float* v, float* out, size_t batch,
                             size_t m, size_t n, size_t d, float scale, int causal) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t bb = 0; bb < batch; bb++) {
        float* scores = (float*)malloc(n * sizeof(float));
        float* probs = (float*)malloc(n * sizeof(float));
        for (size_t i = 0; i < m; i++) {
            for (size_t j = 0; j < n; j++) {
                if (causal && j > i) {
                    scores[j] = -INFINITY;
                    continue;
                }
                float dot = 0.0f;
                for (size_t dd = 0; dd < d; dd++) dot += q[(bb * m + i) * d + dd] * k[(bb * n + j) * d + dd];
                scores[j] = dot * scale;
            }
            float mx = -INFINITY;
            for (size_t j = 0; j < n; j++) mx = fmaxf(mx, scores[j]);
            float denom = 0.0f;
            for (size_t j = 0; j < n; j++) {
                const float e = expf(scores[j] - mx);
                probs[j] = e;
                denom += e;
            }
            for (size_t j = 0; j < n; j++) probs[j] /= denom;
            for (size_t dd = 0; dd < d; dd++) {
                float acc = 0.0f;
                for (size_t j = 0; j < n; j++) acc += probs[j] * v[(bb * n + j) * d + dd];
                out[(bb * m + i) * d + dd] = acc;
            }
        }
        free(scores);
        free(probs);
    }
}

/* src/nn/optim.rs:336-338 (bias corrections), :533-542 (element update). */
void ref_adamw_bias_corrections(float beta1, float beta2, int t, float* bc1, float* bc2) {
    *bc1 = 1.0f / (1.0f - powi_f32(beta1, t));
    *bc2 = 1.0f / (1.0f - powi_f32(beta2, t));
}
void ref_adamw_update(float* w, const float* g, float* m, float* v, size_t n, float lr, float beta1,
                      float beta2, float eps, float wd, float bc1, float bc2) {
#pragma omp parallel for schedule(static) if (g_threads > 1)
    for (size_t i = 0; i < n; i++) {
        const float grad = g[i];
        const float decayed = w[i] * (1.0f - lr * wd);
        m[i] = beta1 * m[i] + (1.0f - beta1) * grad;
        v[i] = beta2 * v[i] + (1.0f - beta2) * grad * grad;
        const float m_hat = m[i] * bc1;
        const float v_hat = v[i] * bc2;
        w[i] = decayed - lr * m_hat / (sqrtf(v_hat) + eps);
    }
}

/* src/nn/optim.rs:250-321: f64 sum of squares over every grad, in params order. */
double ref_sum_squares_f64(const float* g, size_t n, double acc) {
    for (size_t i = 0; i < n; i++) {
        const double x = (double)g[i];
        acc += x * x;
    }
    return acc;
}
float ref_clip_coef(double sum_sq, float max_norm, float* grad_norm_out) {
    const float grad_norm = (float)sqrt(sum_sq);
    if (grad_norm_out) *grad_norm_out = grad_norm;
    float coef = 1.0f;
    if (grad_norm > 0.0f) {
        coef = max_norm / (grad_norm + 1e-6f);
        if (coef > 1.0f) coef = 1.0f;
    }
    return coef;
}

/* src/nn/scheduler.rs:45-55. */
float ref_cosine_lr(float lr_max, float lr_min, size_t warmup_steps, size_t total_steps, size_t step) {
    if (step < warmup_steps) return lr_max * (float)(step + 1) / (float)warmup_steps;
    size_t decay_steps = total_steps - warmup_steps;
    if (decay_steps < 1) decay_steps = 1;
    float progress = (float)(step - warmup_steps) / (float)decay_steps;
    if (progress < 0.0f) progress = 0.0f;
    if (progress > 1.0f) progress = 1.0f;
    return lr_min + 0.5f * (lr_max - lr_min) * (1.0f + cosf(3.14159274101257324f * progress));
}

/* ------------------------------------------------------------------------- */
/* Graph / tape (src/graph/mod.rs, src/tape.rs, src/tensor.rs)               */
/* ------------------------------------------------------------------------- */

typedef struct {
    size_t shape[REF_MAX_RANK];
    int rank;
    size_t numel;
    float* data;
    float* grad;
    int owns_data; /* 0 for reshape-free views (none today) */
} ref_tensor;

enum {
    OP_ADD, OP_MUL, OP_SILU, OP_MATMUL, OP_MATMUL_TB, OP_BMM, OP_SOFTMAX, OP_CE, OP_CE_MASKED,
    OP_T0213, OP_GATHER, OP_RESHAPE, OP_ROPE, OP_RMSNORM, OP_REPEAT_KV, OP_SUM, OP_MAX, OP_TRANSPOSE
};

typedef struct {
    int op;
    int in0, in1, out;
    size_t p[6];    /* op-specific integer parameters */
    float f[2];     /* op-specific float parameters */
    float* aux;     /* saved forward values (probs, rrms cache, softmax out) */
    int64_t* iaux;  /* saved integer values (targets, argmax) */
    int discard_in1_grad; /* constant operand whose gradient is dropped */
} ref_node;

typedef struct ref_graph {
    ref_tensor* t;
    int nt, cap_t;
    ref_node* nodes;
    int nn, cap_n;
    int num_params;
    int no_grad;
} ref_graph;

ref_graph* ref_graph_new(void) { return (ref_graph*)calloc(1, sizeof(ref_graph)); }

static void tensor_free(ref_tensor* t) {
    if (t->owns_data) free(t->data);
    free(t->grad);
}
static void node_free(ref_node* n) {
    free(n->aux);
    free(n->iaux);
}
void ref_graph_free(ref_graph* g) {
    for (int i = 0; i < g->nt; i++) tensor_free(&g->t[i]);
    for (int i = 0; i < g->nn; i++) node_free(&g->nodes[i]);
    free(g->t);
    free(g->nodes);
    free(g);
}

static size_t shape_numel(const size_t* shape, int rank) {
    size_t n = 1;
    for (int i = 0; i < rank; i++) n *= shape[i];
    return n;
}

/* Graph::alloc (src/graph/mod.rs:558-564, Tensor::new src/tensor.rs:145-175):
 * data copied in, grad zero-filled.  data == NULL gives zero data. */
int ref_alloc(ref_graph* g, const size_t* shape, int rank, const float* data) {
    if (g->nt == g->cap_t) {
        g->cap_t = g->cap_t ? g->cap_t * 2 : 64;
        g->t = (ref_tensor*)realloc(g->t, (size_t)g->cap_t * sizeof(ref_tensor));
    }
    ref_tensor* t = &g->t[g->nt];
    memset(t, 0, sizeof(*t));
    t->rank = rank;
    for (int i = 0; i < rank; i++) t->shape[i] = shape[i];
    t->numel = shape_numel(shape, rank);
    t->data = (float*)calloc(t->numel ? t->numel : 1, sizeof(float));
    t->grad = (float*)calloc(t->numel ? t->numel : 1, sizeof(float));
    t->owns_data = 1;
    if (data) memcpy(t->data, data, t->numel * sizeof(float));
    return g->nt++;
}

static ref_node* push_node(ref_graph* g, int op, int in0, int in1, int out) {
    if (g->nn == g->cap_n) {
        g->cap_n = g->cap_n ? g->cap_n * 2 : 64;
        g->nodes = (ref_node*)realloc(g->nodes, (size_t)g->cap_n * sizeof(ref_node));
    }
    ref_node* n = &g->nodes[g->nn++];
    memset(n, 0, sizeof(*n));
    n->op = op;
    n->in0 = in0;
    n->in1 = in1;
    n->out = out;
    return n;
}
/* When no_grad is set the reference skips the tape push (e.g. src/graph/ops/linear.rs:288);
 * the saved buffers are then dropped immediately. */
static void finish_node(ref_graph* g) {
    if (g->no_grad) {
        node_free(&g->nodes[g->nn - 1]);
        g->nn--;
    }
}

float* ref_data(ref_graph* g, int id) { return g->t[id].data; }
float* ref_grad(ref_graph* g, int id) { return g->t[id].grad; }
size_t ref_numel(ref_graph* g, int id) { return g->t[id].numel; }
int ref_rank(ref_graph* g, int id) { return g->t[id].rank; }
size_t ref_dim(ref_graph* g, int id, int i) { return g->t[id].shape[i]; }
int ref_num_tensors(ref_graph* g) { return g->nt; }
int ref_tape_len(ref_graph* g) { return g->nn; }
void ref_set_no_grad(ref_graph* g, int v) { g->no_grad = v; }
void ref_mark_params(ref_graph* g) { g->num_params = g->nt; } /* src/graph/mod.rs:328-330 */

/* Graph::load_tensor_data, CPU arm (src/graph/mod.rs:368-392). */
void ref_load_tensor_data(ref_graph* g, int id, const float* host, size_t n) {
    if (n != g->t[id].numel) {
        fprintf(stderr, "ref_load_tensor_data: tensor %d expects %zu elements, got %zu\n", id, g->t[id].numel, n);
        abort();
    }
    memcpy(g->t[id].data, host, n * sizeof(float));
}

/* Graph::reinterpret_shape (src/graph/ops/transform.rs:413-426). */
void ref_reinterpret_shape(ref_graph* g, int id, const size_t* shape, int rank) {
    if (shape_numel(shape, rank) != g->t[id].numel) {
        fprintf(stderr, "reinterpret_shape: element count mismatch\n");
        abort();
    }
    g->t[id].rank = rank;
    for (int i = 0; i < rank; i++) g->t[id].shape[i] = shape[i];
}

/* Graph::clear_activations (src/graph/mod.rs:432-435) + restore_save_point (:336-365). */
void ref_restore_save_point(ref_graph* g, int save_point) {
    while (g->nt > save_point) tensor_free(&g->t[--g->nt]);
}
void ref_clear_activations(ref_graph* g) {
    for (int i = 0; i < g->nn; i++) node_free(&g->nodes[i]);
    g->nn = 0;
    ref_restore_save_point(g, g->num_params);
}
void ref_zero_grad(ref_graph* g, int id) { memset(g->t[id].grad, 0, g->t[id].numel * sizeof(float)); }

/* --- broadcasting helpers (src/tensor.rs:236-272) --- */
static void bcast_shape(const ref_tensor* a, const ref_tensor* b, size_t* out, int* rank) {
    const int ml = a->rank > b->rank ? a->rank : b->rank;
    for (int i = 0; i < ml; i++) {
        const size_t da = i < ml - a->rank ? 1 : a->shape[i - (ml - a->rank)];
        const size_t db = i < ml - b->rank ? 1 : b->shape[i - (ml - b->rank)];
        out[i] = da > db ? da : db;
    }
    *rank = ml;
}
static void bcast_strides(const ref_tensor* t, const size_t* oshape, int orank, size_t* strides) {
    size_t base[REF_MAX_RANK];
    size_t cur = 1;
    for (int i = t->rank - 1; i >= 0; i--) {
        base[i] = cur;
        cur *= t->shape[i];
    }
    const int pad = orank - t->rank;
    for (int i = 0; i < orank; i++) strides[i] = 0;
    for (int i = 0; i < t->rank; i++)
        if (t->shape[i] == oshape[pad + i]) strides[pad + i] = base[i];
}
static size_t bcast_index(size_t flat, const size_t* oshape, int orank, const size_t* strides) {
    size_t idx = 0;
    for (int i = orank - 1; i >= 0; i--) {
        idx += (flat % oshape[i]) * strides[i];
        flat /= oshape[i];
    }
    return idx;
}

/* Graph::add CPU arm (src/graph/ops/elementwise.rs:146-183). */
int ref_add(ref_graph* g, int a, int b) {
    size_t os[REF_MAX_RANK];
    int orank;
    bcast_shape(&g->t[a], &g->t[b], os, &orank);
    const int out = ref_alloc(g, os, orank, NULL);
    size_t sa[REF_MAX_RANK], sb[REF_MAX_RANK];
    bcast_strides(&g->t[a], os, orank, sa);
    bcast_strides(&g->t[b], os, orank, sb);
    const ref_tensor* ta = &g->t[a];
    const ref_tensor* tb = &g->t[b];
    float* o = g->t[out].data;
    const size_t n = g->t[out].numel;
    if (ta->numel == n && tb->numel == n) {
        for (size_t i = 0; i < n; i++) o[i] = ta->data[i] + tb->data[i];
    } else {
#pragma omp parallel for schedule(static) if (g_threads > 1)
        for (size_t i = 0; i < n; i++)
            o[i] = ta->data[bcast_index(i, os, orank, sa)] + tb->data[bcast_index(i, os, orank, sb)];
    }
    push_node(g, OP_ADD, a, b, out);
    finish_node(g);
    return out;
}

/* Graph::mul CPU arm (src/graph/ops/elementwise.rs:294-331).  discard_b_grad marks the
 * operand as a constant (the attention scale tensor). */
int ref_mul_ex(ref_graph* g, int a, int b, int discard_b_grad) {
    size_t os[REF_MAX_RANK];
    int orank;
    bcast_shape(&g->t[a], &g->t[b], os, &orank);
    const int out = ref_alloc(g, os, orank, NULL);
    size_t sa[REF_MAX_RANK], sb[REF_MAX_RANK];
    bcast_strides(&g->t[a], os, orank, sa);
    bcast_strides(&g->t[b], os, orank, sb);
    const ref_tensor* ta = &g->t[a];
    const ref_tensor* tb = &g->t[b];
    float* o = g->t[out].data;
    const size_t n = g->t[out].numel;
    if (ta->numel == n && tb->numel == n) {
        for (size_t i = 0; i < n; i++) o[i] = ta->data[i] * tb->data[i];
    } else {
        for (size_t i = 0; i < n; i++)
            o[i] = ta->data[bcast_index(i, os, orank, sa)] * tb->data[bcast_index(i, os, orank, sb)];
    }
    ref_node* nd = push_node(g, OP_MUL, a, b, out);
    nd->discard_in1_grad = discard_b_grad;
    finish_node(g);
    return out;
}
int ref_mul(ref_graph* g, int a, int b) { return ref_mul_ex(g, a, b, 0); }

/* Graph::silu CPU arm (src/graph/ops/elementwise.rs:439-465). */
int ref_silu(ref_graph* g, int a) {
    const int out = ref_alloc(g, g->t[a].shape, g->t[a].rank, NULL);
    ref_silu_fwd(g->t[a].data, g->t[out].data, g->t[a].numel);
    push_node(g, OP_SILU, a, -1, out);
    finish_node(g);
    return out;
}

/* Graph::matmul CPU arm (src/graph/ops/linear.rs:250-297).  A is flattened to [M,K]
 * over its leading dims (:20-33); the output is [M,N]. */
int ref_matmul(ref_graph* g, int a, int b) {
    const ref_tensor* ta = &g->t[a];
    const size_t k = ta->shape[ta->rank - 1];
    const size_t m = ta->numel / k;
    const size_t n = g->t[b].shape[1];
    if (g->t[b].shape[0] != k) {
        fprintf(stderr, "ref_matmul: inner dims differ (%zu vs %zu)\n", k, g->t[b].shape[0]);
        abort();
    }
    size_t os[2] = {m, n};
    const int out = ref_alloc(g, os, 2, NULL);
    ref_matmul_fwd(g->t[a].data, g->t[b].data, g->t[out].data, m, k, n);
    ref_node* nd = push_node(g, OP_MATMUL, a, b, out);
    nd->p[0] = m; nd->p[1] = k; nd->p[2] = n;
    finish_node(g);
    return out;
}

/* Graph::matmul_trans_b: a [M,K] (leading dims flattened), b [N,K] -> [M,N]. */
int ref_matmul_trans_b(ref_graph* g, int a, int b) {
    const ref_tensor* ta = &g->t[a];
    const size_t k = ta->shape[ta->rank - 1];
    const size_t m = ta->numel / k;
    const size_t n = g->t[b].shape[0];
    size_t os[REF_MAX_RANK];
    int orank = ta->rank;
    for (int i = 0; i < orank - 1; i++) os[i] = ta->shape[i];
    os[orank - 1] = n;
    const int out = ref_alloc(g, os, orank, NULL);
    ref_matmul_trans_b_fwd(g->t[a].data, g->t[b].data, g->t[out].data, m, k, n);
    ref_node* nd = push_node(g, OP_MATMUL_TB, a, b, out);
    nd->p[0] = m; nd->p[1] = k; nd->p[2] = n;
    finish_node(g);
    return out;
}

/* Graph::bmm CPU arm (src/graph/ops/linear.rs:1425-1511).  a [B,M,K]; b [B,N,K] if
 * trans_b else [B,K,N]. */
int ref_bmm(ref_graph* g, int a, int b, int trans_b) {
    const ref_tensor* ta = &g->t[a];
    const ref_tensor* tb = &g->t[b];
    const size_t batch = ta->shape[0], m = ta->shape[1], k = ta->shape[2];
    const size_t n = trans_b ? tb->shape[1] : tb->shape[2];
    size_t os[3] = {batch, m, n};
    const int out = ref_alloc(g, os, 3, NULL);
    ref_bmm_fwd(ta->data, tb->data, g->t[out].data, batch, m, k, n, trans_b);
    ref_node* nd = push_node(g, OP_BMM, a, b, out);
    nd->p[0] = batch; nd->p[1] = m; nd->p[2] = k; nd->p[3] = n; nd->p[4] = (size_t)trans_b;
    finish_node(g);
    return out;
}

/* Graph::softmax CPU arm (src/graph/ops/reduction.rs:476-523): over the last dim. */
int ref_softmax(ref_graph* g, int a) {
    const ref_tensor* ta = &g->t[a];
    const size_t n = ta->shape[ta->rank - 1];
    const size_t rows = ta->numel / n;
    const int out = ref_alloc(g, ta->shape, ta->rank, NULL);
    ref_softmax_fwd(g->t[a].data, g->t[out].data, rows, n);
    ref_node* nd = push_node(g, OP_SOFTMAX, a, -1, out);
    nd->p[0] = rows; nd->p[1] = n;
    finish_node(g);
    return out;
}

/* Graph::cross_entropy CPU arm (src/graph/ops/reduction.rs:668-716). */
int ref_cross_entropy(ref_graph* g, int logits, const int64_t* targets) {
    const size_t rows = g->t[logits].shape[0], classes = g->t[logits].shape[1];
    float* probs = (float*)malloc(rows * classes * sizeof(float));
    const float loss = ref_cross_entropy_fwd(g->t[logits].data, targets, probs, rows, classes);
    const int out = ref_alloc(g, NULL, 0, &loss);
    ref_node* nd = push_node(g, OP_CE, logits, -1, out);
    nd->p[0] = rows; nd->p[1] = classes;
    nd->aux = probs;
    nd->iaux = (int64_t*)malloc(rows * sizeof(int64_t));
    memcpy(nd->iaux, targets, rows * sizeof(int64_t));
    finish_node(g);
    return out;
}

/* Graph::cross_entropy_masked (src/graph/ops/reduction.rs:724-944): falls back to the
 * plain loss when no target is IGNORE (:733-735); valid_count 0 gives a zero loss
 * with no tape node (:737-741). */
int ref_cross_entropy_masked(ref_graph* g, int logits, const int64_t* targets) {
    const size_t rows = g->t[logits].shape[0], classes = g->t[logits].shape[1];
    size_t valid = 0;
    for (size_t b = 0; b < rows; b++) valid += targets[b] != REF_IGNORE_INDEX;
    if (valid == rows) return ref_cross_entropy(g, logits, targets);
    if (valid == 0) {
        const float z = 0.0f;
        return ref_alloc(g, NULL, 0, &z);
    }
    const float normalizer = 1.0f / (float)valid;
    float* probs = (float*)malloc(rows * classes * sizeof(float));
    const float loss = ref_cross_entropy_masked_fwd(g->t[logits].data, targets, probs, rows, classes, normalizer);
    const int out = ref_alloc(g, NULL, 0, &loss);
    ref_node* nd = push_node(g, OP_CE_MASKED, logits, -1, out);
    nd->p[0] = rows; nd->p[1] = classes;
    nd->f[0] = normalizer;
    nd->aux = probs;
    nd->iaux = (int64_t*)malloc(rows * sizeof(int64_t));
    memcpy(nd->iaux, targets, rows * sizeof(int64_t));
    finish_node(g);
    return out;
}

/* Graph::transpose_0213 CPU arm (src/graph/ops/transform.rs:83-127). */
int ref_transpose_0213(ref_graph* g, int a) {
    const ref_tensor* ta = &g->t[a];
    const size_t b = ta->shape[0], s = ta->shape[1], h = ta->shape[2], d = ta->shape[3];
    size_t os[4] = {b, h, s, d};
    const int out = ref_alloc(g, os, 4, NULL);
    ref_transpose_0213_fwd(g->t[a].data, g->t[out].data, b, s, h, d);
    ref_node* nd = push_node(g, OP_T0213, a, -1, out);
    nd->p[0] = b; nd->p[1] = s; nd->p[2] = h; nd->p[3] = d;
    finish_node(g);
    return out;
}

/* Graph::gather CPU arm (src/graph/ops/transform.rs:287-324): out shape = idx.shape + [H]. */
int ref_gather(ref_graph* g, int w, int idx) {
    const size_t hidden = g->t[w].shape[1];
    const ref_tensor* ti = &g->t[idx];
    size_t os[REF_MAX_RANK];
    for (int i = 0; i < ti->rank; i++) os[i] = ti->shape[i];
    os[ti->rank] = hidden;
    const int out = ref_alloc(g, os, ti->rank + 1, NULL);
    ref_gather_fwd(g->t[w].data, g->t[idx].data, g->t[out].data, g->t[idx].numel, hidden);
    ref_node* nd = push_node(g, OP_GATHER, w, idx, out);
    nd->p[0] = g->t[idx].numel; nd->p[1] = hidden;
    finish_node(g);
    return out;
}

/* Graph::reshape CPU arm (src/graph/ops/transform.rs:389-406): a copy. */
int ref_reshape(ref_graph* g, int a, const size_t* shape, int rank) {
    const int out = ref_alloc(g, shape, rank, g->t[a].data);
    if (g->t[out].numel != g->t[a].numel) {
        fprintf(stderr, "ref_reshape: element count mismatch\n");
        abort();
    }
    push_node(g, OP_RESHAPE, a, -1, out);
    finish_node(g);
    return out;
}

/* Graph::rope CPU arm (src/graph/ops/transform.rs:541-610). */
int ref_rope(ref_graph* g, int a, size_t head_dim) {
    const ref_tensor* ta = &g->t[a];
    const int out = ref_alloc(g, ta->shape, ta->rank, NULL);
    ref_rope_fwd(g->t[a].data, g->t[out].data, ta->shape[0], ta->shape[1], ta->shape[2], head_dim);
    ref_node* nd = push_node(g, OP_ROPE, a, -1, out);
    nd->p[0] = ta->shape[0]; nd->p[1] = ta->shape[1]; nd->p[2] = ta->shape[2]; nd->p[3] = head_dim;
    finish_node(g);
    return out;
}

/* Graph::rms_norm CPU arm (src/graph/ops/normalization.rs:132-182). */
int ref_rms_norm(ref_graph* g, int x, int w, float eps) {
    const ref_tensor* tx = &g->t[x];
    const size_t dim = tx->shape[tx->rank - 1];
    const size_t nv = tx->numel / dim;
    const int out = ref_alloc(g, tx->shape, tx->rank, NULL);
    float* cache = (float*)malloc(nv * sizeof(float));
    ref_rms_norm_fwd(g->t[x].data, g->t[w].data, g->t[out].data, cache, nv, dim, eps);
    ref_node* nd = push_node(g, OP_RMSNORM, x, w, out);
    nd->p[0] = nv; nd->p[1] = dim;
    nd->aux = cache;
    finish_node(g);
    return out;
}

/* Graph::repeat_kv CPU arm (src/graph/ops/gqa.rs:13-23, :143-194). */
int ref_repeat_kv(ref_graph* g, int x, size_t repeats) {
    if (repeats == 1) return x;
    const ref_tensor* tx = &g->t[x];
    const size_t batch = tx->shape[0], kvh = tx->shape[1], seq = tx->shape[2], hd = tx->shape[3];
    size_t os[4] = {batch, kvh * repeats, seq, hd};
    const int out = ref_alloc(g, os, 4, NULL);
    ref_repeat_kv_fwd(g->t[x].data, g->t[out].data, batch, kvh, seq, hd, repeats);
    ref_node* nd = push_node(g, OP_REPEAT_KV, x, -1, out);
    nd->p[0] = batch; nd->p[1] = kvh; nd->p[2] = seq; nd->p[3] = hd; nd->p[4] = repeats;
    finish_node(g);
    return out;
}

/* Graph::flash_attention CPU arm (src/graph/ops/attention.rs:7-41, :145-191): no tape. */
int ref_flash_attention(ref_graph* g, int q, int k, int v, float scale, int causal) {
    if (!g->no_grad) {
        fprintf(stderr, "flash_attention currently supports no_grad/inference path only\n");
        abort();
    }
    const ref_tensor* tq = &g->t[q];
    const size_t batch = tq->shape[0], m = tq->shape[1], d = tq->shape[2], n = g->t[k].shape[1];
    size_t os[3] = {batch, m, d};
    const int out = ref_alloc(g, os, 3, NULL);
    ref_flash_attention_fwd(g->t[q].data, g->t[k].data, g->t[v].data, g->t[out].data, batch, m, n, d, scale,
                            causal);
    return out;
}

/* Graph::sum CPU arm (src/graph/ops/reduction.rs:149-194). */
int ref_sum(ref_graph* g, int a, int dim) {
    const ref_tensor* ta = &g->t[a];
    size_t os[REF_MAX_RANK];
    int orank = 0;
    for (int i = 0; i < ta->rank; i++)
        if (i != dim) os[orank++] = ta->shape[i];
    const int out = ref_alloc(g, os, orank, NULL);
    ta = &g->t[a];
    size_t inner = 1;
    for (int i = dim + 1; i < ta->rank; i++) inner *= ta->shape[i];
    const size_t red = ta->shape[dim];
    float* o = g->t[out].data;
    for (size_t i = 0; i < ta->numel; i++) {
        const size_t outer = i / (inner * red), in = i % inner;
        o[outer * inner + in] += ta->data[i];
    }
    ref_node* nd = push_node(g, OP_SUM, a, -1, out);
    nd->p[0] = inner; nd->p[1] = red;
    finish_node(g);
    return out;
}

/* Graph::max CPU arm (src/graph/ops/reduction.rs:352-396): first strict maximum wins. */
int ref_max(ref_graph* g, int a, int dim) {
    const ref_tensor* ta = &g->t[a];
    size_t os[REF_MAX_RANK];
    int orank = 0;
    for (int i = 0; i < ta->rank; i++)
        if (i != dim) os[orank++] = ta->shape[i];
    const int out = ref_alloc(g, os, orank, NULL);
    ta = &g->t[a];
    size_t inner = 1;
    for (int i = dim + 1; i < ta->rank; i++) inner *= ta->shape[i];
    const size_t red = ta->shape[dim];
    float* o = g->t[out].data;
    const size_t on = g->t[out].numel;
    int64_t* argmax = (int64_t*)calloc(on, sizeof(int64_t));
    for (size_t i = 0; i < on; i++) o[i] = -INFINITY;
    for (size_t i = 0; i < ta->numel; i++) {
        const size_t idx = (i / (inner * red)) * inner + i % inner;
        if (ta->data[i] > o[idx]) {
            o[idx] = ta->data[i];
            argmax[idx] = (int64_t)i;
        }
    }
    ref_node* nd = push_node(g, OP_MAX, a, -1, out);
    nd->iaux = argmax;
    finish_node(g);
    return out;
}

/* Graph::transpose CPU arm (src/graph/ops/transform.rs:428-465). */
int ref_transpose(ref_graph* g, int a, int dim0, int dim1) {
    const ref_tensor* ta = &g->t[a];
    size_t os[REF_MAX_RANK], st[REF_MAX_RANK];
    size_t cur = 1;
    for (int i = ta->rank - 1; i >= 0; i--) {
        st[i] = cur;
        cur *= ta->shape[i];
        os[i] = ta->shape[i];
    }
    size_t tmp = os[dim0]; os[dim0] = os[dim1]; os[dim1] = tmp;
    tmp = st[dim0]; st[dim0] = st[dim1]; st[dim1] = tmp;
    const int rank = ta->rank;
    const int out = ref_alloc(g, os, rank, NULL);
    ta = &g->t[a];
    for (size_t i = 0; i < ta->numel; i++) g->t[out].data[i] = ta->data[bcast_index(i, os, rank, st)];
    ref_node* nd = push_node(g, OP_TRANSPOSE, a, -1, out);
    for (int i = 0; i < rank; i++) nd->p[i] = st[i];
    finish_node(g);
    return out;
}

static void node_backward(ref_graph* g, const ref_node* nd) {
    ref_tensor* T = g->t;
    const float* go = T[nd->out].grad;
    switch (nd->op) {
    case OP_ADD: { /* src/graph/ops/elementwise.rs:166-174 */
        size_t os[REF_MAX_RANK], sa[REF_MAX_RANK], sb[REF_MAX_RANK];
        int orank;
        bcast_shape(&T[nd->in0], &T[nd->in1], os, &orank);
        bcast_strides(&T[nd->in0], os, orank, sa);
        bcast_strides(&T[nd->in1], os, orank, sb);
        const size_t n = T[nd->out].numel;
        if (T[nd->in0].numel == n && T[nd->in1].numel == n && nd->in0 != nd->in1) {
            float* ga = T[nd->in0].grad;
            float* gb = T[nd->in1].grad;
            for (size_t i = 0; i < n; i++) { ga[i] += go[i]; gb[i] += go[i]; }
        } else {
            for (size_t i = 0; i < n; i++) {
                T[nd->in0].grad[bcast_index(i, os, orank, sa)] += go[i];
                T[nd->in1].grad[bcast_index(i, os, orank, sb)] += go[i];
            }
        }
    } break;
    case OP_MUL: { /* src/graph/ops/elementwise.rs:314-322 */
        size_t os[REF_MAX_RANK], sa[REF_MAX_RANK], sb[REF_MAX_RANK];
        int orank;
        bcast_shape(&T[nd->in0], &T[nd->in1], os, &orank);
        bcast_strides(&T[nd->in0], os, orank, sa);
        bcast_strides(&T[nd->in1], os, orank, sb);
        const size_t n = T[nd->out].numel;
        for (size_t i = 0; i < n; i++) {
            const size_t ia = bcast_index(i, os, orank, sa), ib = bcast_index(i, os, orank, sb);
            T[nd->in0].grad[ia] += T[nd->in1].data[ib] * go[i];
            if (!nd->discard_in1_grad) T[nd->in1].grad[ib] += T[nd->in0].data[ia] * go[i];
        }
    } break;
    case OP_SILU:
        ref_silu_bwd(T[nd->in0].data, go, T[nd->in0].grad, T[nd->in0].numel);
        break;
    case OP_MATMUL:
        ref_matmul_bwd(T[nd->in0].data, T[nd->in1].data, go, T[nd->in0].grad, T[nd->in1].grad, nd->p[0], nd->p[1],
                       nd->p[2]);
        break;
    case OP_MATMUL_TB:
        ref_matmul_trans_b_bwd(T[nd->in0].data, T[nd->in1].data, go, T[nd->in0].grad, T[nd->in1].grad, nd->p[0],
                               nd->p[1], nd->p[2]);
        break;
    case OP_BMM:
        ref_bmm_bwd(T[nd->in0].data, T[nd->in1].data, go, T[nd->in0].grad, T[nd->in1].grad, nd->p[0], nd->p[1],
                    nd->p[2], nd->p[3], (int)nd->p[4]);
        break;
    case OP_SOFTMAX:
        ref_softmax_bwd(T[nd->out].data, go, T[nd->in0].grad, nd->p[0], nd->p[1]);
        break;
    case OP_CE:
        ref_cross_entropy_bwd(nd->aux, nd->iaux, go[0], T[nd->in0].grad, nd->p[0], nd->p[1]);
        break;
    case OP_CE_MASKED:
        ref_cross_entropy_masked_bwd(nd->aux, nd->iaux, go[0], T[nd->in0].grad, nd->p[0], nd->p[1], nd->f[0]);
        break;
    case OP_T0213:
        ref_transpose_0213_bwd(go, T[nd->in0].grad, nd->p[0], nd->p[1], nd->p[2], nd->p[3]);
        break;
    case OP_GATHER:
        ref_gather_bwd(T[nd->in1].data, go, T[nd->in0].grad, nd->p[0], nd->p[1]);
        break;
    case OP_RESHAPE: { /* src/graph/ops/transform.rs:392-398 */
        float* ga = T[nd->in0].grad;
        for (size_t i = 0; i < T[nd->in0].numel; i++) ga[i] += go[i];
    } break;
    case OP_ROPE:
        ref_rope_bwd(go, T[nd->in0].grad, nd->p[0], nd->p[1], nd->p[2], nd->p[3]);
        break;
    case OP_RMSNORM:
        ref_rms_norm_bwd(T[nd->in0].data, T[nd->in1].data, nd->aux, go, T[nd->in0].grad, T[nd->in1].grad, nd->p[0],
                         nd->p[1]);
        break;
    case OP_REPEAT_KV:
        ref_repeat_kv_bwd(go, T[nd->in0].grad, nd->p[0], nd->p[1], nd->p[2], nd->p[3], nd->p[4]);
        break;
    case OP_SUM: { /* src/graph/ops/reduction.rs:174-185 */
        const size_t inner = nd->p[0], red = nd->p[1];
        float* ga = T[nd->in0].grad;
        for (size_t i = 0; i < T[nd->in0].numel; i++) ga[i] += go[(i / (inner * red)) * inner + i % inner];
    } break;
    case OP_MAX: { /* src/graph/ops/reduction.rs:379-384 */
        for (size_t i = 0; i < T[nd->out].numel; i++) T[nd->in0].grad[nd->iaux[i]] += go[i];
    } break;
    case OP_TRANSPOSE: { /* src/graph/ops/transform.rs:447-454 */
        const ref_tensor* to = &T[nd->out];
        for (size_t i = 0; i < to->numel; i++) T[nd->in0].grad[bcast_index(i, to->shape, to->rank, nd->p)] += go[i];
    } break;
    default:
        fprintf(stderr, "node_backward: unknown op %d\n", nd->op);
        abort();
    }
}

/* Graph::backward (src/graph/mod.rs:670-711, :795): seed every element of the loss grad
 * with 1.0, replay the tape in reverse insertion order, keep the tape. */
void ref_backward(ref_graph* g, int loss_id) {
    if (g->no_grad) return;
    for (size_t i = 0; i < g->t[loss_id].numel; i++) g->t[loss_id].grad[i] = 1.0f;
    for (int i = g->nn - 1; i >= 0; i--) node_backward(g, &g->nodes[i]);
}

/* ------------------------------------------------------------------------- */
/* nn modules (src/nn/*.rs)                                                  */
/* ------------------------------------------------------------------------- */

typedef struct {
    int norm1, wq, wk, wv, wo, norm2, w_gate, w_up, w_down;
} ref_block;

typedef struct ref_lm {
    size_t vocab, hidden, heads, kv_heads, head_dim, ffn, layers;
    int tie;
    int emb, norm_f, lm_head;
    ref_block* blocks;
} ref_lm;

/* Parameter tensors are allocated in the reference's construction order
 * (src/nn/transformer.rs:19-28, :77-117): embedding; per block norm1, q, k, v, o,
 * norm2, gate, up (ffn1), down (ffn2); final norm; lm_head unless tied.
 * Norm gains start at 1.0 (src/nn/rmsnorm.rs:11-20); matrices start at zero here and
 * are loaded by the caller (the configurations prescribe their own seeded weights). */
ref_lm* ref_lm_new(ref_graph* g, size_t vocab, size_t hidden, size_t heads, size_t kv_heads, size_t ffn,
                   size_t layers, int tie) {
    ref_lm* lm = (ref_lm*)calloc(1, sizeof(ref_lm));
    lm->vocab = vocab; lm->hidden = hidden; lm->heads = heads; lm->kv_heads = kv_heads;
    lm->head_dim = hidden / heads; lm->ffn = ffn; lm->layers = layers; lm->tie = tie;
    const size_t kv_dim = kv_heads * lm->head_dim;
    float* ones = (float*)malloc(hidden * sizeof(float));
    for (size_t i = 0; i < hidden; i++) ones[i] = 1.0f;
    size_t s2[2];
    s2[0] = vocab; s2[1] = hidden;
    lm->emb = ref_alloc(g, s2, 2, NULL);
    lm->blocks = (ref_block*)calloc(layers, sizeof(ref_block));
    for (size_t l = 0; l < layers; l++) {
        ref_block* b = &lm->blocks[l];
        b->norm1 = ref_alloc(g, &hidden, 1, ones);
        s2[0] = hidden; s2[1] = hidden; b->wq = ref_alloc(g, s2, 2, NULL);
        s2[0] = hidden; s2[1] = kv_dim; b->wk = ref_alloc(g, s2, 2, NULL);
        b->wv = ref_alloc(g, s2, 2, NULL);
        s2[0] = hidden; s2[1] = hidden; b->wo = ref_alloc(g, s2, 2, NULL);
        b->norm2 = ref_alloc(g, &hidden, 1, ones);
        s2[0] = hidden; s2[1] = ffn; b->w_gate = ref_alloc(g, s2, 2, NULL);
        b->w_up = ref_alloc(g, s2, 2, NULL);
        s2[0] = ffn; s2[1] = hidden; b->w_down = ref_alloc(g, s2, 2, NULL);
    }
    lm->norm_f = ref_alloc(g, &hidden, 1, ones);
    if (tie) {
        lm->lm_head = lm->emb;
    } else {
        s2[0] = hidden; s2[1] = vocab;
        lm->lm_head = ref_alloc(g, s2, 2, NULL);
    }
    free(ones);
    return lm;
}
void ref_lm_free(ref_lm* lm) {
    free(lm->blocks);
    free(lm);
}

/* TransformerLM::params order (src/nn/transformer.rs:198-210; block order :57-66 is
 * norm1, q, k, v, o, norm2, ffn1(up), ffn2(down), gate).  Returns the count. */
int ref_lm_params(const ref_lm* lm, int* out) {
    int n = 0;
    out[n++] = lm->emb;
    for (size_t l = 0; l < lm->layers; l++) {
        const ref_block* b = &lm->blocks[l];
        out[n++] = b->norm1; out[n++] = b->wq; out[n++] = b->wk; out[n++] = b->wv; out[n++] = b->wo;
        out[n++] = b->norm2; out[n++] = b->w_up; out[n++] = b->w_down; out[n++] = b->w_gate;
    }
    out[n++] = lm->norm_f;
    if (!lm->tie) out[n++] = lm->lm_head;
    return n;
}

/* Linear::forward (src/nn/linear.rs:53-95): matmul over flattened rows, 3-D shape restored. */
static int linear_forward(ref_graph* g, int w, int x) {
    const ref_tensor* tx = &g->t[x];
    const int is3d = tx->rank == 3;
    const size_t b0 = tx->shape[0], b1 = tx->shape[1];
    const int out = ref_matmul(g, x, w);
    if (is3d) {
        size_t s3[3] = {b0, b1, g->t[w].shape[1]};
        ref_reinterpret_shape(g, out, s3, 3);
    }
    return out;
}

/* GroupedQueryAttention::forward_with_mask (src/nn/attention.rs:289-388). */
int ref_gqa_forward(ref_graph* g, size_t heads, size_t kv_heads, size_t head_dim, int wq, int wk, int wv, int wo,
                    int x, int causal) {
    const size_t batch = g->t[x].shape[0], seq = g->t[x].shape[1];
    const size_t hidden = heads * head_dim;
    const int q = linear_forward(g, wq, x);
    const int k = linear_forward(g, wk, x);
    const int v = linear_forward(g, wv, x);
    const int q_rope = ref_rope(g, q, head_dim);
    const int k_rope = ref_rope(g, k, head_dim);
    size_t s4[4] = {batch, seq, heads, head_dim};
    const int q4 = ref_reshape(g, q_rope, s4, 4);
    s4[2] = kv_heads;
    const int k4 = ref_reshape(g, k_rope, s4, 4);
    const int v4 = ref_reshape(g, v, s4, 4);
    const int qt = ref_transpose_0213(g, q4);
    const int kt = ref_transpose_0213(g, k4);
    const int vt = ref_transpose_0213(g, v4);
    const size_t repeats = heads / kv_heads;
    const int kr = ref_repeat_kv(g, kt, repeats);
    const int vr = ref_repeat_kv(g, vt, repeats);
    const size_t bh = batch * heads;
    size_t s3[3] = {bh, seq, head_dim};
    ref_reinterpret_shape(g, qt, s3, 3);
    ref_reinterpret_shape(g, kr, s3, 3);
    ref_reinterpret_shape(g, vr, s3, 3);
    const float scale = 1.0f / sqrtf((float)head_dim);
    int ctx;
    if (g->no_grad) {
        ctx = ref_flash_attention(g, qt, kr, vr, scale, causal);
    } else {
        const int scores = ref_bmm(g, qt, kr, 1);
        size_t ss[3] = {bh, seq, seq};
        const int scale_id = ref_alloc(g, ss, 3, NULL);
        for (size_t i = 0; i < g->t[scale_id].numel; i++) g->t[scale_id].data[i] = scale;
        int scaled = ref_mul_ex(g, scores, scale_id, 1);
        if (causal) {
            size_t ms[3] = {1, seq, seq};
            const int mask = ref_alloc(g, ms, 3, NULL);
            for (size_t r = 0; r < seq; r++)
                for (size_t c = r + 1; c < seq; c++) g->t[mask].data[r * seq + c] = -1e20f;
            scaled = ref_add(g, scaled, mask);
        }
        const int probs = ref_softmax(g, scaled);
        ctx = ref_bmm(g, probs, vr, 0);
    }
    size_t c4[4] = {batch, heads, seq, head_dim};
    ref_reinterpret_shape(g, ctx, c4, 4);
    const int ctx_t = ref_transpose_0213(g, ctx);
    size_t c3[3] = {batch, seq, hidden};
    const int ctx_flat = ref_reshape(g, ctx_t, c3, 3);
    return linear_forward(g, wo, ctx_flat);
}

/* TransformerBlock::forward_with_mask (src/nn/transformer.rs:31-49). */
static int block_forward(ref_graph* g, const ref_lm* lm, const ref_block* b, int x) {
    const int norm1 = ref_rms_norm(g, x, b->norm1, 1e-5f);
    const int attn = ref_gqa_forward(g, lm->heads, lm->kv_heads, lm->head_dim, b->wq, b->wk, b->wv, b->wo, norm1, 1);
    const int res1 = ref_add(g, x, attn);
    const int norm2 = ref_rms_norm(g, res1, b->norm2, 1e-5f);
    const int gate_out = linear_forward(g, b->w_gate, norm2);
    const int gate = ref_silu(g, gate_out);
    const int up = linear_forward(g, b->w_up, norm2);
    const int gated = ref_mul(g, gate, up);
    const int down = linear_forward(g, b->w_down, gated);
    return ref_add(g, res1, down);
}

/* TransformerLM::forward (src/nn/transformer.rs:184-196). */
int ref_lm_forward(ref_graph* g, const ref_lm* lm, int x_id) {
    int h = ref_gather(g, lm->emb, x_id);
    for (size_t l = 0; l < lm->layers; l++) h = block_forward(g, lm, &lm->blocks[l], h);
    h = ref_rms_norm(g, h, lm->norm_f, 1e-5f);
    if (lm->tie) return ref_matmul_trans_b(g, h, lm->lm_head);
    return linear_forward(g, lm->lm_head, h);
}

/* One micro-step of examples/train_llm.rs:433-458: upload ids, forward, flatten logits,
 * cross entropy, backward, clear activations.  ids are f32 token ids [mb*seq]; targets
 * int64.  Returns the micro-batch loss. */
float ref_lm_micro_step(ref_graph* g, const ref_lm* lm, const float* ids, const int64_t* targets, size_t mb,
                        size_t seq) {
    size_t xs[2] = {mb, seq};
    const int x_id = ref_alloc(g, xs, 2, ids);
    const int logits = ref_lm_forward(g, lm, x_id);
    size_t fs[2] = {mb * seq, lm->vocab};
    const int flat = ref_reshape(g, logits, fs, 2);
    const int loss = ref_cross_entropy_masked(g, flat, targets);
    const float lv = g->t[loss].data[0];
    ref_backward(g, loss);
    ref_clear_activations(g);
    return lv;
}

/* AdamW (src/nn/optim.rs). */
typedef struct ref_adamw {
    int* params;
    int nparams;
    float lr, beta1, beta2, eps, weight_decay;
    int t;
    float** m;
    float** v;
    float grad_clip_norm; /* <= 0: none */
    float last_grad_norm, last_grad_scale;
} ref_adamw;

/* AdamW::new defaults (src/nn/optim.rs:32-52). */
ref_adamw* ref_adamw_new(ref_graph* g, const int* params, int nparams, float lr) {
    ref_adamw* o = (ref_adamw*)calloc(1, sizeof(ref_adamw));
    o->params = (int*)malloc((size_t)nparams * sizeof(int));
    memcpy(o->params, params, (size_t)nparams * sizeof(int));
    o->nparams = nparams;
    o->lr = lr; o->beta1 = 0.9f; o->beta2 = 0.999f; o->eps = 1e-8f; o->weight_decay = 0.01f;
    o->m = (float**)calloc((size_t)nparams, sizeof(float*));
    o->v = (float**)calloc((size_t)nparams, sizeof(float*));
    for (int i = 0; i < nparams; i++) {
        o->m[i] = (float*)calloc(g->t[params[i]].numel, sizeof(float));
        o->v[i] = (float*)calloc(g->t[params[i]].numel, sizeof(float));
    }
    o->last_grad_scale = 1.0f;
    return o;
}
void ref_adamw_free(ref_adamw* o) {
    for (int i = 0; i < o->nparams; i++) { free(o->m[i]); free(o->v[i]); }
    free(o->m); free(o->v); free(o->params); free(o);
}
void ref_adamw_config(ref_adamw* o, float lr, float beta1, float beta2, float eps, float wd, float clip) {
    o->lr = lr; o->beta1 = beta1; o->beta2 = beta2; o->eps = eps; o->weight_decay = wd;
    o->grad_clip_norm = clip;
}
float* ref_adamw_m(ref_adamw* o, int i) { return o->m[i]; }
float* ref_adamw_v(ref_adamw* o, int i) { return o->v[i]; }
int ref_adamw_t(ref_adamw* o) { return o->t; }
float ref_adamw_last_grad_norm(ref_adamw* o) { return o->last_grad_norm; }

/* AdamW::zero_grad (src/nn/optim.rs:207-245). */
void ref_adamw_zero_grad(ref_adamw* o, ref_graph* g) {
    for (int i = 0; i < o->nparams; i++) ref_zero_grad(g, o->params[i]);
}
/* AdamW::clip_grad_norm (src/nn/optim.rs:250-321).  Returns the norm; *coef the factor. */
float ref_adamw_clip_grad_norm(ref_adamw* o, ref_graph* g, float max_norm, float* coef_out) {
    double ss = 0.0;
    for (int i = 0; i < o->nparams; i++) ss = ref_sum_squares_f64(g->t[o->params[i]].grad, g->t[o->params[i]].numel, ss);
    float norm;
    const float coef = ref_clip_coef(ss, max_norm, &norm);
    if (coef < 1.0f)
        for (int i = 0; i < o->nparams; i++) {
            float* gr = g->t[o->params[i]].grad;
            for (size_t e = 0; e < g->t[o->params[i]].numel; e++) gr[e] *= coef;
        }
    if (coef_out) *coef_out = coef;
    return norm;
}
/* AdamW::maybe_clip_gradients (src/nn/optim.rs:114-200): differs from clip_grad_norm in
 * two details -- the f64 sum is narrowed to f32 before the square root, and the scale is
 * 1 unless norm > max_norm. */
static void adamw_maybe_clip(ref_adamw* o, ref_graph* g) {
    if (!(o->grad_clip_norm > 0.0f)) {
        o->last_grad_norm = 0.0f;
        o->last_grad_scale = 1.0f;
        return;
    }
    double ss = 0.0;
    for (int i = 0; i < o->nparams; i++) ss = ref_sum_squares_f64(g->t[o->params[i]].grad, g->t[o->params[i]].numel, ss);
    const float norm = sqrtf((float)ss);
    const float scale = norm > o->grad_clip_norm ? o->grad_clip_norm / (norm + 1e-6f) : 1.0f;
    o->last_grad_norm = norm;
    o->last_grad_scale = scale;
    if (scale >= 1.0f) return;
    for (int i = 0; i < o->nparams; i++) {
        float* gr = g->t[o->params[i]].grad;
        for (size_t e = 0; e < g->t[o->params[i]].numel; e++) gr[e] *= scale;
    }
}
/* AdamW::step (src/nn/optim.rs:334-338, :523-543). */
void ref_adamw_step(ref_adamw* o, ref_graph* g) {
    adamw_maybe_clip(o, g);
    o->t += 1;
    float bc1, bc2;
    ref_adamw_bias_corrections(o->beta1, o->beta2, o->t, &bc1, &bc2);
    for (int i = 0; i < o->nparams; i++) {
        ref_tensor* p = &g->t[o->params[i]];
        ref_adamw_update(p->data, p->grad, o->m[i], o->v[i], p->numel, o->lr, o->beta1, o->beta2, o->eps,
                         o->weight_decay, bc1, bc2);
    }
}
