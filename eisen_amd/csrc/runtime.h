// Internal: the context behind the C-ABI handles and the helpers every op file shares.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/eisen_hip.h"

struct eisen_rope_table {
    size_t seq = 0, head_dim = 0;
    float* cos_sin = nullptr;  // [seq][head_dim/2][2] f32 on the device
};

// Optional per-kernel timing: every instrumented launch is bracketed by two events on the stream.
struct eisen_prof_rec {
    int key;
    hipEvent_t start, stop;
    double work;  // algorithmic flops or bytes of the launch
};
struct eisen_prof {
    bool enabled = false;
    std::vector<std::string> names;
    std::vector<int> is_flops;
    std::vector<hipEvent_t> pool;
    size_t pool_used = 0;
    std::vector<eisen_prof_rec> recs;
};

struct eisen_ctx {
    int device = 0;
    hipStream_t stream = nullptr;       // the stream every entry point launches on (the side stream between side_begin and side_end)
    hipStream_t main_stream = nullptr, side_stream = nullptr;
    hipEvent_t ev_fork = nullptr, ev_side = nullptr;
    bool side_active = false, side_pending = false;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    bool timer_running = false;
    // size-keyed free lists in front of hipMallocAsync (exact-size buckets, like the
    // reference's vram_pool keyed by element count)
    std::unordered_map<size_t, std::vector<void*>> free_lists;
    std::unordered_map<void*, size_t> live;
    size_t in_use_bytes = 0, cached_bytes = 0;
    size_t peak_in_use_bytes = 0;  // high-water mark of in_use_bytes since the last reset
    size_t driver_allocs = 0;      // requests for memory that reached the driver (device pool misses, workspace growth, tables, pinned staging)
    // pinned staging ring for asynchronous uploads: a slot is reused only after its copy's event fired
    struct StageSlot {
        void* ptr = nullptr;
        size_t bytes = 0;
        hipEvent_t done = nullptr;
        bool in_flight = false;
        bool reserved = false;  // holds the result of a device-to-host copy that eisen_hip_dtoh_finish has not collected yet
    };
    static constexpr int kStageSlots = 16;
    StageSlot stage[kStageSlots];
    int stage_next = 0;
    // grow-only device workspace for two-stage reductions and tables
    void* ws = nullptr;
    size_t ws_bytes = 0;
    void* ws_side = nullptr;  // the same for launches on the side stream, which run beside main-stream kernels that use `ws`
    size_t ws_side_bytes = 0;
    std::vector<eisen_rope_table> rope_tables;
    float* attn_scratch = nullptr;  // this device's copy of the file-scope scratch array in attention.hip (never freed)
    int attn_ablation = 0;  // measurement only: the part of the attention backward kernels' tile loop to leave out (0 = none)
    long long* attn_stamps = nullptr;  // measurement only: where the attention kernels drop time stamps (eisen_hip_attention_timeline)
    int attn_stamp_waves = 0;
    int window_meet_us = 40;  // longest wait at a meeting point of the windowed weight-gradient GEMM (eisen_hip_gemm_window_meet); 0 = none
    eisen_prof prof;
    char last_error[512] = {0};
};

// cos/sin table of the rotary embedding, [seq][head_dim/2] float2 on the device, cached in the context (rope.hip)
int eisen_rope_table_get(eisen_ctx* ctx, size_t seq, size_t head_dim, const float2** out);

// Looks up, once per device, the device address of the file-scope scratch array that eisen_hip_attention_backward_noalloc
// uses, and stores it in the context (attention.hip); called by eisen_hip_init with the context's device current.
int eisen_attention_scratch_init(eisen_ctx* ctx);

// Brackets the launches issued during its lifetime when profiling is on; free when it is off.
int eisen_prof_begin(eisen_ctx* ctx, const char* name, double work, bool is_flops);
void eisen_prof_end(eisen_ctx* ctx, int rec);
struct EisenProfScope {
    eisen_ctx* ctx;
    int rec;
    EisenProfScope(eisen_ctx* c, const char* name, double work, bool is_flops = false)
        : ctx(c), rec(c->prof.enabled ? eisen_prof_begin(c, name, work, is_flops) : -1) {}
    ~EisenProfScope() {
        if (rec >= 0) eisen_prof_end(ctx, rec);
    }
};

struct eisen_module {
    hipModule_t mod;
};
struct eisen_function {
    hipFunction_t fn;
};

int eisen_set_error(eisen_ctx* ctx, int code, const char* fmt, ...);
// Returns a device workspace of at least `bytes` (grow-only, stream-ordered reuse).
int eisen_workspace(eisen_ctx* ctx, size_t bytes, void** out);
// Next pinned staging slot, grown to at least `bytes`; waits only if that slot's last copy is still in flight.
int eisen_staging(eisen_ctx* ctx, size_t bytes, eisen_ctx::StageSlot** out);

#define EISEN_HIP_TRY(ctx, expr)                                                              \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess)                                                                 \
            return eisen_set_error((ctx), (int)_e, "%s failed: %s (%s:%d)", #expr,           \
                                   hipGetErrorString(_e), __FILE__, __LINE__);                \
    } while (0)

#define EISEN_REQUIRE(ctx, cond, code, ...)                                                   \
    do {                                                                                      \
        if (!(cond)) return eisen_set_error((ctx), (code), __VA_ARGS__);                      \
    } while (0)

#define EISEN_CHECK_CTX(ctx)        \
    do {                            \
        if (!(ctx)) return EISEN_E_ARG; \
    } while (0)

#define EISEN_LAUNCH_CHECK(ctx, name)                                                         \
    do {                                                                                      \
        hipError_t _e = hipGetLastError();                                                    \
        if (_e != hipSuccess)                                                                 \
            return eisen_set_error((ctx), (int)_e, "launch of %s failed: %s", (name),         \
                                   hipGetErrorString(_e));                                    \
    } while (0)

static inline bool eisen_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
static inline size_t eisen_dtype_size(int dtype) { return dtype == EISEN_BF16 ? 2 : 4; }
static inline bool eisen_dtype_ok(int dtype) { return dtype == EISEN_F32 || dtype == EISEN_BF16; }
static inline size_t eisen_ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
