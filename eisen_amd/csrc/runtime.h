// Internal: the context behind the C-ABI handles and the helpers every op file shares.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <unordered_map>
#include <vector>

#include "../../include/eisen_hip.h"

struct eisen_rope_table {
    size_t seq = 0, head_dim = 0;
    float* cos_sin = nullptr;  // [seq][head_dim/2][2] f32 on the device
};

struct eisen_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    bool timer_running = false;
    // size-keyed free lists in front of hipMallocAsync (exact-size buckets, like the
    // reference's vram_pool keyed by element count)
    std::unordered_map<size_t, std::vector<void*>> free_lists;
    std::unordered_map<void*, size_t> live;
    size_t in_use_bytes = 0, cached_bytes = 0;
    // pinned staging for asynchronous uploads
    void* stage = nullptr;
    size_t stage_bytes = 0;
    // grow-only device workspace for two-stage reductions and tables
    void* ws = nullptr;
    size_t ws_bytes = 0;
    std::vector<eisen_rope_table> rope_tables;
    char last_error[512] = {0};
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
// Pinned staging buffer of at least `bytes`; waits for earlier uploads that still read it.
int eisen_staging(eisen_ctx* ctx, size_t bytes, void** out);

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
