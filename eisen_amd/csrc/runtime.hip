// Runtime half of the C-ABI: context, one stream, stream-ordered pool, copies, module
// load / launch by name, event timer.  Replaces the cudarc calls of the reference
// (src/graph/mod.rs:152-307, src/graph/memory.rs:189-266, src/tensor.rs:145-223).
#include "runtime.h"

int eisen_set_error(eisen_ctx* ctx, int code, const char* fmt, ...) {
    if (ctx) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(ctx->last_error, sizeof(ctx->last_error), fmt, ap);
        va_end(ap);
    }
    return code;
}

extern "C" const char* eisen_hip_last_error(eisen_ctx* ctx) { return ctx ? ctx->last_error : "null context"; }

extern "C" int eisen_hip_init(int device, eisen_ctx** out) {
    if (!out) return EISEN_E_ARG;
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) return (int)e;
    if (device < 0 || device >= count) return EISEN_E_ARG;
    e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    eisen_ctx* ctx = new eisen_ctx();
    ctx->device = device;
    // default priority, non-blocking with respect to the legacy null stream
    e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    ctx->main_stream = ctx->stream;
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&ctx->side_stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&ctx->ev_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&ctx->ev_side, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev_start);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev_stop);
    if (e == hipSuccess) {
        // keep freed blocks inside the driver pool instead of returning them to the OS
        hipMemPool_t pool;
        if (hipDeviceGetDefaultMemPool(&pool, device) == hipSuccess) {
            uint64_t threshold = UINT64_MAX;
            (void)hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &threshold);
        }
        (void)hipGetLastError();
    }
    if (e != hipSuccess) {
        delete ctx;
        return (int)e;
    }
    const int rc = eisen_attention_scratch_init(ctx);
    if (rc != 0) {
        (void)eisen_hip_destroy(ctx);
        return rc;
    }
    *out = ctx;
    return 0;
}

extern "C" int eisen_hip_pool_trim(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    EISEN_HIP_TRY(ctx, hipSetDevice(ctx->device));
    // every block leaves the lists before it is freed, so a failing hipFreeAsync cannot leave a freed pointer behind
    hipError_t first = hipSuccess;
    for (auto& kv : ctx->free_lists) {
        while (!kv.second.empty()) {
            void* p = kv.second.back();
            kv.second.pop_back();
            ctx->cached_bytes -= kv.first;
            const hipError_t e = hipFreeAsync(p, ctx->stream);
            if (e != hipSuccess && first == hipSuccess) first = e;
        }
    }
    ctx->free_lists.clear();
    ctx->cached_bytes = 0;
    if (first != hipSuccess) {
        (void)hipGetLastError();
        return eisen_set_error(ctx, (int)first, "eisen_hip_pool_trim: hipFreeAsync failed: %s", hipGetErrorString(first));
    }
    return 0;
}

extern "C" int eisen_hip_destroy(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    (void)hipSetDevice(ctx->device);
    ctx->stream = ctx->main_stream;
    (void)hipStreamSynchronize(ctx->side_stream);
    (void)hipStreamSynchronize(ctx->stream);
    (void)eisen_hip_pool_trim(ctx);
    for (auto& kv : ctx->live) (void)hipFreeAsync(kv.first, ctx->stream);
    for (auto& t : ctx->rope_tables) (void)hipFreeAsync(t.cos_sin, ctx->stream);
    if (ctx->ws) (void)hipFreeAsync(ctx->ws, ctx->stream);
    if (ctx->ws_side) (void)hipFreeAsync(ctx->ws_side, ctx->side_stream);
    (void)hipStreamSynchronize(ctx->side_stream);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto& sl : ctx->stage) {
        if (sl.ptr) (void)hipHostFree(sl.ptr);
        if (sl.done) (void)hipEventDestroy(sl.done);
    }
    for (hipEvent_t e : ctx->prof.pool) (void)hipEventDestroy(e);
    (void)hipEventDestroy(ctx->ev_start);
    (void)hipEventDestroy(ctx->ev_stop);
    (void)hipEventDestroy(ctx->ev_fork);
    (void)hipEventDestroy(ctx->ev_side);
    (void)hipStreamDestroy(ctx->side_stream);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return 0;
}

// Work issued between side_begin and side_end runs on a second stream, after everything issued before side_begin and
// concurrently with what the main stream is given next; side_wait makes the main stream wait for it.
extern "C" int eisen_hip_side_begin(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, !ctx->side_active, EISEN_E_ARG, "eisen_hip_side_begin: already on the side stream");
    EISEN_HIP_TRY(ctx, hipEventRecord(ctx->ev_fork, ctx->main_stream));
    EISEN_HIP_TRY(ctx, hipStreamWaitEvent(ctx->side_stream, ctx->ev_fork, 0));
    ctx->stream = ctx->side_stream;
    ctx->side_active = true;
    return 0;
}
extern "C" int eisen_hip_side_end(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ctx->side_active, EISEN_E_ARG, "eisen_hip_side_end: not on the side stream");
    ctx->stream = ctx->main_stream;
    ctx->side_active = false;
    EISEN_HIP_TRY(ctx, hipEventRecord(ctx->ev_side, ctx->side_stream));
    ctx->side_pending = true;
    return 0;
}
extern "C" int eisen_hip_side_wait(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, !ctx->side_active, EISEN_E_ARG, "eisen_hip_side_wait: still on the side stream");
    if (ctx->side_pending) EISEN_HIP_TRY(ctx, hipStreamWaitEvent(ctx->main_stream, ctx->ev_side, 0));
    ctx->side_pending = false;
    return 0;
}

extern "C" int eisen_hip_stream_sync(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    if (ctx->side_pending || ctx->side_active) EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->side_stream));
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->main_stream));
    return 0;
}

extern "C" void* eisen_hip_stream(eisen_ctx* ctx) { return ctx ? (void*)ctx->stream : nullptr; }

extern "C" int eisen_hip_malloc(eisen_ctx* ctx, size_t bytes, void** out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out != nullptr, EISEN_E_ARG, "eisen_hip_malloc: out is null");
    if (bytes == 0) bytes = 4;
    bytes = (bytes + 255) & ~size_t(255);  // 256-byte granules keep every block 16-byte aligned
    void* p = nullptr;
    auto it = ctx->free_lists.find(bytes);
    if (it != ctx->free_lists.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        ctx->cached_bytes -= bytes;
    } else {
        ctx->driver_allocs++;
        hipError_t e = hipMallocAsync(&p, bytes, ctx->stream);
        if (e != hipSuccess) {
            // out of memory: give cached blocks back and retry once
            (void)hipGetLastError();
            (void)eisen_hip_pool_trim(ctx);
            (void)hipStreamSynchronize(ctx->stream);
            e = hipMallocAsync(&p, bytes, ctx->stream);
            if (e != hipSuccess)
                return eisen_set_error(ctx, (int)e, "hipMallocAsync(%zu bytes) failed: %s", bytes,
                                       hipGetErrorString(e));
        }
    }
    ctx->live[p] = bytes;
    ctx->in_use_bytes += bytes;
    if (ctx->in_use_bytes > ctx->peak_in_use_bytes) ctx->peak_in_use_bytes = ctx->in_use_bytes;
    *out = p;
    return 0;
}

extern "C" int eisen_hip_malloc_zeroed(eisen_ctx* ctx, size_t bytes, void** out) {
    int rc = eisen_hip_malloc(ctx, bytes, out);
    if (rc) return rc;
    return eisen_hip_memset_zero(ctx, *out, ctx->live[*out]);
}

extern "C" int eisen_hip_free(eisen_ctx* ctx, void* ptr) {
    EISEN_CHECK_CTX(ctx);
    if (!ptr) return 0;
    auto it = ctx->live.find(ptr);
    EISEN_REQUIRE(ctx, it != ctx->live.end(), EISEN_E_ARG, "eisen_hip_free: %p was not allocated by this context", ptr);
    const size_t bytes = it->second;
    ctx->live.erase(it);
    ctx->in_use_bytes -= bytes;
    ctx->free_lists[bytes].push_back(ptr);
    ctx->cached_bytes += bytes;
    return 0;
}

extern "C" int eisen_hip_pool_peak(eisen_ctx* ctx, size_t* peak_in_use_bytes, int reset) {
    EISEN_CHECK_CTX(ctx);
    if (peak_in_use_bytes) *peak_in_use_bytes = ctx->peak_in_use_bytes;
    if (reset) ctx->peak_in_use_bytes = ctx->in_use_bytes;
    return 0;
}

extern "C" int eisen_hip_mem_info(eisen_ctx* ctx, size_t* free_bytes, size_t* total_bytes) {
    EISEN_CHECK_CTX(ctx);
    size_t f = 0, t = 0;
    EISEN_HIP_TRY(ctx, hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

extern "C" int eisen_hip_driver_allocs(eisen_ctx* ctx, size_t* count_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, count_out != nullptr, EISEN_E_ARG, "driver_allocs: count_out is null");
    *count_out = ctx->driver_allocs;
    return 0;
}

extern "C" int eisen_hip_pool_stats(eisen_ctx* ctx, size_t* in_use_bytes, size_t* cached_bytes) {
    EISEN_CHECK_CTX(ctx);
    if (in_use_bytes) *in_use_bytes = ctx->in_use_bytes;
    if (cached_bytes) *cached_bytes = ctx->cached_bytes;
    return 0;
}

int eisen_workspace(eisen_ctx* ctx, size_t bytes, void** out) {
    // one block per stream: each is allocated, used and freed in the order of its own stream
    void*& ws = ctx->side_active ? ctx->ws_side : ctx->ws;
    size_t& ws_bytes = ctx->side_active ? ctx->ws_side_bytes : ctx->ws_bytes;
    if (bytes > ws_bytes) {
        // stream order makes the old block safe to free while earlier kernels still read it
        if (ws) EISEN_HIP_TRY(ctx, hipFreeAsync(ws, ctx->stream));
        ws = nullptr;
        ws_bytes = 0;
        size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        ctx->driver_allocs++;
        hipError_t e = hipMallocAsync(&ws, want, ctx->stream);
        if (e != hipSuccess)
            return eisen_set_error(ctx, EISEN_E_NOMEM, "workspace of %zu bytes: %s", want, hipGetErrorString(e));
        ws_bytes = want;
    }
    *out = ws;
    return 0;
}

int eisen_staging(eisen_ctx* ctx, size_t bytes, eisen_ctx::StageSlot** out) {
    int tries = 0;
    while (ctx->stage[ctx->stage_next].reserved && tries < eisen_ctx::kStageSlots) {
        ctx->stage_next = (ctx->stage_next + 1) % eisen_ctx::kStageSlots;
        tries++;
    }
    EISEN_REQUIRE(ctx, tries < eisen_ctx::kStageSlots, EISEN_E_STATE, "every staging slot holds an uncollected eisen_hip_dtoh_begin result");
    eisen_ctx::StageSlot& s = ctx->stage[ctx->stage_next];
    ctx->stage_next = (ctx->stage_next + 1) % eisen_ctx::kStageSlots;
    if (!s.done) EISEN_HIP_TRY(ctx, hipEventCreateWithFlags(&s.done, hipEventDisableTiming));
    if (s.in_flight) {
        EISEN_HIP_TRY(ctx, hipEventSynchronize(s.done));
        s.in_flight = false;
    }
    if (bytes > s.bytes) {
        if (s.ptr) EISEN_HIP_TRY(ctx, hipHostFree(s.ptr));
        s.ptr = nullptr;
        s.bytes = 0;
        size_t want = (bytes + (size_t(1) << 16) - 1) & ~((size_t(1) << 16) - 1);
        ctx->driver_allocs++;
        EISEN_HIP_TRY(ctx, hipHostMalloc(&s.ptr, want, hipHostMallocDefault));
        s.bytes = want;
    }
    *out = &s;
    return 0;
}

static constexpr size_t kStageLimit = size_t(8) << 20;

extern "C" int eisen_hip_htod(eisen_ctx* ctx, void* dst, const void* src, size_t bytes) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst && src, EISEN_E_ARG, "eisen_hip_htod: null pointer");
    if (bytes == 0) return 0;
    if (bytes <= kStageLimit) {
        // small uploads (token ids, targets, tables) go through pinned staging and stay asynchronous
        eisen_ctx::StageSlot* st = nullptr;
        int rc = eisen_staging(ctx, bytes, &st);
        if (rc) return rc;
        memcpy(st->ptr, src, bytes);
        EISEN_HIP_TRY(ctx, hipMemcpyAsync(dst, st->ptr, bytes, hipMemcpyHostToDevice, ctx->stream));
        EISEN_HIP_TRY(ctx, hipEventRecord(st->done, ctx->stream));
        st->in_flight = true;
        return 0;
    }
    EISEN_HIP_TRY(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return 0;
}

extern "C" int eisen_hip_dtoh(eisen_ctx* ctx, void* dst, const void* src, size_t bytes) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst && src, EISEN_E_ARG, "eisen_hip_dtoh: null pointer");
    if (bytes == 0) return 0;
    EISEN_HIP_TRY(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return 0;
}

extern "C" int eisen_hip_dtoh_begin(eisen_ctx* ctx, const void* src, size_t bytes, int* ticket_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, src && ticket_out, EISEN_E_ARG, "eisen_hip_dtoh_begin: null pointer");
    EISEN_REQUIRE(ctx, bytes > 0 && bytes <= kStageLimit, EISEN_E_SHAPE, "eisen_hip_dtoh_begin: %zu bytes (1 .. %zu supported)", bytes, kStageLimit);
    int reserved = 0;
    for (const auto& sl : ctx->stage) reserved += sl.reserved ? 1 : 0;
    EISEN_REQUIRE(ctx, reserved < eisen_ctx::kStageSlots / 2, EISEN_E_STATE, "eisen_hip_dtoh_begin: %d copies not collected yet", reserved);
    eisen_ctx::StageSlot* st = nullptr;
    int rc = eisen_staging(ctx, bytes, &st);
    if (rc) return rc;
    EISEN_HIP_TRY(ctx, hipMemcpyAsync(st->ptr, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    EISEN_HIP_TRY(ctx, hipEventRecord(st->done, ctx->stream));
    st->in_flight = true;
    st->reserved = true;
    *ticket_out = (int)(st - ctx->stage);
    return 0;
}

extern "C" int eisen_hip_dtoh_finish(eisen_ctx* ctx, int ticket, void* dst, size_t bytes) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst != nullptr, EISEN_E_ARG, "eisen_hip_dtoh_finish: null pointer");
    EISEN_REQUIRE(ctx, ticket >= 0 && ticket < eisen_ctx::kStageSlots && ctx->stage[ticket].reserved, EISEN_E_STATE,
                  "eisen_hip_dtoh_finish: ticket %d names no pending copy", ticket);
    eisen_ctx::StageSlot& s = ctx->stage[ticket];
    EISEN_REQUIRE(ctx, bytes <= s.bytes, EISEN_E_ARG, "eisen_hip_dtoh_finish: %zu bytes asked of a %zu-byte slot", bytes, s.bytes);
    s.reserved = false;
    EISEN_HIP_TRY(ctx, hipEventSynchronize(s.done));  // waits for this copy only: later work stays queued
    s.in_flight = false;
    memcpy(dst, s.ptr, bytes);
    return 0;
}

extern "C" int eisen_hip_dtod(eisen_ctx* ctx, void* dst, const void* src, size_t bytes) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst && src, EISEN_E_ARG, "eisen_hip_dtod: null pointer");
    if (bytes == 0) return 0;
    EISEN_HIP_TRY(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return 0;
}

extern "C" int eisen_hip_memset_zero(eisen_ctx* ctx, void* dst, size_t bytes) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst != nullptr, EISEN_E_ARG, "eisen_hip_memset_zero: null pointer");
    if (bytes == 0) return 0;
    // a fill kernel, not hipMemsetAsync: a memset node recorded into a captured graph has replayed wrongly on this
    // hardware generation, and callers may capture the step
    if (bytes % 4 == 0 && eisen_aligned(dst, 4)) return eisen_hip_fill(ctx, dst, EISEN_F32, 0.0f, bytes / 4);
    EISEN_HIP_TRY(ctx, hipMemsetAsync(dst, 0, bytes, ctx->stream));
    return 0;
}

extern "C" int eisen_hip_module_load(eisen_ctx* ctx, const void* image, size_t len, eisen_module** out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, image && len && out, EISEN_E_ARG, "eisen_hip_module_load: null image or out");
    hipModule_t mod;
    EISEN_HIP_TRY(ctx, hipModuleLoadData(&mod, image));
    *out = new eisen_module{mod};
    return 0;
}

extern "C" int eisen_hip_module_unload(eisen_ctx* ctx, eisen_module* mod) {
    EISEN_CHECK_CTX(ctx);
    if (!mod) return 0;
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    EISEN_HIP_TRY(ctx, hipModuleUnload(mod->mod));
    delete mod;
    return 0;
}

extern "C" int eisen_hip_get_function(eisen_ctx* ctx, eisen_module* mod, const char* name, eisen_function** out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, mod && name && out, EISEN_E_ARG, "eisen_hip_get_function: null argument");
    hipFunction_t fn;
    hipError_t e = hipModuleGetFunction(&fn, mod->mod, name);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return eisen_set_error(ctx, (int)e, "kernel '%s' not found in module: %s", name, hipGetErrorString(e));
    }
    *out = new eisen_function{fn};  // lives as long as the process; a handful per module
    return 0;
}

extern "C" int eisen_hip_launch(eisen_ctx* ctx, eisen_function* fn, const unsigned grid[3], const unsigned block[3],
                                unsigned shared_bytes, void** args) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, fn && grid && block, EISEN_E_ARG, "eisen_hip_launch: null argument");
    EISEN_REQUIRE(ctx, grid[0] && grid[1] && grid[2] && block[0] && block[1] && block[2], EISEN_E_ARG,
                  "eisen_hip_launch: zero grid or block dimension");
    EISEN_REQUIRE(ctx, (size_t)block[0] * block[1] * block[2] <= 1024, EISEN_E_SHAPE,
                  "eisen_hip_launch: more than 1024 threads per block");
    EISEN_HIP_TRY(ctx, hipModuleLaunchKernel(fn->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                             shared_bytes, ctx->stream, args, nullptr));
    return 0;
}

extern "C" int eisen_hip_timer_start(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    EISEN_HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
    ctx->timer_running = true;
    return 0;
}

extern "C" int eisen_hip_timer_stop(eisen_ctx* ctx, float* ms_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ctx->timer_running, EISEN_E_STATE, "eisen_hip_timer_stop without eisen_hip_timer_start");
    EISEN_HIP_TRY(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
    EISEN_HIP_TRY(ctx, hipEventSynchronize(ctx->ev_stop));
    float ms = 0.f;
    EISEN_HIP_TRY(ctx, hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop));
    ctx->timer_running = false;
    if (ms_out) *ms_out = ms;
    return 0;
}

// ---- per-kernel timing ----------------------------------------------------------------------------

int eisen_prof_begin(eisen_ctx* ctx, const char* name, double work, bool is_flops) {
    eisen_prof& p = ctx->prof;
    int key = -1;
    for (size_t i = 0; i < p.names.size(); i++)
        if (p.names[i] == name) key = (int)i;
    if (key < 0) {
        p.names.push_back(name);
        p.is_flops.push_back(is_flops ? 1 : 0);
        key = (int)p.names.size() - 1;
    }
    while (p.pool.size() < p.pool_used + 2) {
        hipEvent_t e;
        if (hipEventCreate(&e) != hipSuccess) return -1;
        p.pool.push_back(e);
    }
    eisen_prof_rec r{key, p.pool[p.pool_used], p.pool[p.pool_used + 1], work};
    p.pool_used += 2;
    if (hipEventRecord(r.start, ctx->stream) != hipSuccess) return -1;
    p.recs.push_back(r);
    return (int)p.recs.size() - 1;
}
void eisen_prof_end(eisen_ctx* ctx, int rec) { (void)hipEventRecord(ctx->prof.recs[rec].stop, ctx->stream); }

extern "C" int eisen_hip_profile_start(eisen_ctx* ctx) {
    EISEN_CHECK_CTX(ctx);
    ctx->prof.enabled = true;
    ctx->prof.recs.clear();
    ctx->prof.pool_used = 0;
    return 0;
}

extern "C" int eisen_hip_profile_stop(eisen_ctx* ctx, eisen_prof_entry* out, size_t capacity, size_t* count_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, count_out != nullptr, EISEN_E_ARG, "eisen_hip_profile_stop: null count_out");
    eisen_prof& p = ctx->prof;
    p.enabled = false;
    // instrumented launches may sit on either stream: both have to be done before their events are read
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->side_stream));
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->main_stream));
    std::vector<eisen_prof_entry> acc(p.names.size());
    for (size_t i = 0; i < p.names.size(); i++) {
        std::memset(&acc[i], 0, sizeof(eisen_prof_entry));
        std::strncpy(acc[i].name, p.names[i].c_str(), sizeof(acc[i].name) - 1);
        acc[i].work_is_flops = p.is_flops[i];
    }
    for (const eisen_prof_rec& r : p.recs) {
        float ms = 0.f;
        EISEN_HIP_TRY(ctx, hipEventElapsedTime(&ms, r.start, r.stop));
        acc[r.key].ms += ms;
        acc[r.key].work += r.work;
        acc[r.key].launches += 1;
    }
    size_t n = 0;
    for (const eisen_prof_entry& e : acc)
        if (e.launches) {
            if (out && n < capacity) out[n] = e;
            n++;
        }
    *count_out = n;
    p.recs.clear();
    p.pool_used = 0;
    return 0;
}
