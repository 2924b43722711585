// Context, status and device-memory entry points of libperegrine_hip.
#include <stdarg.h>
#include <stdio.h>
#include <new>
#include "pg_internal.h"

static thread_local char g_err[512] = "";

pg_status pg_fail(pg_status st, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return st;
}

PG_API const char *pg_last_error(void) { return g_err; }

PG_API const char *pg_status_string(pg_status st) {
    switch (st) {
        case PG_OK: return "ok";
        case PG_EINVAL: return "invalid argument";
        case PG_EDEVICE: return "device error";
        case PG_ENOMEM: return "out of memory";
        case PG_EUNSUPPORTED: return "unsupported";
        default: return "unknown status";
    }
}

pg_status pg_use(pg_ctx *ctx) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    PG_HIP(hipSetDevice(ctx->device));
    return PG_OK;
}

pg_status pg_launch_check(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return pg_fail(PG_EDEVICE, "launch of %s failed: %s", what, hipGetErrorString(e));
    return PG_OK;
}

pg_status pg_allow_dynamic_lds(pg_ctx *ctx, const void *kernel, size_t bytes) {
    // (the limit only ever grows: a kernel launched with more than an earlier call asked for is raised again)
    std::pair<const void *, size_t> *slot = nullptr;
    for (auto &k : ctx->lds_raised)
        if (k.first == kernel) {
            if (k.second >= bytes) return PG_OK;
            slot = &k;
        }
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return pg_fail(PG_EDEVICE, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    if (slot) slot->second = bytes;
    else ctx->lds_raised.emplace_back(kernel, bytes);
    return PG_OK;
}

pg_status pg_workspace(pg_ctx *ctx, size_t bytes, void **out) {
    if (bytes > ctx->ws_bytes) {
        // Work already queued may still use the old arena: drain before replacing it.
        PG_HIP(hipStreamSynchronize(ctx->stream));
        if (ctx->ws) PG_HIP(hipFree(ctx->ws));
        ctx->ws = nullptr;
        ctx->ws_bytes = 0;
        size_t want = pg_round_up(bytes + bytes / 4, 1 << 20);
        PG_HIP(hipMalloc(&ctx->ws, want));
        ctx->ws_bytes = want;
    }
    *out = ctx->ws;
    return PG_OK;
}

PG_API pg_status pg_ctx_create(int device, void *hip_stream, pg_ctx **out) {
    PG_CHECK_ARG(out != nullptr, "pg_ctx_create: out is null");
    *out = nullptr;
    int count = 0;
    PG_HIP(hipGetDeviceCount(&count));
    PG_CHECK_ARG(device >= 0 && device < count, "pg_ctx_create: device %d of %d", device, count);
    PG_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    PG_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return pg_fail(PG_EUNSUPPORTED, "device %d is %s; this library holds gfx950 code only",
                       device, prop.gcnArchName);
    pg_ctx *ctx = new (std::nothrow) pg_ctx();
    if (!ctx) return pg_fail(PG_ENOMEM, "pg_ctx_create: host allocation failed");
    ctx->device = device;
    ctx->ws = nullptr;
    ctx->ws_bytes = 0;
    ctx->num_cu = prop.multiProcessorCount;
    ctx->profiling = false;
    ctx->lds_raised.reserve(256);  // so that noting a kernel's raised LDS limit never allocates later
    if (hip_stream) {
        ctx->stream = static_cast<hipStream_t>(hip_stream);
        ctx->owns_stream = false;
    } else {
        hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            delete ctx;
            return pg_fail(PG_EDEVICE, "hipStreamCreate failed: %s", hipGetErrorString(e));
        }
        ctx->owns_stream = true;
    }
    *out = ctx;
    return PG_OK;
}

static void prof_drop(pg_ctx *ctx);

PG_API void pg_ctx_destroy(pg_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->ws) (void)hipFree(ctx->ws);
    for (auto &t : ctx->moe_tabs)
        if (t.dev) (void)hipFree(t.dev);
    prof_drop(ctx);
    if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

PG_API pg_status pg_sync(pg_ctx *ctx) {
    PG_TRY(pg_use(ctx));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API void *pg_ctx_stream(pg_ctx *ctx) { return ctx ? static_cast<void *>(ctx->stream) : nullptr; }

PG_API pg_status pg_dev_alloc(pg_ctx *ctx, size_t bytes, void **dptr) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(dptr != nullptr, "pg_dev_alloc: dptr is null");
    PG_HIP(hipMalloc(dptr, bytes ? bytes : 1));
    return PG_OK;
}

PG_API pg_status pg_dev_free(pg_ctx *ctx, void *dptr) {
    PG_TRY(pg_use(ctx));
    if (!dptr) return PG_OK;
    PG_HIP(hipStreamSynchronize(ctx->stream));
    PG_HIP(hipFree(dptr));
    return PG_OK;
}

PG_API pg_status pg_memcpy_h2d(pg_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    PG_TRY(pg_use(ctx));
    if (!bytes) return PG_OK;
    PG_CHECK_ARG(dst_dev && src_host, "pg_memcpy_h2d: null pointer");
    PG_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_memcpy_d2h(pg_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    PG_TRY(pg_use(ctx));
    if (!bytes) return PG_OK;
    PG_CHECK_ARG(dst_host && src_dev, "pg_memcpy_d2h: null pointer");
    PG_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// ---- per-kernel timing with HIP events ------------------------------------------

static void prof_drop(pg_ctx *ctx) {
    for (auto &r : ctx->prof) {
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    ctx->prof.clear();
}

PG_API pg_status pg_profile_begin(pg_ctx *ctx) {
    PG_TRY(pg_use(ctx));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    prof_drop(ctx);
    ctx->totals.clear();
    ctx->profiling = true;
    return PG_OK;
}

PG_API pg_status pg_profile_end(pg_ctx *ctx, size_t *num_kernels) {
    PG_TRY(pg_use(ctx));
    ctx->profiling = false;
    PG_HIP(hipStreamSynchronize(ctx->stream));
    ctx->totals.clear();
    for (auto &r : ctx->prof) {
        float ms = 0.0f;
        const hipError_t ee = hipEventElapsedTime(&ms, r.start, r.stop);
        if (ee != hipSuccess) { (void)pg_fail(PG_EDEVICE, "hipEventElapsedTime(%s): %s", r.name, hipGetErrorString(ee)); continue; }
        pg_prof_total *t = nullptr;
        for (auto &x : ctx->totals)
            if (x.name == r.name) t = &x;
        if (!t) {
            ctx->totals.push_back({r.name, 0.0, 0, {}});
            t = &ctx->totals.back();
        }
        t->total_ms += ms;
        t->launches += 1;
        bool seen = false;
        for (auto &g : t->grids)
            if (g.first == r.threads) { g.second += 1; seen = true; }
        if (!seen) t->grids.push_back({r.threads, 1});
    }
    prof_drop(ctx);
    if (num_kernels) *num_kernels = ctx->totals.size();
    return PG_OK;
}

PG_API pg_status pg_profile_get(pg_ctx *ctx, size_t i, const char **name, double *total_ms,
                                size_t *launches) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    PG_CHECK_ARG(i < ctx->totals.size(), "pg_profile_get: index %zu of %zu", i, ctx->totals.size());
    if (name) *name = ctx->totals[i].name.c_str();
    if (total_ms) *total_ms = ctx->totals[i].total_ms;
    if (launches) *launches = ctx->totals[i].launches;
    return PG_OK;
}

PG_API pg_status pg_profile_get_grids(pg_ctx *ctx, size_t i, size_t *work_items, size_t *launches, size_t cap, size_t *count) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    PG_CHECK_ARG(i < ctx->totals.size(), "pg_profile_get_grids: index %zu of %zu", i, ctx->totals.size());
    const auto &g = ctx->totals[i].grids;
    if (count) *count = g.size();
    for (size_t j = 0; j < g.size() && j < cap; ++j) {
        if (work_items) work_items[j] = g[j].first;
        if (launches) launches[j] = g[j].second;
    }
    return PG_OK;
}
