// exhip runtime: context, memory, events. Everything runs on one stream per context.
#include <stdarg.h>
#include <string.h>

#include <algorithm>

#include "common.h"

static thread_local char g_err[512] = "";

void exhip_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char* exhip_last_error(void) { return g_err; }

exhip_options g_exhip_options;

extern "C" int exhip_set_option(const char* name, int value) {
    EXHIP_REQUIRE(name, "exhip_set_option: NULL name");
    exhip_options& o = g_exhip_options;
    if (!strcmp(name, "force_variant")) o.force_variant = value;
    else if (!strcmp(name, "force_chunk")) o.force_chunk = value;
    else if (!strcmp(name, "force_rs")) o.force_rs = value;
    else if (!strcmp(name, "force_abufs")) o.force_abufs = value;
    else if (!strcmp(name, "debug_plan")) o.debug_plan = value;
    else if (!strcmp(name, "dw_band_rows")) o.dw_band_rows = value;
    else if (!strcmp(name, "force_splits")) o.force_splits = value;
    else if (!strcmp(name, "share_gpu")) o.share_gpu = value;
    else if (!strcmp(name, "lean")) o.lean = value;
    else if (!strcmp(name, "lean_cfg")) o.lean_cfg = value;
    else if (!strcmp(name, "pw")) o.pw = value;
    else if (!strcmp(name, "direct")) o.direct = value;
    else if (!strcmp(name, "pw_tile")) o.pw_tile = value;
    else if (!strcmp(name, "lean_f16")) o.lean_f16 = value;
    else if (!strcmp(name, "lean_groups")) o.lean_groups = value;
    else if (!strcmp(name, "lean_wres")) o.lean_wres = value;
    else if (!strcmp(name, "stem")) o.stem = value;
    else if (!strcmp(name, "lean_stagger")) o.lean_stagger = value;
    else {
        exhip_set_error("exhip_set_option: unknown option %s", name);
        return EXHIP_ERR_ARG;
    }
    return 0;
}

extern "C" int exhip_init(int device, exhip_ctx** out) {
    EXHIP_REQUIRE(out != nullptr, "exhip_init: ctx is NULL");
    int count = 0;
    EXHIP_CHECK(hipGetDeviceCount(&count));
    EXHIP_REQUIRE(device >= 0 && device < count, "exhip_init: device %d out of range (have %d)", device, count);
    EXHIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    EXHIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        exhip_set_error("exhip_init: device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
        return EXHIP_ERR_UNSUPPORTED;
    }
    const int rc = exhip_static_scratch_setup(device);
    if (rc != 0) return rc;
    exhip_ctx* c = new exhip_ctx();
    c->device = device;
    hipError_t e = hipStreamCreate(&c->stream);  // default priority
    if (e != hipSuccess) {
        delete c;
        exhip_set_error("hipStreamCreate failed: %s", hipGetErrorString(e));
        return (int)e;
    }
    *out = c;
    return 0;
}

extern "C" int exhip_destroy(exhip_ctx* ctx) {
    if (!ctx) return 0;
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->split_acc) (void)hipFree(ctx->split_acc);
    if (ctx->split_count) (void)hipFree(ctx->split_count);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return 0;
}

extern "C" int exhip_malloc(exhip_ctx* ctx, size_t bytes, void** dptr) {
    EXHIP_REQUIRE(ctx && dptr, "exhip_malloc: NULL argument");
    const hipError_t e = hipMalloc(dptr, bytes ? bytes : 1);
    if (e != hipSuccess) {
        // the runtime keeps a failed call's code as the thread's last error, where the next launch check would find it: a
        // caller that recovers (frees blocks, asks again) must not be failed by it later
        (void)hipGetLastError();
        exhip_set_error("hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
        return (int)e;
    }
    return 0;
}

extern "C" int exhip_free(exhip_ctx* ctx, void* dptr) {
    EXHIP_REQUIRE(ctx, "exhip_free: NULL ctx");
    if (dptr) {
        EXHIP_CHECK(hipStreamSynchronize(ctx->stream));
        EXHIP_CHECK(hipFree(dptr));
    }
    return 0;
}

extern "C" int exhip_memset(exhip_ctx* ctx, void* dptr, int value, size_t bytes) {
    EXHIP_REQUIRE(ctx && (dptr || !bytes), "exhip_memset: NULL argument");
    if (bytes) EXHIP_CHECK(hipMemsetAsync(dptr, value, bytes, ctx->stream));
    return 0;
}

extern "C" int exhip_memcpy_h2d(exhip_ctx* ctx, void* dst, const void* src, size_t bytes) {
    EXHIP_REQUIRE(ctx && ((dst && src) || !bytes), "exhip_memcpy_h2d: NULL argument");
    if (bytes) {
        EXHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
        EXHIP_CHECK(hipStreamSynchronize(ctx->stream));  // src may be pageable and reused by the caller
    }
    return 0;
}

extern "C" int exhip_memcpy_d2h(exhip_ctx* ctx, void* dst, const void* src, size_t bytes) {
    EXHIP_REQUIRE(ctx && ((dst && src) || !bytes), "exhip_memcpy_d2h: NULL argument");
    if (bytes) {
        EXHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
        EXHIP_CHECK(hipStreamSynchronize(ctx->stream));
    }
    return 0;
}

extern "C" int exhip_memcpy_d2d(exhip_ctx* ctx, void* dst, const void* src, size_t bytes) {
    EXHIP_REQUIRE(ctx && ((dst && src) || !bytes), "exhip_memcpy_d2d: NULL argument");
    if (bytes) EXHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return 0;
}

extern "C" int exhip_sync(exhip_ctx* ctx) {
    EXHIP_REQUIRE(ctx, "exhip_sync: NULL ctx");
    EXHIP_CHECK(hipStreamSynchronize(ctx->stream));
    return 0;
}

extern "C" int exhip_device_name(exhip_ctx* ctx, char* buf, size_t len) {
    EXHIP_REQUIRE(ctx && buf && len, "exhip_device_name: NULL argument");
    hipDeviceProp_t prop;
    EXHIP_CHECK(hipGetDeviceProperties(&prop, ctx->device));
    snprintf(buf, len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return 0;
}

extern "C" int exhip_event_create(void** ev) {
    EXHIP_REQUIRE(ev, "exhip_event_create: NULL argument");
    hipEvent_t e;
    EXHIP_CHECK(hipEventCreate(&e));
    *ev = (void*)e;
    return 0;
}

extern "C" int exhip_event_destroy(void* ev) {
    if (ev) EXHIP_CHECK(hipEventDestroy((hipEvent_t)ev));
    return 0;
}

extern "C" int exhip_event_record(exhip_ctx* ctx, void* ev) {
    EXHIP_REQUIRE(ctx && ev, "exhip_event_record: NULL argument");
    EXHIP_CHECK(hipEventRecord((hipEvent_t)ev, ctx->stream));
    return 0;
}

extern "C" int exhip_event_elapsed_ms(void* ev_start, void* ev_stop, float* ms) {
    EXHIP_REQUIRE(ev_start && ev_stop && ms, "exhip_event_elapsed_ms: NULL argument");
    EXHIP_CHECK(hipEventSynchronize((hipEvent_t)ev_stop));
    EXHIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)ev_start, (hipEvent_t)ev_stop));
    return 0;
}

// ---- stream capture: a fixed sequence of launches recorded once and replayed as one graph ----
extern "C" int exhip_graph_begin(exhip_ctx* ctx) {
    EXHIP_REQUIRE(ctx, "exhip_graph_begin: NULL ctx");
    EXHIP_CHECK(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    return 0;
}

extern "C" int exhip_graph_end(exhip_ctx* ctx, void** graph_exec) {
    EXHIP_REQUIRE(ctx && graph_exec, "exhip_graph_end: NULL argument");
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    EXHIP_CHECK(hipStreamEndCapture(ctx->stream, &graph));
    EXHIP_REQUIRE(graph != nullptr, "exhip_graph_end: the capture recorded nothing");
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        exhip_set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return (int)e;
    }
    *graph_exec = (void*)exec;
    return 0;
}

extern "C" int exhip_graph_launch(exhip_ctx* ctx, void* graph_exec) {
    EXHIP_REQUIRE(ctx && graph_exec, "exhip_graph_launch: NULL argument");
    EXHIP_CHECK(hipGraphLaunch((hipGraphExec_t)graph_exec, ctx->stream));
    return 0;
}

extern "C" int exhip_graph_destroy(void* graph_exec) {
    if (graph_exec) EXHIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return 0;
}

// The scratch never moves once it exists: a recorded HIP graph keeps its address in kernel nodes, so it is allocated once per
// context at its upper bound (the planner splits a launch into at most kSplitGroups groups of at most 512 threads, 256 bytes
// of accumulators per thread) together with one arrival counter per possible tile.
int exhip_split_scratch(exhip_ctx* ctx, size_t acc_bytes, size_t tiles, int** acc, unsigned** count) {
    constexpr size_t kAccBytes = (size_t)kSplitGroups * 512 * 256, kCounters = kSplitGroups;
    EXHIP_REQUIRE(acc_bytes <= kAccBytes && tiles <= kCounters, "split reduction: %zu bytes for %zu tiles exceed the scratch's fixed size", acc_bytes,
                  tiles);
    if (!ctx->split_acc) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        EXHIP_CHECK(hipStreamIsCapturing(ctx->stream, &capturing));
        EXHIP_REQUIRE(capturing == hipStreamCaptureStatusNone,
                      "split reduction: its scratch cannot be allocated while the stream records a graph; run the launch once before recording");
        EXHIP_CHECK(hipMalloc(reinterpret_cast<void**>(&ctx->split_acc), kAccBytes));
        ctx->split_acc_bytes = kAccBytes;
        hipError_t e = hipMalloc(reinterpret_cast<void**>(&ctx->split_count), kCounters * sizeof(unsigned));
        if (e == hipSuccess) e = hipMemset(ctx->split_count, 0, kCounters * sizeof(unsigned));  // every launch leaves its counters at zero
        if (e != hipSuccess) {
            (void)hipFree(ctx->split_acc);
            if (ctx->split_count) (void)hipFree(ctx->split_count);
            ctx->split_acc = nullptr;
            ctx->split_count = nullptr;
            exhip_set_error("split reduction: allocating the arrival counters failed: %s", hipGetErrorString(e));
            return (int)e;
        }
        ctx->split_count_n = kCounters;
    }
    *acc = ctx->split_acc;
    *count = ctx->split_count;
    return 0;
}
