// Device / stream / buffer layer of libgalois_hip (replaces what src/cuda.rs:35-308
// obtains from cudarc).  One context = one device ordinal + one stream.
#include "common.h"


// Called once the stream has drained.  A kernel whose bounded wait for other workgroups of its launch ran out has
// set the context's status word (and poisoned its own result with NaN); the workgroups it gave up on may have counted
// themselves after the counters were returned to zero, so the counters are cleared here before anything else runs.
int32_t gh_check_device_status(galois_hip_ctx *ctx) {
    if (!ctx->dev_status || __atomic_load_n(ctx->dev_status, __ATOMIC_ACQUIRE) == 0) return GALOIS_HIP_OK;
    __atomic_store_n(ctx->dev_status, 0u, __ATOMIC_RELEASE);
    hipError_t e = hipMemsetAsync(ctx->attn_done, 0, 4 * GH_ATTN_HEADS * sizeof(unsigned), ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return gh_hip(ctx, e, "clearing the wait counters");
    return gh_fail(ctx, GALOIS_HIP_E_DEVICE_WAIT,
                   "qkv_attn_decode: a workgroup gave up waiting for the products of its launch; the attention output of "
                   "that call is NaN and what was launched after it on this context is not to be trusted (the counters "
                   "have been cleared: the context can be used again)");
}

extern "C" {

const char *galois_hip_status_string(int32_t s) {
    switch (s) {
        case GALOIS_HIP_OK: return "ok";
        case GALOIS_HIP_E_NULL: return "null pointer argument";
        case GALOIS_HIP_E_SHAPE: return "bad shape argument";
        case GALOIS_HIP_E_ALIGN: return "misaligned device pointer";
        case GALOIS_HIP_E_ORDINAL: return "no such device";
        case GALOIS_HIP_E_UNSUPPORTED: return "unsupported combination";
        case GALOIS_HIP_E_ARCH: return "device is not gfx950";
        case GALOIS_HIP_E_DEVICE_WAIT: return "a bounded wait inside a launch ran out";
        default: return s > 0 ? hipGetErrorString((hipError_t)s) : "unknown status";
    }
}

int32_t galois_hip_create(int32_t ordinal, galois_hip_ctx **out) {
    if (!out) return GALOIS_HIP_E_NULL;
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return (int32_t)e;
    if (ordinal < 0 || ordinal >= n) return GALOIS_HIP_E_ORDINAL;
    e = hipSetDevice(ordinal);
    if (e != hipSuccess) return (int32_t)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, ordinal);
    if (e != hipSuccess) return (int32_t)e;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return GALOIS_HIP_E_ARCH;
    galois_hip_ctx *ctx = new galois_hip_ctx();
    ctx->ordinal = ordinal;
    ctx->n_cu = prop.multiProcessorCount;
    ctx->last_error[0] = 0;
    ctx->ws = nullptr;
    ctx->ws_bytes = 0;
    ctx->scratch = nullptr;
    ctx->attn_done = nullptr;
    ctx->attn_static = nullptr;
    ctx->capturing = false;
    ctx->dev_status = nullptr;
    ctx->dev_status_dev = nullptr;
    ctx->wait_spin_limit = GH_WAIT_SPIN_DEFAULT;
    ctx->wait_target_bias = 0;
    ctx->gemv_f32 = false;
    e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete ctx;
        return (int32_t)e;
    }
    const size_t scratch_bytes = GH_PARTIAL_FLOATS * sizeof(float);
    e = hipMalloc(&ctx->scratch, scratch_bytes);
    if (e == hipSuccess) e = hipMemsetAsync(ctx->scratch, 0, scratch_bytes, ctx->stream);
    if (e == hipSuccess) e = hipMalloc((void **)&ctx->attn_done, 4 * GH_ATTN_HEADS * sizeof(unsigned));
    if (e == hipSuccess) e = hipMemsetAsync(ctx->attn_done, 0, 4 * GH_ATTN_HEADS * sizeof(unsigned), ctx->stream);
    // the status word lives in pinned host memory that the device writes directly: reading it costs the host nothing
    if (e == hipSuccess) e = hipHostMalloc((void **)&ctx->dev_status, 64, hipHostMallocMapped);
    if (e == hipSuccess) {
        *ctx->dev_status = 0;
        e = hipHostGetDevicePointer((void **)&ctx->dev_status_dev, ctx->dev_status, 0);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    // only galois_hip_attn_decode_f32_static needs the static scratch; without it that entry point refuses by itself
    if (e == hipSuccess) (void)gh_attn_static_init(ctx);
    if (e != hipSuccess) {
        if (ctx->scratch) (void)hipFree(ctx->scratch);
        if (ctx->attn_done) (void)hipFree(ctx->attn_done);
        if (ctx->dev_status) (void)hipHostFree(ctx->dev_status);
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return (int32_t)e;
    }
    *out = ctx;
    return GALOIS_HIP_OK;
}

int32_t galois_hip_destroy(galois_hip_ctx *ctx) {
    GH_REQUIRE_CTX(ctx);
    (void)hipSetDevice(ctx->ordinal);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->ws) (void)hipFree(ctx->ws);
    for (void *p : ctx->ws_retired) (void)hipFree(p);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    if (ctx->attn_done) (void)hipFree(ctx->attn_done);
    if (ctx->dev_status) (void)hipHostFree(ctx->dev_status);
    hipError_t e = hipStreamDestroy(ctx->stream);
    delete ctx;
    return (int32_t)e;
}

int32_t galois_hip_abi_version(void) { return GALOIS_HIP_ABI_VERSION; }

int32_t galois_hip_set_option(galois_hip_ctx *ctx, int32_t option, int32_t value) {
    GH_REQUIRE_CTX(ctx);
    switch (option) {
        case GALOIS_HIP_OPT_GEMV_F32_ARITHMETIC:
            ctx->gemv_f32 = value != 0;
            return GALOIS_HIP_OK;
        case GALOIS_HIP_OPT_WAIT_SPIN_LIMIT:
            GH_REQUIRE(ctx, value >= 0, GALOIS_HIP_E_SHAPE, "set_option: the poll limit is 0 (the default) or positive");
            ctx->wait_spin_limit = value > 0 ? value : GH_WAIT_SPIN_DEFAULT;
            return GALOIS_HIP_OK;
        case GALOIS_HIP_OPT_WAIT_TARGET_BIAS:
            GH_REQUIRE(ctx, value >= 0 && value <= 1, GALOIS_HIP_E_SHAPE, "set_option: the target bias is 0 or 1");
            ctx->wait_target_bias = value;
            return GALOIS_HIP_OK;
        default:
            return gh_fail(ctx, GALOIS_HIP_E_UNSUPPORTED, "set_option: unknown option");
    }
}

int32_t galois_hip_init_functions(galois_hip_ctx *ctx, int32_t abi_version, int32_t *n_kernels) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, abi_version == GALOIS_HIP_ABI_VERSION, GALOIS_HIP_E_UNSUPPORTED, "init_functions: ABI version");
    if (n_kernels) *n_kernels = 16;  // the reference registers 16 kernel names (src/kernels.rs:5-20)
    return GALOIS_HIP_OK;
}

const char *galois_hip_last_error(const galois_hip_ctx *ctx) { return ctx ? ctx->last_error : ""; }

int32_t galois_hip_device_info(galois_hip_ctx *ctx, char *name, int32_t name_cap, char *arch, int32_t arch_cap,
                               int32_t *n_cu, int32_t *clock_khz, int32_t *mem_clock_khz, int64_t *mem_bytes) {
    GH_REQUIRE_CTX(ctx);
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, ctx->ordinal);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipGetDeviceProperties");
    if (name && name_cap > 0) snprintf(name, (size_t)name_cap, "%s", prop.name);
    if (arch && arch_cap > 0) snprintf(arch, (size_t)arch_cap, "%s", prop.gcnArchName);
    if (n_cu) *n_cu = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (mem_clock_khz) *mem_clock_khz = prop.memoryClockRate;
    if (mem_bytes) *mem_bytes = (int64_t)prop.totalGlobalMem;
    return GALOIS_HIP_OK;
}

int32_t galois_hip_alloc_zeros(galois_hip_ctx *ctx, size_t bytes, void **out) {
    GH_REQUIRE_CTX(ctx);
    GH_NOT_CAPTURING(ctx, "alloc_zeros");
    GH_REQUIRE(ctx, out != nullptr, GALOIS_HIP_E_NULL, "alloc_zeros: out");
    *out = nullptr;
    GH_BIND(ctx);
    if (bytes == 0) return GALOIS_HIP_OK;  // empty slice: NULL pointer, like an empty CudaSlice
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipMalloc");
    e = hipMemsetAsync(p, 0, bytes, ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(p);
        return gh_hip(ctx, e, "hipMemsetAsync");
    }
    *out = p;
    return GALOIS_HIP_OK;
}

int32_t galois_hip_free(galois_hip_ctx *ctx, void *dptr) {
    GH_REQUIRE_CTX(ctx);
    GH_NOT_CAPTURING(ctx, "free");
    if (!dptr) return GALOIS_HIP_OK;
    GH_BIND(ctx);
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipStreamSynchronize");
    return gh_hip(ctx, hipFree(dptr), "hipFree");
}

int32_t galois_hip_htod_sync_copy(galois_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    GH_REQUIRE_CTX(ctx);
    GH_NOT_CAPTURING(ctx, "htod_sync_copy");
    if (bytes == 0) return GALOIS_HIP_OK;
    GH_REQUIRE(ctx, dst_dev && src_host, GALOIS_HIP_E_NULL, "htod_sync_copy");
    GH_BIND(ctx);
    hipError_t e = hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipMemcpyAsync(H2D)");
    return gh_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

int32_t galois_hip_dtoh_sync_copy(galois_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    GH_REQUIRE_CTX(ctx);
    GH_NOT_CAPTURING(ctx, "dtoh_sync_copy");
    if (bytes == 0) return GALOIS_HIP_OK;
    GH_REQUIRE(ctx, dst_host && src_dev, GALOIS_HIP_E_NULL, "dtoh_sync_copy");
    GH_BIND(ctx);
    hipError_t e = hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipMemcpyAsync(D2H)");
    e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipStreamSynchronize");
    return gh_check_device_status(ctx);
}

int32_t galois_hip_dtod_copy(galois_hip_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes) {
    GH_REQUIRE_CTX(ctx);
    if (bytes == 0) return GALOIS_HIP_OK;
    GH_REQUIRE(ctx, dst_dev && src_dev, GALOIS_HIP_E_NULL, "dtod_copy");
    GH_BIND(ctx);
    return gh_hip(ctx, hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream),
                  "hipMemcpyAsync(D2D)");
}

int32_t galois_hip_dtod_copy_2d(galois_hip_ctx *ctx, void *dst_dev, size_t dpitch, const void *src_dev,
                                size_t spitch, size_t width_bytes, size_t height) {
    GH_REQUIRE_CTX(ctx);
    if (width_bytes == 0 || height == 0) return GALOIS_HIP_OK;
    GH_REQUIRE(ctx, dst_dev && src_dev, GALOIS_HIP_E_NULL, "dtod_copy_2d");
    GH_REQUIRE(ctx, dpitch >= width_bytes && spitch >= width_bytes, GALOIS_HIP_E_SHAPE, "dtod_copy_2d: pitch < width");
    GH_BIND(ctx);
    return gh_hip(ctx,
                  hipMemcpy2DAsync(dst_dev, dpitch, src_dev, spitch, width_bytes, height, hipMemcpyDeviceToDevice,
                                   ctx->stream),
                  "hipMemcpy2DAsync(D2D)");
}

int32_t galois_hip_synchronize(galois_hip_ctx *ctx) {
    GH_REQUIRE_CTX(ctx);
    GH_NOT_CAPTURING(ctx, "synchronize");
    GH_BIND(ctx);
    const hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipStreamSynchronize");
    return gh_check_device_status(ctx);
}

int32_t galois_hip_event_create(galois_hip_ctx *ctx, galois_hip_event **out) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, out != nullptr, GALOIS_HIP_E_NULL, "event_create: out");
    GH_BIND(ctx);
    galois_hip_event *ev = new galois_hip_event();
    hipError_t e = hipEventCreate(&ev->ev);
    if (e != hipSuccess) {
        delete ev;
        *out = nullptr;
        return gh_hip(ctx, e, "hipEventCreate");
    }
    *out = ev;
    return GALOIS_HIP_OK;
}

int32_t galois_hip_event_record(galois_hip_ctx *ctx, galois_hip_event *ev) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, ev != nullptr, GALOIS_HIP_E_NULL, "event_record");
    GH_BIND(ctx);
    return gh_hip(ctx, hipEventRecord(ev->ev, ctx->stream), "hipEventRecord");
}

int32_t galois_hip_event_elapsed_ms(galois_hip_ctx *ctx, galois_hip_event *start, galois_hip_event *stop, float *ms) {
    GH_REQUIRE_CTX(ctx);
    GH_NOT_CAPTURING(ctx, "event_elapsed_ms");
    GH_REQUIRE(ctx, start && stop && ms, GALOIS_HIP_E_NULL, "event_elapsed_ms");
    GH_BIND(ctx);
    hipError_t e = hipEventSynchronize(stop->ev);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipEventSynchronize");
    return gh_hip(ctx, hipEventElapsedTime(ms, start->ev, stop->ev), "hipEventElapsedTime");
}

int32_t galois_hip_event_destroy(galois_hip_ctx *ctx, galois_hip_event *ev) {
    GH_REQUIRE_CTX(ctx);
    if (!ev) return GALOIS_HIP_OK;
    GH_BIND(ctx);
    hipError_t e = hipEventDestroy(ev->ev);
    delete ev;
    return gh_hip(ctx, e, "hipEventDestroy");
}

// ---- stream capture: a launch-bound op sequence recorded once and replayed as one HIP graph ----

int32_t galois_hip_graph_begin_capture(galois_hip_ctx *ctx) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, !ctx->capturing, GALOIS_HIP_E_UNSUPPORTED, "graph_begin_capture: a capture is already open");
    GH_BIND(ctx);
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e == hipSuccess) ctx->capturing = true;
    return gh_hip(ctx, e, "hipStreamBeginCapture");
}

int32_t galois_hip_graph_end_capture(galois_hip_ctx *ctx, galois_hip_graph **out) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, out != nullptr, GALOIS_HIP_E_NULL, "graph_end_capture: out");
    GH_REQUIRE(ctx, ctx->capturing, GALOIS_HIP_E_UNSUPPORTED, "graph_end_capture: no capture is open");
    GH_BIND(ctx);
    *out = nullptr;
    ctx->capturing = false;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &g);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipStreamEndCapture");
    hipGraphExec_t x = nullptr;
    e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return gh_hip(ctx, e, "hipGraphInstantiate");
    }
    galois_hip_graph *gr = new galois_hip_graph();
    gr->graph = g, gr->exec = x;
    *out = gr;
    return GALOIS_HIP_OK;
}

int32_t galois_hip_graph_launch(galois_hip_ctx *ctx, galois_hip_graph *graph) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, graph != nullptr, GALOIS_HIP_E_NULL, "graph_launch");
    GH_REQUIRE(ctx, !ctx->capturing, GALOIS_HIP_E_UNSUPPORTED, "graph_launch inside a capture");
    GH_BIND(ctx);
    return gh_hip(ctx, hipGraphLaunch(graph->exec, ctx->stream), "hipGraphLaunch");
}

int32_t galois_hip_graph_destroy(galois_hip_ctx *ctx, galois_hip_graph *graph) {
    GH_REQUIRE_CTX(ctx);
    if (!graph) return GALOIS_HIP_OK;
    GH_BIND(ctx);
    hipError_t e1 = hipGraphExecDestroy(graph->exec);
    hipError_t e2 = hipGraphDestroy(graph->graph);
    delete graph;
    return gh_hip(ctx, e1 != hipSuccess ? e1 : e2, "hipGraphDestroy");
}

}  // extern "C"
