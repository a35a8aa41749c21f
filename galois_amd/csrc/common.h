// Shared internals of libgalois_hip: context object, status helpers, Q4_0 block.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "../../include/galois_hip.h"

struct galois_hip_ctx {
    int32_t ordinal;
    hipStream_t stream;
    int32_t n_cu;
    void *ws;         // workspace owned by the context (fp16 activations of the prefill matmul)
    size_t ws_bytes;
    std::vector<void *> ws_retired;  // outgrown workspaces: a graph captured earlier may still point into them
    void *scratch;    // fixed block made at creation: partial sums of the split f32 matmul, partial results of the decode attention
    unsigned *attn_done;  // 4 x GH_ATTN_HEADS counters, zero between calls: splits finished per head (decode attention), then
                          // per head the workgroups that have stored its q, its k, its v (the launch that carries both)
    void *attn_static;    // this device's copy of the decode attention's static scratch (attn_decode.hip), found at creation
                          // (null if the lookup failed: only the entry point that needs it then refuses)
    unsigned *dev_status;      // one word of pinned host memory that kernels set when a bounded wait inside a launch runs
    unsigned *dev_status_dev;  // out (the device's address of the same word); read and cleared after every stream wait
    int32_t wait_spin_limit;   // polls a bounded in-launch wait makes before it gives up (GALOIS_HIP_OPT_WAIT_SPIN_LIMIT)
    int32_t wait_target_bias;  // added to the count such a wait waits for: test hook (GALOIS_HIP_OPT_WAIT_TARGET_BIAS)
    bool gemv_f32;             // GALOIS_HIP_OPT_GEMV_F32_ARITHMETIC: one-product GEMV in the reference's f32 arithmetic
    bool capturing;   // between graph_begin_capture and graph_end_capture: nothing may allocate or block
    char last_error[256];
};

// galois_hip_ctx::scratch holds GH_PARTIAL_FLOATS floats of partial sums.
constexpr int64_t GH_PARTIAL_FLOATS = 1 << 20;
constexpr int64_t GH_ATTN_HEADS = 65536;
constexpr int32_t GH_WAIT_SPIN_DEFAULT = 1 << 20;  // polls of a bounded in-launch wait (a poll and its sleep take about a microsecond)

struct galois_hip_event {
    hipEvent_t ev;
};

struct galois_hip_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

// Q4_0 block exactly as the reference stores it (src/ggml_quants.rs:140-145).
struct block_q4_0 {
    uint16_t d;      // f16 bits
    uint8_t qs[16];  // weight j = low nibble of qs[j], weight j+16 = high nibble
};
static_assert(sizeof(block_q4_0) == 18, "Q4_0 block must be 18 bytes");

static inline int32_t gh_fail(galois_hip_ctx *ctx, int32_t status, const char *what) {
    if (ctx) snprintf(ctx->last_error, sizeof(ctx->last_error), "%s: %s", what, galois_hip_status_string(status));
    return status;
}

static inline int32_t gh_hip(galois_hip_ctx *ctx, hipError_t e, const char *what) {
    if (e == hipSuccess) return GALOIS_HIP_OK;
    if (ctx) snprintf(ctx->last_error, sizeof(ctx->last_error), "%s: %s", what, hipGetErrorString(e));
    return (int32_t)e;
}

#define GH_REQUIRE_CTX(ctx) \
    do {                    \
        if (!(ctx)) return GALOIS_HIP_E_NULL; \
    } while (0)

#define GH_REQUIRE(ctx, cond, status, what)            \
    do {                                               \
        if (!(cond)) return gh_fail((ctx), (status), (what)); \
    } while (0)

// Calls that allocate, free or block are refused while the stream is being captured.
#define GH_NOT_CAPTURING(ctx, what) GH_REQUIRE((ctx), !(ctx)->capturing, GALOIS_HIP_E_UNSUPPORTED, what " during a graph capture")

// Binds the context's device to the calling thread, then checks the launch that follows.
#define GH_BIND(ctx)                                                       \
    do {                                                                   \
        hipError_t e__ = hipSetDevice((ctx)->ordinal);                     \
        if (e__ != hipSuccess) return gh_hip((ctx), e__, "hipSetDevice"); \
    } while (0)

#define GH_LAUNCH_CHECK(ctx, what) return gh_hip((ctx), hipGetLastError(), (what))

// device.hip: after a wait for the stream, reports (and clears) what kernels left in the context's status word.
int32_t gh_check_device_status(galois_hip_ctx *ctx);

// attn_decode.hip: looks up the device's copy of the attention's static scratch (the context's device is current).
int32_t gh_attn_static_init(galois_hip_ctx *ctx);

static inline bool gh_aligned(const void *p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }
