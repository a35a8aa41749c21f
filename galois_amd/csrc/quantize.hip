// f32 -> Q4_0 quantizer on the device.
//
// galois leaves BlockQ4_0::from_f32 as todo!() (src/ggml_quants.rs:198-200); Q4_0 data
// reaches it as ready-made bytes (src/lib.rs:2477-2491).  This kernel produces those bytes
// with the canonical ggml rule so that to_f32 (src/ggml_quants.rs:209-228) inverts them:
// per block of 32 the element of largest magnitude (first wins) fixes d = max / -8,
// id = 1/d (0 when d == 0) from the unrounded f32 d, q = min(15, trunc(x*id + 8.5)).
// Every operation is a separately rounded IEEE f32 operation (no fused multiply-add), so
// the bytes are identical to a CPU evaluation of the same rule.
#include "common.h"

namespace {

__global__ __launch_bounds__(256) void quantize_q4_0_blocks(const float *__restrict__ x, uint16_t *__restrict__ y,
                                                           int64_t nblocks) {
#pragma clang fp contract(off)  // the rule is defined with separately rounded multiply and add
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nblocks) return;
    const float *xb = x + b * 32;
    float v[32];
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = xb[j];
    float amax = 0.0f, mx = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; j++) {
        const float a = __builtin_fabsf(v[j]);
        if (amax < a) {
            amax = a;
            mx = v[j];
        }
    }
    float d = mx * -0.125f;  // == mx / -8 exactly (power of two), keeps the sign of zero
    // keep the product a value of its own: fused into the f16 conversion it would be formed as
    // mx * -0.125 + 0, and (-0) + (+0) loses the sign of an all-zero block's scale
    asm volatile("" : "+v"(d));
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint16_t *out = y + b * 9;
    out[0] = __builtin_bit_cast(uint16_t, (_Float16)d);
#pragma unroll
    for (int j = 0; j < 16; j += 2) {
        uint32_t bytes = 0;
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int q0 = (int)(v[j + t] * id + 8.5f);
            const int q1 = (int)(v[j + t + 16] * id + 8.5f);
            bytes |= (uint32_t)(min(q0, 15) | (min(q1, 15) << 4)) << (8 * t);
        }
        out[1 + j / 2] = (uint16_t)bytes;
    }
}

// to_f32 (src/ggml_quants.rs:209-228): blocks -> f32, exact.
__global__ __launch_bounds__(256) void dequantize_q4_0_blocks(const uint16_t *__restrict__ x, float *__restrict__ y,
                                                             int64_t nblocks) {
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nblocks) return;
    const uint16_t *p = x + b * 9;
    const float d = (float)__builtin_bit_cast(_Float16, p[0]);
    float *out = y + b * 32;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t v = p[1 + j];
        out[2 * j] = (float)((int)(v & 0xF) - 8) * d;
        out[2 * j + 16] = (float)((int)((v >> 4) & 0xF) - 8) * d;
        out[2 * j + 1] = (float)((int)((v >> 8) & 0xF) - 8) * d;
        out[2 * j + 17] = (float)((int)((v >> 12) & 0xF) - 8) * d;
    }
}

}  // namespace

extern "C" {

int32_t galois_hip_quantize_row_q4_0(galois_hip_ctx *ctx, const float *x, void *y, int64_t k) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && y, GALOIS_HIP_E_NULL, "quantize_row_q4_0");
    GH_REQUIRE(ctx, k > 0 && k % 32 == 0 && k / 32 <= (int64_t)0x7FFFFFFF * 256, GALOIS_HIP_E_SHAPE,
               "quantize_row_q4_0: k must be a positive multiple of 32");
    GH_REQUIRE(ctx, gh_aligned(x, 4) && gh_aligned(y, 2), GALOIS_HIP_E_ALIGN, "quantize_row_q4_0");
    GH_BIND(ctx);
    const int64_t nb = k / 32;
    hipLaunchKernelGGL(quantize_q4_0_blocks, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, ctx->stream, x,
                       (uint16_t *)y, nb);
    GH_LAUNCH_CHECK(ctx, "quantize_row_q4_0 launch");
}

int32_t galois_hip_dequantize_row_q4_0(galois_hip_ctx *ctx, const void *x, float *y, int64_t k) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && y, GALOIS_HIP_E_NULL, "dequantize_row_q4_0");
    GH_REQUIRE(ctx, k > 0 && k % 32 == 0 && k / 32 <= (int64_t)0x7FFFFFFF * 256, GALOIS_HIP_E_SHAPE,
               "dequantize_row_q4_0: k must be a positive multiple of 32");
    GH_REQUIRE(ctx, gh_aligned(x, 2) && gh_aligned(y, 4), GALOIS_HIP_E_ALIGN, "dequantize_row_q4_0");
    GH_BIND(ctx);
    const int64_t nb = k / 32;
    hipLaunchKernelGGL(dequantize_q4_0_blocks, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, ctx->stream,
                       (const uint16_t *)x, y, nb);
    GH_LAUNCH_CHECK(ctx, "dequantize_row_q4_0 launch");
}

}  // extern "C"
