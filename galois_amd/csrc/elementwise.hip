// Elementwise, copy and gather kernels around the Q4_0 path (the reference's add / mul / scale /
// silu / cpy kernels and the CPU-only get_rows).  All are HBM-bound, one read and one write per element.
#include "common.h"

namespace {

constexpr int kEwThreads = 256;

enum { EW_ADD = 0, EW_MUL = 1 };

// add_f32 / mul_f32 (galois-kernels/src/add.cu:3-12, mul.cu:3-12): dst[i] = x[i] op y[i % ky].
// The reference launcher swaps grid and block (src/cuda.rs:1206-1210, 1235-1239); not copied.
template <int OP>
__global__ __launch_bounds__(kEwThreads) void ew_bcast(const float *__restrict__ x, const float *__restrict__ y,
                                                       float *__restrict__ dst, int64_t kx, int64_t ky) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i >= kx) return;
    const float b = y[i % ky];
    dst[i] = OP == EW_ADD ? x[i] + b : x[i] * b;
}

// Vector form when kx, ky are multiples of 4 and pointers 16-byte aligned: y index never splits a float4.
template <int OP>
__global__ __launch_bounds__(kEwThreads) void ew_bcast4(const float4 *__restrict__ x, const float4 *__restrict__ y,
                                                        float4 *__restrict__ dst, int64_t kx4, int64_t ky4) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i >= kx4) return;
    const float4 a = x[i], b = y[i % ky4];
    dst[i] = OP == EW_ADD ? make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w)
                          : make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w);
}

// scale_f32 (scale.cu:1-11)
__global__ __launch_bounds__(kEwThreads) void ew_scale(const float *__restrict__ x, float *__restrict__ dst,
                                                       float scale, int64_t k) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i < k) dst[i] = scale * x[i];
}

// Four elements per thread when k % 4 == 0 and the pointers are 16-byte aligned.
__global__ __launch_bounds__(kEwThreads) void ew_scale4(const float4 *__restrict__ x, float4 *__restrict__ dst,
                                                        float scale, int64_t k4) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i >= k4) return;
    const float4 a = x[i];
    dst[i] = make_float4(scale * a.x, scale * a.y, scale * a.z, scale * a.w);
}

__device__ __forceinline__ float silu1(float v) { return v / (1.0f + expf(-v)); }

// silu_f32 (unary.cu:1-10): x / (1 + exp(-x)); with `up` != nullptr the SwiGLU product silu(x) * up.
__global__ __launch_bounds__(kEwThreads) void ew_silu(const float *__restrict__ x, const float *__restrict__ up,
                                                      float *__restrict__ dst, int64_t k) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i >= k) return;
    const float s = silu1(x[i]);
    dst[i] = up ? s * up[i] : s;
}

__global__ __launch_bounds__(kEwThreads) void ew_silu4(const float4 *__restrict__ x, const float4 *__restrict__ up,
                                                       float4 *__restrict__ dst, int64_t k4) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i >= k4) return;
    const float4 v = x[i];
    float4 s = make_float4(silu1(v.x), silu1(v.y), silu1(v.z), silu1(v.w));
    if (up) {
        const float4 u = up[i];
        s.x *= u.x, s.y *= u.y, s.z *= u.z, s.w *= u.w;
    }
    dst[i] = s;
}

// cpy_f32_f32 / cpy_f32_f16 (cpy.cu:79-156): element i of a [ne00, ne01, *] source with byte
// strides nb00.. is written to element i of a [ne10, ne11, *] destination with byte strides nb10..
template <typename DST>
__global__ __launch_bounds__(kEwThreads) void cpy_strided(const char *__restrict__ cx, char *__restrict__ cdst,
                                                          int64_t ne, int64_t ne00, int64_t ne01, int64_t nb00,
                                                          int64_t nb01, int64_t nb02, int64_t ne10, int64_t ne11,
                                                          int64_t nb10, int64_t nb11, int64_t nb12) {
    const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (i >= ne) return;
    const int64_t i02 = i / (ne00 * ne01), r0 = i - i02 * ne00 * ne01;
    const int64_t i01 = r0 / ne00, i00 = r0 - i01 * ne00;
    const int64_t i12 = i / (ne10 * ne11), r1 = i - i12 * ne10 * ne11;
    const int64_t i11 = r1 / ne10, i10 = r1 - i11 * ne10;
    const float v = *reinterpret_cast<const float *>(cx + i00 * nb00 + i01 * nb01 + i02 * nb02);
    *reinterpret_cast<DST *>(cdst + i10 * nb10 + i11 * nb11 + i12 * nb12) = (DST)v;
}

// get_rows for a Q4_0 table (GetRows::f_q_x_f32, src/op.rs:2546-2571; CPU-only in the reference):
// dst row i = to_f32(table row ids[i]).  One wave per row, one block per lane per step.  The ids come from device
// memory, so they are checked here: a row whose id is outside the table is filled with NaN and no table byte is
// read for it (the reference indexes bounded slices and would panic).
__global__ __launch_bounds__(kEwThreads) void get_rows_q4_0(const uint16_t *__restrict__ table,
                                                            const int32_t *__restrict__ ids, float *__restrict__ dst,
                                                            int nblocks, int nr, int n_table_rows) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kEwThreads / 64) + (threadIdx.x >> 6);
    if (r >= nr) return;
    const int id = ids[r];
    float *out = dst + (size_t)r * nblocks * 32;
    if (id < 0 || id >= n_table_rows) {  // wave-uniform
        for (int i = lane; i < nblocks * 32; i += 64) out[i] = __builtin_nanf("");
        return;
    }
    const uint16_t *row = table + (size_t)id * nblocks * 9;
    for (int b = lane; b < nblocks; b += 64) {
        const uint16_t *p = row + (size_t)b * 9;
        const float d = (float)__builtin_bit_cast(_Float16, p[0]);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t v = p[1 + j];
            out[b * 32 + 2 * j] = (float)((int)(v & 0xF) - 8) * d;
            out[b * 32 + 2 * j + 16] = (float)((int)((v >> 4) & 0xF) - 8) * d;
            out[b * 32 + 2 * j + 1] = (float)((int)((v >> 8) & 0xF) - 8) * d;
            out[b * 32 + 2 * j + 17] = (float)((int)((v >> 12) & 0xF) - 8) * d;
        }
    }
}

int32_t launch_bcast(galois_hip_ctx *ctx, int op, const float *x, const float *y, float *dst, int64_t kx, int64_t ky,
                     const char *what) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && y && dst, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, kx > 0 && ky > 0 && kx <= (int64_t)0x7FFFFFFF * kEwThreads, GALOIS_HIP_E_SHAPE, what);
    GH_REQUIRE(ctx, gh_aligned(x, 4) && gh_aligned(y, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN, what);
    GH_BIND(ctx);
    if (kx % 4 == 0 && ky % 4 == 0 && gh_aligned(x, 16) && gh_aligned(y, 16) && gh_aligned(dst, 16)) {
        const dim3 grid((unsigned)((kx / 4 + kEwThreads - 1) / kEwThreads));
        if (op == EW_ADD)
            hipLaunchKernelGGL(ew_bcast4<EW_ADD>, grid, dim3(kEwThreads), 0, ctx->stream, (const float4 *)x,
                               (const float4 *)y, (float4 *)dst, kx / 4, ky / 4);
        else
            hipLaunchKernelGGL(ew_bcast4<EW_MUL>, grid, dim3(kEwThreads), 0, ctx->stream, (const float4 *)x,
                               (const float4 *)y, (float4 *)dst, kx / 4, ky / 4);
    } else {
        const dim3 grid((unsigned)((kx + kEwThreads - 1) / kEwThreads));
        if (op == EW_ADD)
            hipLaunchKernelGGL(ew_bcast<EW_ADD>, grid, dim3(kEwThreads), 0, ctx->stream, x, y, dst, kx, ky);
        else
            hipLaunchKernelGGL(ew_bcast<EW_MUL>, grid, dim3(kEwThreads), 0, ctx->stream, x, y, dst, kx, ky);
    }
    GH_LAUNCH_CHECK(ctx, what);
}

}  // namespace

extern "C" {

int32_t galois_hip_add_f32(galois_hip_ctx *ctx, const float *x, const float *y, float *dst, int64_t kx, int64_t ky) {
    return launch_bcast(ctx, EW_ADD, x, y, dst, kx, ky, "add_f32");
}

int32_t galois_hip_mul_f32(galois_hip_ctx *ctx, const float *x, const float *y, float *dst, int64_t kx, int64_t ky) {
    return launch_bcast(ctx, EW_MUL, x, y, dst, kx, ky, "mul_f32");
}

int32_t galois_hip_scale_f32(galois_hip_ctx *ctx, const float *x, float *dst, float scale, int64_t k) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && dst, GALOIS_HIP_E_NULL, "scale_f32");
    GH_REQUIRE(ctx, k > 0 && k <= (int64_t)0x7FFFFFFF * kEwThreads, GALOIS_HIP_E_SHAPE, "scale_f32");
    GH_REQUIRE(ctx, gh_aligned(x, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN, "scale_f32");
    GH_BIND(ctx);
    if (k % 4 == 0 && gh_aligned(x, 16) && gh_aligned(dst, 16))
        hipLaunchKernelGGL(ew_scale4, dim3((unsigned)((k / 4 + kEwThreads - 1) / kEwThreads)), dim3(kEwThreads), 0,
                           ctx->stream, (const float4 *)x, (float4 *)dst, scale, k / 4);
    else
        hipLaunchKernelGGL(ew_scale, dim3((unsigned)((k + kEwThreads - 1) / kEwThreads)), dim3(kEwThreads), 0,
                           ctx->stream, x, dst, scale, k);
    GH_LAUNCH_CHECK(ctx, "scale_f32 launch");
}

static int32_t launch_silu(galois_hip_ctx *ctx, const float *x, const float *up, float *dst, int64_t k,
                           const char *what) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && dst, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, k > 0 && k <= (int64_t)0x7FFFFFFF * kEwThreads, GALOIS_HIP_E_SHAPE, what);
    GH_REQUIRE(ctx, gh_aligned(x, 4) && gh_aligned(up, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN, what);
    GH_BIND(ctx);
    if (k % 4 == 0 && gh_aligned(x, 16) && gh_aligned(up, 16) && gh_aligned(dst, 16))
        hipLaunchKernelGGL(ew_silu4, dim3((unsigned)((k / 4 + kEwThreads - 1) / kEwThreads)), dim3(kEwThreads), 0,
                           ctx->stream, (const float4 *)x, (const float4 *)up, (float4 *)dst, k / 4);
    else
        hipLaunchKernelGGL(ew_silu, dim3((unsigned)((k + kEwThreads - 1) / kEwThreads)), dim3(kEwThreads), 0,
                           ctx->stream, x, up, dst, k);
    GH_LAUNCH_CHECK(ctx, what);
}

int32_t galois_hip_silu_f32(galois_hip_ctx *ctx, const float *x, float *dst, int64_t k) {
    return launch_silu(ctx, x, nullptr, dst, k, "silu_f32");
}

int32_t galois_hip_silu_mul_f32(galois_hip_ctx *ctx, const float *gate, const float *up, float *dst, int64_t k) {
    if (ctx && !up) return gh_fail(ctx, GALOIS_HIP_E_NULL, "silu_mul_f32: up");
    return launch_silu(ctx, gate, up, dst, k, "silu_mul_f32");
}

int32_t galois_hip_cpy_f32(galois_hip_ctx *ctx, const void *x, void *dst, int32_t dst_is_f16, int64_t ne, int64_t ne00,
                           int64_t ne01, int64_t nb00, int64_t nb01, int64_t nb02, int64_t ne10, int64_t ne11,
                           int64_t nb10, int64_t nb11, int64_t nb12) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && dst, GALOIS_HIP_E_NULL, "cpy_f32");
    GH_REQUIRE(ctx, ne > 0 && ne00 > 0 && ne01 > 0 && ne10 > 0 && ne11 > 0 && ne <= (int64_t)0x7FFFFFFF * kEwThreads,
               GALOIS_HIP_E_SHAPE, "cpy_f32");
    const int64_t dsz = dst_is_f16 ? 2 : 4;
    GH_REQUIRE(ctx, nb00 % 4 == 0 && nb01 % 4 == 0 && nb02 % 4 == 0 && nb10 % dsz == 0 && nb11 % dsz == 0 &&
                        nb12 % dsz == 0 && gh_aligned(x, 4) && gh_aligned(dst, (size_t)dsz),
               GALOIS_HIP_E_ALIGN, "cpy_f32: strides and pointers must be multiples of the element size");
    GH_BIND(ctx);
    const dim3 grid((unsigned)((ne + kEwThreads - 1) / kEwThreads));
    if (dst_is_f16)
        hipLaunchKernelGGL(cpy_strided<_Float16>, grid, dim3(kEwThreads), 0, ctx->stream, (const char *)x, (char *)dst,
                           ne, ne00, ne01, nb00, nb01, nb02, ne10, ne11, nb10, nb11, nb12);
    else
        hipLaunchKernelGGL(cpy_strided<float>, grid, dim3(kEwThreads), 0, ctx->stream, (const char *)x, (char *)dst, ne,
                           ne00, ne01, nb00, nb01, nb02, ne10, ne11, nb10, nb11, nb12);
    GH_LAUNCH_CHECK(ctx, "cpy_f32 launch");
}

int32_t galois_hip_get_rows_q4_0(galois_hip_ctx *ctx, const void *table, const int32_t *ids, float *dst, int32_t ncols,
                                 int32_t nr, int32_t n_table_rows) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, table && ids && dst, GALOIS_HIP_E_NULL, "get_rows_q4_0");
    GH_REQUIRE(ctx, ncols > 0 && ncols % 32 == 0 && nr > 0 && n_table_rows > 0, GALOIS_HIP_E_SHAPE, "get_rows_q4_0");
    GH_REQUIRE(ctx, gh_aligned(table, 2) && gh_aligned(ids, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN, "get_rows_q4_0");
    GH_BIND(ctx);
    hipLaunchKernelGGL(get_rows_q4_0, dim3((nr + 3) / 4), dim3(kEwThreads), 0, ctx->stream, (const uint16_t *)table,
                       ids, dst, ncols / 32, nr, n_table_rows);
    GH_LAUNCH_CHECK(ctx, "get_rows_q4_0 launch");
}

}  // extern "C"
