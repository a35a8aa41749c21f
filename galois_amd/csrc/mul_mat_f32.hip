// f32 x f32 and f16 x f32 batched matmul over strided views: the two products of a decode step's attention
// over the KV cache (scores = K^T q, out = V p), which the reference routes to cuBLAS -- sgemm after a cont()
// copy for f32 (src/cuda.rs:698-782, todo!() at src/cuda.rs:867-879), gemm_ex for an f16 src0
// (CudaMatMul::f_x_y_y, src/cuda.rs:881-992 -> cuda_op_mul_mat_cublas, src/cuda.rs:698-782).
//
//   dst[i2][m][n] = sum_k a[(i2 / r2) * a_s2 + n * a_s1 + k * a_s0] * b[(i2 * M + m) * K + k]
//
// a is f32 or f16 (widened exactly), b and dst f32, sums in f32.  Both attention products read the cache exactly
// once and are HBM-bound.  With M == 1 (decode) two streaming kernels are used; f16 weights with M > 1 go to
// the matrix cores (mul_mat_f16.hip); other shapes take the generic kernels.
#include "common.h"

namespace {

constexpr int kThreads = 256;

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over aligned groups of LANES lanes (8, 16, 32 or 64); every lane of a group ends with its total.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm(1,0,3,2)
    v += dpp_mov<0x4E>(v);   // quad_perm(2,3,0,1)
    v += dpp_mov<0x141>(v);  // row_half_mirror
    if (LANES >= 16) v += dpp_mov<0x140>(v);  // row_mirror
    if (LANES >= 32) v += __shfl_xor(v, 16, 64);
    if (LANES >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// Element loads of the a operand: f32 as it is, f16 widened.
typedef _Float16 mm_half4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float mm_ld1(const float *p) { return *p; }
__device__ __forceinline__ float mm_ld1(const _Float16 *p) { return (float)*p; }
__device__ __forceinline__ float4 mm_ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 mm_ld4(const _Float16 *p) {
    const mm_half4 h = *reinterpret_cast<const mm_half4 *>(p);
    return make_float4((float)h.x, (float)h.y, (float)h.z, (float)h.w);
}

// ---- generic kernels (any K, N, M) ---------------------------------------------------------------

// Rows of `a` contiguous along K (a_s0 == 1).  One wave per (n, i2).
template <typename AT>
__global__ __launch_bounds__(kThreads) void mul_mat_f32_krows(const AT *__restrict__ a, const float *__restrict__ b,
                                                              float *__restrict__ dst, int K, int N, int M, int r2,
                                                              int64_t a_s1, int64_t a_s2) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const int i2 = blockIdx.y;
    if (n >= N) return;
    const AT *ar = a + (int64_t)(i2 / r2) * a_s2 + (int64_t)n * a_s1;
    for (int m = 0; m < M; m++) {
        const float *br = b + ((int64_t)i2 * M + m) * K;
        float acc = 0.0f;
        for (int k = lane; k < K; k += 64) acc = __builtin_fmaf(mm_ld1(ar + k), br[k], acc);
        acc = group_sum<64>(acc);
        if (lane == 0) dst[((int64_t)i2 * M + m) * N + n] = acc;
    }
}

// `a` contiguous along N (a_s1 == 1, K strided by a_s0).  A workgroup owns 64 columns n of one
// batch slice; its 4 waves split K and combine through LDS.
template <typename AT>
__global__ __launch_bounds__(kThreads) void mul_mat_f32_ncols(const AT *__restrict__ a, const float *__restrict__ b,
                                                              float *__restrict__ dst, int K, int N, int M, int r2,
                                                              int64_t a_s0, int64_t a_s2) {
    __shared__ float part[kThreads];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + lane;
    const int i2 = blockIdx.y;
    const AT *ab = a + (int64_t)(i2 / r2) * a_s2;
    for (int m = 0; m < M; m++) {
        const float *br = b + ((int64_t)i2 * M + m) * K;
        float acc = 0.0f;
        if (n < N)
            for (int k = wave; k < K; k += kThreads / 64) acc = __builtin_fmaf(mm_ld1(ab + (int64_t)k * a_s0 + n), br[k], acc);
        part[threadIdx.x] = acc;
        __syncthreads();
        if (wave == 0 && n < N)
            dst[((int64_t)i2 * M + m) * N + n] = (part[lane] + part[64 + lane]) + (part[128 + lane] + part[192 + lane]);
        __syncthreads();
    }
}

// ---- decode kernels (M == 1) -----------------------------------------------------------------------

// scores = K^T q.  K = 4 * LPR floats per row; LPR lanes take one row with a 16-byte load each, so a
// wave-load covers 64 / LPR rows, and a wave keeps U wave-loads in flight before it reduces any.
// Rows are numbered with the batch index fastest when that is the smaller stride, so that the rows
// of one wave-load (and of neighbouring waves) are neighbours in memory.
template <int LPR, int U, typename AT>
__global__ __launch_bounds__(kThreads) void mul_vec_f32_krows(const AT *__restrict__ a, const float *__restrict__ b,
                                                              float *__restrict__ dst, int N, int ne12, int r2,
                                                              int64_t a_s1, int64_t a_s2, int batch_fastest) {
    constexpr int RPL = 64 / LPR, K = LPR * 4;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR, kl = lane % LPR;
    const int64_t R = (int64_t)N * ne12;
    const int64_t r0 = ((int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6)) * (RPL * U);
    if (r0 >= R) return;
    float4 av[U], bv[U];
    int64_t out[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t r = r0 + u * RPL + sub;
        const int64_t rc = r < R ? r : R - 1;
        const int64_t i2 = batch_fastest ? rc % ne12 : rc / N;
        const int64_t n = batch_fastest ? rc / ne12 : rc % N;
        av[u] = mm_ld4(a + (i2 / r2) * a_s2 + n * a_s1 + kl * 4);
        bv[u] = *reinterpret_cast<const float4 *>(b + i2 * K + kl * 4);
        out[u] = r < R ? i2 * N + n : -1;
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        float acc = av[u].x * bv[u].x;
        acc = __builtin_fmaf(av[u].y, bv[u].y, acc);
        acc = __builtin_fmaf(av[u].z, bv[u].z, acc);
        acc = __builtin_fmaf(av[u].w, bv[u].w, acc);
        acc = group_sum<LPR>(acc);
        if (kl == 0 && out[u] >= 0) dst[out[u]] = acc;
    }
}

// out = V p.  Columns c = i2 * N + n of all batch slices are cut into tiles of 256 (a wave reads 1 KB of one
// cache row with a 16-byte load per lane); the K rows are cut into gridDim.y slabs.  The 4 waves of a
// workgroup take a quarter of the slab each, 16 rows at a time all in flight, and combine through LDS.
// With more than one slab the workgroup writes its partial sums to `part` and sum_slabs_f32 adds the
// slabs in slab order afterwards, so the result is the same on every launch.
constexpr int kVecRows = 16;
template <typename AT>
__global__ __launch_bounds__(kThreads) void mul_vec_f32_ncols(const AT *__restrict__ a, const float *__restrict__ b,
                                                              float *__restrict__ dst, float *__restrict__ part, int K, int N, int C, int r2,
                                                              int64_t a_s0, int64_t a_s2, int rows_per_wave) {
    __shared__ float4 red[kThreads / 64][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tile = blockIdx.x, slab = blockIdx.y, nslabs = gridDim.y;
    const int c = tile * 256 + lane * 4;
    const bool col_ok = c < C;  // C and N are multiples of 4: a lane's four columns stay in one batch slice
    const int cc = col_ok ? c : 0;
    const int i2 = cc / N, n = cc % N;
    const AT *ac = a + (int64_t)(i2 / r2) * a_s2 + n;
    const float *bc = b + (int64_t)i2 * K;
    const int k_begin = (slab * (kThreads / 64) + wave) * rows_per_wave;
    const int k_end = min(K, k_begin + rows_per_wave);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k0 = k_begin; k0 < k_end; k0 += kVecRows) {
        float4 v[kVecRows];
        float p[kVecRows];
#pragma unroll
        for (int u = 0; u < kVecRows; u++) {
            const int k = k0 + u;
            const int kc = k < k_end ? k : k_end - 1;
            v[u] = mm_ld4(ac + (int64_t)kc * a_s0);
            p[u] = bc[kc];
        }
#pragma unroll
        for (int u = 0; u < kVecRows; u++) {
            if (k0 + u < k_end) {  // uniform across the wave
                acc.x = __builtin_fmaf(v[u].x, p[u], acc.x);
                acc.y = __builtin_fmaf(v[u].y, p[u], acc.y);
                acc.z = __builtin_fmaf(v[u].z, p[u], acc.z);
                acc.w = __builtin_fmaf(v[u].w, p[u], acc.w);
            }
        }
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0) {
        const float4 s0 = red[0][lane], s1 = red[1][lane], s2 = red[2][lane], s3 = red[3][lane];
        float4 s;
        s.x = (s0.x + s1.x) + (s2.x + s3.x);
        s.y = (s0.y + s1.y) + (s2.y + s3.y);
        s.z = (s0.z + s1.z) + (s2.z + s3.z);
        s.w = (s0.w + s1.w) + (s2.w + s3.w);
        if (col_ok) *reinterpret_cast<float4 *>((nslabs == 1 ? dst : part + (int64_t)slab * C) + c) = s;
    }
}

// Second pass of the split product: adds the slabs in slab order.
__global__ __launch_bounds__(kThreads) void sum_slabs_f32(const float *__restrict__ part, float *__restrict__ dst,
                                                          int C, int nslabs) {
    const int c = blockIdx.x * kThreads + threadIdx.x;
    if (c >= C) return;
    float s = 0.0f;
    for (int j0 = 0; j0 < nslabs; j0 += 16) {
        float t[16];
#pragma unroll
        for (int j = 0; j < 16; j++) t[j] = part[(int64_t)min(j0 + j, nslabs - 1) * C + c];
#pragma unroll
        for (int j = 0; j < 16; j++)
            if (j0 + j < nslabs) s += t[j];
    }
    dst[c] = s;
}

template <int LPR, typename AT>
void launch_vec_krows(galois_hip_ctx *ctx, const AT *a, const float *b, float *dst, int N, int ne12, int r2,
                      int64_t a_s1, int64_t a_s2) {
    constexpr int U = 8, rows_per_wg = (kThreads / 64) * (64 / LPR) * U;
    const int64_t R = (int64_t)N * ne12;
    hipLaunchKernelGGL((mul_vec_f32_krows<LPR, U, AT>), dim3((unsigned)((R + rows_per_wg - 1) / rows_per_wg)),
                       dim3(kThreads), 0, ctx->stream, a, b, dst, N, ne12, r2, a_s1, a_s2, (int)(a_s2 < a_s1));
}

}  // namespace

// gemm_f16_f32_mfma (mul_mat_f16.hip): f16 rows contiguous along K against M > 1 rows of b on the matrix cores;
// returns false when the operands do not fit it (the generic kernels then serve the call).
bool gh_mul_mat_f16_mfma(galois_hip_ctx *ctx, const _Float16 *a, const float *b, float *dst, int K, int N, int M,
                         int ne02, int ne12, int64_t a_s1, int64_t a_s2);

// gemm_f32_mfma (mul_mat_f32_mfma.hip): many rows of b on the matrix cores in full f32, a contiguous along K or N.
template <typename AT>
bool gh_mul_mat_f32_mfma(galois_hip_ctx *ctx, const AT *a, const float *b, float *dst, int K, int N, int M, int ne02,
                         int ne12, int64_t a_s0, int64_t a_s1, int64_t a_s2);

namespace {

constexpr int kMfmaMinRows = 16;  // rows of b from which the 128-row tiles of the f32 matrix-core kernel pay

template <typename AT>
int32_t mul_mat_any(galois_hip_ctx *ctx, const AT *a, const float *b, float *dst, int32_t K, int32_t N, int32_t M,
                    int32_t ne02, int32_t ne12, int64_t a_s0, int64_t a_s1, int64_t a_s2) {
    constexpr bool F16 = sizeof(AT) == 2;
    constexpr size_t A16 = F16 ? 8 : 16;  // alignment of a four-element load
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, a && b && dst, GALOIS_HIP_E_NULL, "mul_mat_f32");
    GH_REQUIRE(ctx, K > 0 && N > 0 && M > 0 && ne02 > 0 && ne12 > 0 && ne12 % ne02 == 0 && ne12 <= 65535,
               GALOIS_HIP_E_SHAPE, "mul_mat_f32");
    GH_REQUIRE(ctx, a_s0 == 1 || a_s1 == 1, GALOIS_HIP_E_UNSUPPORTED,
               "mul_mat_f32: a must be contiguous along K (a_s0 == 1) or along N (a_s1 == 1)");
    GH_REQUIRE(ctx, gh_aligned(a, sizeof(AT)) && gh_aligned(b, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN, "mul_mat_f32");
    GH_BIND(ctx);
    const int r2 = ne12 / ne02;
    if (F16 && M > 1 && a_s0 == 1 &&
        gh_mul_mat_f16_mfma(ctx, (const _Float16 *)a, b, dst, K, N, M, ne02, ne12, a_s1, a_s2))
        GH_LAUNCH_CHECK(ctx, "mul_mat_f16_f32 launch");
    if (M >= kMfmaMinRows && gh_mul_mat_f32_mfma<AT>(ctx, a, b, dst, K, N, M, ne02, ne12, a_s0, a_s1, a_s2))
        GH_LAUNCH_CHECK(ctx, "mul_mat_f32 launch (matrix cores)");
    const bool vec16 = M == 1 && gh_aligned(a, A16) && gh_aligned(b, 16) && a_s2 % 4 == 0;
    if (a_s0 == 1) {
        const bool fast = vec16 && a_s1 % 4 == 0 && (K == 32 || K == 64 || K == 128 || K == 256);
        if (fast) {
            switch (K) {
                case 32: launch_vec_krows<8>(ctx, a, b, dst, N, ne12, r2, a_s1, a_s2); break;
                case 64: launch_vec_krows<16>(ctx, a, b, dst, N, ne12, r2, a_s1, a_s2); break;
                case 128: launch_vec_krows<32>(ctx, a, b, dst, N, ne12, r2, a_s1, a_s2); break;
                default: launch_vec_krows<64>(ctx, a, b, dst, N, ne12, r2, a_s1, a_s2); break;
            }
        } else {
            hipLaunchKernelGGL(mul_mat_f32_krows<AT>, dim3((N + 3) / 4, ne12), dim3(kThreads), 0, ctx->stream, a, b, dst, K,
                               N, M, r2, a_s1, a_s2);
        }
    } else {
        const int64_t C = (int64_t)N * ne12;
        const int64_t tiles = (C + 255) / 256;
        // slabs of K: 16 rows per wave while that gives at most 64 slabs, more rows per wave beyond
        int rows_per_wave = kVecRows;
        while ((int64_t)rows_per_wave * (kThreads / 64) * 64 < K) rows_per_wave += kVecRows;
        const int rows_per_wg = rows_per_wave * (kThreads / 64);
        const int nslabs = (K + rows_per_wg - 1) / rows_per_wg;
        const bool fast = vec16 && gh_aligned(dst, 16) && a_s0 % 4 == 0 && N % 4 == 0 && tiles <= 65535 &&
                          (nslabs == 1 || (int64_t)nslabs * C <= GH_PARTIAL_FLOATS) && ctx->scratch != nullptr;
        if (fast) {
            float *part = (float *)ctx->scratch;
            hipLaunchKernelGGL(mul_vec_f32_ncols<AT>, dim3((unsigned)tiles, nslabs), dim3(kThreads), 0, ctx->stream, a, b,
                               dst, part, K, N, (int)C, r2, a_s0, a_s2, rows_per_wave);
            if (nslabs > 1)
                hipLaunchKernelGGL(sum_slabs_f32, dim3((unsigned)((C + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                                   ctx->stream, part, dst, (int)C, nslabs);
        } else {
            hipLaunchKernelGGL(mul_mat_f32_ncols<AT>, dim3((N + 63) / 64, ne12), dim3(kThreads), 0, ctx->stream, a, b, dst,
                               K, N, M, r2, a_s0, a_s2);
        }
    }
    GH_LAUNCH_CHECK(ctx, "mul_mat_f32 launch");
}

}  // namespace

extern "C" int32_t galois_hip_mul_mat_f32(galois_hip_ctx *ctx, const float *a, const float *b, float *dst, int32_t K,
                                          int32_t N, int32_t M, int32_t ne02, int32_t ne12, int64_t a_s0, int64_t a_s1,
                                          int64_t a_s2) {
    return mul_mat_any<float>(ctx, a, b, dst, K, N, M, ne02, ne12, a_s0, a_s1, a_s2);
}

extern "C" int32_t galois_hip_mul_mat_f16_f32(galois_hip_ctx *ctx, const void *a, const float *b, float *dst, int32_t K,
                                              int32_t N, int32_t M, int32_t ne02, int32_t ne12, int64_t a_s0,
                                              int64_t a_s1, int64_t a_s2) {
    return mul_mat_any<_Float16>(ctx, (const _Float16 *)a, b, dst, K, N, M, ne02, ne12, a_s0, a_s1, a_s2);
}
