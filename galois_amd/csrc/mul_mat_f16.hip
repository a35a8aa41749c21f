// f16 x f32 batched matmul on the matrix cores: the (F16, F32) -> F32 arm of galois_matmul, which the reference
// serves with cuBLAS gemm_ex after converting src1 to f16 (CudaMatMul::f_x_y_y, src/cuda.rs:881-992 ->
// cuda_op_mul_mat_cublas, src/cuda.rs:698-757: f16 operands, f16 accumulation, f16 result widened to f32).
//
//   dst[i2][m][n] = sum_k a[(i2 / r2) * a_s2 + n * a_s1 + k] * b[(i2 * M + m) * K + k]
//
// Here a stays f16, b is rounded to f16 on its way into LDS as the reference's convert_fp32_to_fp16 does, and
// v_mfma_f32_32x32x16_f16 accumulates in f32 (the reference accumulates in f16: this result is the more exact of
// the two).  Workgroup tile 128 x 128, k step 32, four waves of 64 x 64; one grid layer per batch slice.
#include "common.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int FM = 128, FN = 128;
constexpr int F_STRIDE = 40;  // halfs per tile row: 80-byte rows keep 16-byte fragment reads conflict-free

__device__ __forceinline__ uint32_t f16_pack(float a, float b) {
    half2_t h;
    h.x = (_Float16)a;
    h.y = (_Float16)b;
    return __builtin_bit_cast(uint32_t, h);
}

__global__ __launch_bounds__(256) void gemm_f16_f32_mfma(const _Float16 *__restrict__ a, const float *__restrict__ b,
                                                          float *__restrict__ dst, int K, int N, int M, int r2,
                                                          int64_t a_s1, int64_t a_s2) {
    __shared__ __attribute__((aligned(16))) _Float16 As[FM * F_STRIDE];  // rows of b (m)
    __shared__ __attribute__((aligned(16))) _Float16 Bs[FN * F_STRIDE];  // rows of a (n)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * FM, n0 = blockIdx.x * FN, i2 = blockIdx.z;
    const _Float16 *ab = a + (int64_t)(i2 / r2) * a_s2;
    const float *bb = b + (int64_t)i2 * M * K;
    float *db = dst + (int64_t)i2 * M * N;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // staging roles: thread -> (tile row, half of the 32-wide k slice); rows past the end repeat the last row
    const int srow = tid >> 1, shalf = tid & 1;
    const float *xp = bb + (size_t)min(m0 + srow, M - 1) * K + shalf * 16;
    const _Float16 *wp = ab + (int64_t)min(n0 + srow, N - 1) * a_s1 + shalf * 16;

    for (int k0 = 0; k0 < K; k0 += 32) {
        {
            const float4 *p = reinterpret_cast<const float4 *>(xp + k0);
            const float4 x0 = p[0], x1 = p[1], x2 = p[2], x3 = p[3];
            uint4 lo, hi;
            lo.x = f16_pack(x0.x, x0.y), lo.y = f16_pack(x0.z, x0.w), lo.z = f16_pack(x1.x, x1.y), lo.w = f16_pack(x1.z, x1.w);
            hi.x = f16_pack(x2.x, x2.y), hi.y = f16_pack(x2.z, x2.w), hi.z = f16_pack(x3.x, x3.y), hi.w = f16_pack(x3.z, x3.w);
            uint4 *d = reinterpret_cast<uint4 *>(As + srow * F_STRIDE + shalf * 16);
            d[0] = lo;
            d[1] = hi;
        }
        {
            const uint4 *p = reinterpret_cast<const uint4 *>(wp + k0);
            const uint4 w0 = p[0], w1 = p[1];
            uint4 *d = reinterpret_cast<uint4 *>(Bs + srow * F_STRIDE + shalf * 16);
            d[0] = w0;
            d[1] = w1;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            half8_t fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                fa[i] = *reinterpret_cast<const half8_t *>(As + (wm * 64 + i * 32 + (lane & 31)) * F_STRIDE + ks * 16 +
                                                           (lane >> 5) * 8);
#pragma unroll
            for (int j = 0; j < 2; j++)
                fb[j] = *reinterpret_cast<const half8_t *>(Bs + (wn * 64 + j * 32 + (lane & 31)) * F_STRIDE + ks * 16 +
                                                           (lane >> 5) * 8);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // C layout of the 32x32 MFMA (A rows = m, B rows = n): column n = lane % 32, row m = 8*(e/4) + 4*(lane/32) + e%4
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m < M && n < N) db[(size_t)m * N + n] = acc[i][j][e];
            }
        }
}

}  // namespace

// f16 rows contiguous along K against M > 1 rows of b; false when the operands do not fit the kernel
// (K % 32, 16-byte alignment of every row of a and b), in which case nothing was launched.
bool gh_mul_mat_f16_mfma(galois_hip_ctx *ctx, const _Float16 *a, const float *b, float *dst, int K, int N, int M,
                         int ne02, int ne12, int64_t a_s1, int64_t a_s2) {
    if (K % 32 != 0 || !gh_aligned(a, 16) || !gh_aligned(b, 16) || a_s1 % 8 != 0 || a_s2 % 8 != 0 || ne12 > 65535 ||
        (M + FM - 1) / FM > 65535)
        return false;
    const dim3 grid((N + FN - 1) / FN, (M + FM - 1) / FM, ne12);
    hipLaunchKernelGGL(gemm_f16_f32_mfma, grid, dim3(256), 0, ctx->stream, a, b, dst, K, N, M, ne12 / ne02, a_s1, a_s2);
    return true;
}
