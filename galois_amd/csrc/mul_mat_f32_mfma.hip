// f32 (or f16) x f32 batched matmul with M > 1 on the matrix cores in full f32: the attention products of a
// prefill (scores = K^T q over many positions, out = V p), which the reference leaves to cuBLAS sgemm for an f32
// src0 (src/cuda.rs:698-782; the f32 arm of CudaMatMul is todo!() at src/cuda.rs:867-879) and to gemm_ex for an f16
// one (src/cuda.rs:881-992).
//
//   dst[i2][m][n] = sum_k a[(i2 / r2) * a_s2 + n * a_s1 + k * a_s0] * b[(i2 * M + m) * K + k]
//
// v_mfma_f32_32x32x2_f32 multiplies and accumulates in f32, so nothing is rounded that the scalar kernels do not
// round (an f16 a is widened exactly).  Workgroup tile 128 x 128, k step 16, four waves of 64 x 64; one grid layer
// per batch slice.  a may be contiguous along K (a K^T-style view of a cache) or along N (a V-style view): the
// staging loads follow the contiguous direction and the tile lands in LDS as [n][k] either way.  Any K, N, M: rows
// and k past the end are staged as zeros.
#include "common.h"

namespace {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int SM = 128, SN = 128, SK = 16;
constexpr int S_STRIDE = SK + 1;  // floats per tile row: an odd stride spreads the 32 rows of a fragment over all banks

template <typename AT, bool K_CONTIG>
__global__ __launch_bounds__(256) void gemm_f32_mfma(const AT *__restrict__ a, const float *__restrict__ b,
                                                      float *__restrict__ dst, int K, int N, int M, int r2, int64_t a_s0,
                                                      int64_t a_s1, int64_t a_s2) {
    __shared__ float As[SM * S_STRIDE];  // rows of b (m)
    __shared__ float Bs[SN * S_STRIDE];  // rows of a (n)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * SM, n0 = blockIdx.x * SN, i2 = blockIdx.z;
    const AT *ab = a + (int64_t)(i2 / r2) * a_s2;
    const float *bb = b + (int64_t)i2 * M * K;
    float *db = dst + (int64_t)i2 * M * N;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // staging along K: thread -> (tile row, half of the 16-wide k slice); along N: thread -> (k, 8 consecutive n)
    const int srow = tid >> 1, sk = (tid & 1) * 8;
    const int tk = tid >> 4, tn = (tid & 15) * 8;
    const bool m_ok = m0 + srow < M, n_ok = n0 + srow < N;
    const float *xp = bb + (size_t)min(m0 + srow, M - 1) * K;
    const AT *wp = ab + (int64_t)min(n0 + srow, N - 1) * a_s1;

    for (int k0 = 0; k0 < K; k0 += SK) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int k = k0 + sk + e;
            As[srow * S_STRIDE + sk + e] = (m_ok && k < K) ? xp[k] : 0.0f;
        }
        if (K_CONTIG) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int k = k0 + sk + e;
                Bs[srow * S_STRIDE + sk + e] = (n_ok && k < K) ? (float)wp[k] : 0.0f;
            }
        } else {
            const int k = k0 + tk;
            const AT *cp = ab + (int64_t)min(k, K - 1) * a_s0;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int n = n0 + tn + e;
                Bs[(tn + e) * S_STRIDE + tk] = (k < K && n < N) ? (float)cp[min(n, N - 1)] : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < SK / 2; ks++) {
            float fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) fa[i] = As[(wm * 64 + i * 32 + (lane & 31)) * S_STRIDE + ks * 2 + (lane >> 5)];
#pragma unroll
            for (int j = 0; j < 2; j++) fb[j] = Bs[(wn * 64 + j * 32 + (lane & 31)) * S_STRIDE + ks * 2 + (lane >> 5)];
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
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

// M > 1 rows of b against a contiguous along K (a_s0 == 1) or along N (a_s1 == 1); false when the grid does not
// fit, in which case nothing was launched.
template <typename AT>
bool gh_mul_mat_f32_mfma(galois_hip_ctx *ctx, const AT *a, const float *b, float *dst, int K, int N, int M, int ne02,
                         int ne12, int64_t a_s0, int64_t a_s1, int64_t a_s2) {
    if (ne12 > 65535 || (M + SM - 1) / SM > 65535 || (a_s0 != 1 && a_s1 != 1)) return false;
    const dim3 grid((N + SN - 1) / SN, (M + SM - 1) / SM, ne12);
    if (a_s0 == 1)
        hipLaunchKernelGGL((gemm_f32_mfma<AT, true>), grid, dim3(256), 0, ctx->stream, a, b, dst, K, N, M, ne12 / ne02, a_s0,
                           a_s1, a_s2);
    else
        hipLaunchKernelGGL((gemm_f32_mfma<AT, false>), grid, dim3(256), 0, ctx->stream, a, b, dst, K, N, M, ne12 / ne02, a_s0,
                           a_s1, a_s2);
    return true;
}
template bool gh_mul_mat_f32_mfma<float>(galois_hip_ctx *, const float *, const float *, float *, int, int, int, int, int,
                                         int64_t, int64_t, int64_t);
template bool gh_mul_mat_f32_mfma<_Float16>(galois_hip_ctx *, const _Float16 *, const float *, float *, int, int, int, int,
                                            int, int64_t, int64_t, int64_t);
