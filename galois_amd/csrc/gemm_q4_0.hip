// Q4_0 x f32 batched matmul for prefill on gfx950 MFMA.
//
// Replaces quantize_q8_1 + mul_mat_q4_0 (galois-kernels/src/matmul.cu:133-174,452-504;
// launcher src/cuda.rs:1035-1136).  Y[m*N + n] = sum_k deq(W)[n,k] * X[m*K + k].
// W tiles are dequantised to fp16 and X tiles rounded to fp16 on their way into LDS;
// v_mfma_f32_32x32x16_f16 accumulates in f32.
#include "common.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128;
constexpr int LDS_STRIDE = 40;  // halfs per tile row: 80-byte rows keep 16-byte fragment reads conflict-free

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    half2_t h;
    h.x = (_Float16)a;
    h.y = (_Float16)b;
    return __builtin_bit_cast(uint32_t, h);
}

// (1024 + n) as f16 for the nibble pairs selected by `mask` position, minus 1032, times d:
// exact (n - 8) * d rounded once to f16 -- d is f16 and |n-8| <= 8, so the product needs at most
// 11 + 4 significant bits and is rounded to the 11 that f16 keeps.
__device__ __forceinline__ uint32_t deq_pair(uint32_t bits, half2_t d2) {
    const half2_t magic = __builtin_bit_cast(half2_t, (bits & 0x000F000Fu) | 0x64006400u);
    const half2_t off = {(_Float16)1032.0f, (_Float16)1032.0f};
    return __builtin_bit_cast(uint32_t, (magic - off) * d2);
}

__global__ __launch_bounds__(256) void gemm_q4_0_mfma_v1(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                          float *__restrict__ Y, int K, int N, int M) {
    __shared__ __attribute__((aligned(16))) _Float16 As[TM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 Bs[TN * LDS_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const int nb = K / 32;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // staging roles: thread -> (tile row, half of the 32-wide k slice)
    const int srow = tid >> 1, shalf = tid & 1;
    const int xm = min(m0 + srow, M - 1);
    const int wn_row = min(n0 + srow, N - 1);
    const float *xp = X + (size_t)xm * K + shalf * 16;
    const uint16_t *wp = reinterpret_cast<const uint16_t *>(W + (size_t)wn_row * nb * 18);

    for (int kb = 0; kb < nb; kb++) {
        // ---- X tile: 16 floats -> 16 halfs
        {
            const float4 *p = reinterpret_cast<const float4 *>(xp + (size_t)kb * 32);
            const float4 a = p[0], b = p[1], c = p[2], d = p[3];
            uint4 lo, hi;
            lo.x = pack_h2(a.x, a.y), lo.y = pack_h2(a.z, a.w), lo.z = pack_h2(b.x, b.y), lo.w = pack_h2(b.z, b.w);
            hi.x = pack_h2(c.x, c.y), hi.y = pack_h2(c.z, c.w), hi.z = pack_h2(d.x, d.y), hi.w = pack_h2(d.z, d.w);
            uint4 *dst = reinterpret_cast<uint4 *>(As + srow * LDS_STRIDE + shalf * 16);
            dst[0] = lo;
            dst[1] = hi;
        }
        // ---- W tile: bytes qs[8h .. 8h+8) of block (row, kb): low nibbles are k = 8h+i, high nibbles k = 16+8h+i
        {
            const uint16_t *bp = wp + (size_t)kb * 9;
            const _Float16 d = __builtin_bit_cast(_Float16, bp[0]);
            const half2_t d2 = {d, d};
            const uint32_t q0 = (uint32_t)bp[1 + shalf * 4] | ((uint32_t)bp[2 + shalf * 4] << 16);  // bytes 8h..8h+3
            const uint32_t q1 = (uint32_t)bp[3 + shalf * 4] | ((uint32_t)bp[4 + shalf * 4] << 16);  // bytes 8h+4..8h+7
            // byte order inside a dword: b0 b1 b2 b3 -> pairs (b0,b2) and (b1,b3); un-interleave with a byte perm first
            const uint32_t e0 = __builtin_amdgcn_perm(0, q0, 0x03010200u);  // b0 b2 b1 b3
            const uint32_t e1 = __builtin_amdgcn_perm(0, q1, 0x03010200u);
            // e: byte0=b0, byte1=b2, byte2=b1, byte3=b3.  (e & 0x000F000F) = (b0.lo, b1.lo); (e>>8) = (b2.lo, b3.lo)
            uint4 lo, hi;
            lo.x = deq_pair(e0, d2), lo.y = deq_pair(e0 >> 8, d2), lo.z = deq_pair(e1, d2), lo.w = deq_pair(e1 >> 8, d2);
            hi.x = deq_pair(e0 >> 4, d2), hi.y = deq_pair(e0 >> 12, d2), hi.z = deq_pair(e1 >> 4, d2),
            hi.w = deq_pair(e1 >> 12, d2);
            *reinterpret_cast<uint4 *>(Bs + srow * LDS_STRIDE + shalf * 8) = lo;
            *reinterpret_cast<uint4 *>(Bs + srow * LDS_STRIDE + 16 + shalf * 8) = hi;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            half8_t a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                a[i] = *reinterpret_cast<const half8_t *>(As + (wm * 64 + i * 32 + (lane & 31)) * LDS_STRIDE + ks * 16 +
                                                          (lane >> 5) * 8);
#pragma unroll
            for (int j = 0; j < 2; j++)
                b[j] = *reinterpret_cast<const half8_t *>(Bs + (wn * 64 + j * 32 + (lane & 31)) * LDS_STRIDE + ks * 16 +
                                                          (lane >> 5) * 8);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // C layout of the 32x32 MFMA: column = lane % 32, row = 8*(e/4) + 4*(lane/32) + e%4
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m < M && n < N) Y[(size_t)m * N + n] = acc[i][j][e];
            }
        }
}

}  // namespace

extern "C" int32_t galois_hip_mul_mat_q4_0_f32(galois_hip_ctx *ctx, const void *W, const float *X, float *Y,
                                               int32_t K, int32_t N, int32_t M) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, W && X && Y, GALOIS_HIP_E_NULL, "mul_mat_q4_0_f32");
    GH_REQUIRE(ctx, K > 0 && N > 0 && M > 0 && K % 32 == 0, GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_f32: K must be a positive multiple of 32, N and M positive");
    GH_REQUIRE(ctx, gh_aligned(W, 2) && gh_aligned(X, 16) && gh_aligned(Y, 4), GALOIS_HIP_E_ALIGN,
               "mul_mat_q4_0_f32: W 2-byte, X 16-byte, Y 4-byte aligned");
    GH_BIND(ctx);
    const dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
    hipLaunchKernelGGL(gemm_q4_0_mfma_v1, grid, dim3(256), 0, ctx->stream, (const uint8_t *)W, X, Y, K, N, M);
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_f32 launch");
}
