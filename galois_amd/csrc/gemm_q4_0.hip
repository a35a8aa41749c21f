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

constexpr int TM = 128, TN = 128;  // tile of the generic kernel
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

// ---------------------------------------------------------------------------------------
// Main kernel: K % 256 == 0, W and X 16-byte aligned.
//
//   - X is rounded to fp16 once by f32_to_f16_tiles into a context-owned workspace, stored in the
//     order the A operand of v_mfma_f32_16x16x32_f16 is held (per lane 8 consecutive k of one row),
//     so a fragment is one contiguous KB: the consumer waves fetch their A fragments straight from
//     global memory (the 4 MB panel stays in L2) two stages ahead, and X never touches LDS.
//   - Workgroup tile 256 (M) x 96 (N), k-stage 64 (two Q4_0 blocks = one 36-byte slot per weight
//     row).  The 512 x 11008 prefill is 2 x 115 = 230 workgroups: one round on 256 CUs.
//   - 8 waves: 4 consumers stacked in M, wave tile 64 x 96 -> 4 x 6 MFMA tiles with f32 accumulators
//     in registers, and 4 producers that fetch the weights as whole 144-byte row pieces (4 stages at
//     a time), park them raw in LDS, and each stage dequantise one slot per row into an fp16 B tile
//     that all four consumers read.  Each SIMD hosts one wave of each kind.
//     For narrow matrices the tile is 256 x 48 (3 MFMA tiles per wave in N): N = 4096 at M = 512 is 86
//     workgroups of 96 columns but 172 of 48.
//   - The fp16 B tile is triple-buffered, one barrier per stage: while the consumers multiply the
//     second k-half of stage s they already hold the first half of stage s+1, and the producers
//     write stage s+2.  LDS carries only B.
//   - A consumer wave has a single instruction stream, so whatever blocks it idles its SIMD's matrix
//     pipe: its A requests and B fragment reads are issued one or two at a time between groups of
//     six matrix instructions instead of in bursts.
//   - blockIdx is mapped so that an XCD (blockIdx % 8) owns one 256-row panel of X and a
//     contiguous range of weight tiles: X stays in that XCD's L2, W streams once per panel.
// The N extent of the tile is a template parameter: 96 columns (6 MFMA tiles per consumer wave) for wide
// matrices, 48 (3 per wave) when 96 would leave most CUs without a workgroup (N = 4096 at M = 512: 86 tiles).
constexpr int GM = 256;
constexpr int GBSTRIDE = 80;                  // halfs per B row in LDS: 160-byte rows
constexpr int GNBUF = 3;
constexpr int GRAW_STRIDE = 144;              // raw bytes per tile row per super-stage (4 slots)
template <int GN>
struct gemm_cfg {
    static constexpr int TASKS = (GN * 4 + 255) / 256;  // dequantisation tasks per producer thread and stage
    static constexpr int B_HALFS = GN * GBSTRIDE;       // halfs per stage buffer (15,360 B for 96 columns)
    static constexpr int RAW_BYTES = GN * GRAW_STRIDE;  // bytes per raw buffer (13,824 B for 96 columns)
    static constexpr int RAW_CHUNKS = GN * 9;           // 16-byte chunks per raw buffer
    static constexpr int RAW_PER_THREAD = (RAW_CHUNKS + 255) / 256;
    static constexpr size_t LDS_BYTES = (size_t)GNBUF * B_HALFS * sizeof(_Float16) + 2 * (size_t)RAW_BYTES + 16;
};
typedef float float4_t __attribute__((ext_vector_type(4)));

// X -> fp16 in the order the MFMA A operand is fetched ("the panel"): tiles of 16 rows x 32 k (1 KB), tile (m16, kb)
// at ((m16 * K/32) + kb) * 1 KB, and inside a tile the 16-byte run k = kb*32 + kg*8 .. +7 of row
// m16*16 + r at (kg * 16 + r) * 16 bytes.  Lane l = kg * 16 + r of a wave owns exactly that run in
// v_mfma_f32_16x16x32_f16, so a fragment load is 64 consecutive 16-byte pieces: one contiguous KB.
// Rows past M (the last tile of a ragged M) are written as zeros.
// SWIGLU: the panel receives silu(x) * up instead of x (silu_f32 then mul_f32, unary.cu:1-10, mul.cu:3-12, with the
// arithmetic of galois_hip_silu_mul_f32), so that a down projection needs neither that launch nor the conversion.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void f32_to_f16_tiles(const float *__restrict__ x, const float *__restrict__ up,
                                                        _Float16 *__restrict__ y, int M, int K, int64_t nchunks) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;  // 16-byte output chunk
    if (o >= nchunks) return;
    const int64_t tile = o >> 6;
    const int c = (int)(o & 63), kg = c >> 4, r = c & 15;
    const int kblocks = K / 32;
    const int64_t m16 = tile / kblocks;
    const int kb = (int)(tile - m16 * kblocks);
    const int64_t m = m16 * 16 + r;
    uint4 out = make_uint4(0, 0, 0, 0);
    if (m < M) {
        const float4 *src = reinterpret_cast<const float4 *>(x + m * K + kb * 32 + kg * 8);
        float4 a = src[0], b = src[1];
        if (SWIGLU) {
            const float4 *us = reinterpret_cast<const float4 *>(up + m * K + kb * 32 + kg * 8);
            const float4 ua = us[0], ub = us[1];
            a = make_float4(a.x / (1.0f + expf(-a.x)) * ua.x, a.y / (1.0f + expf(-a.y)) * ua.y,
                            a.z / (1.0f + expf(-a.z)) * ua.z, a.w / (1.0f + expf(-a.w)) * ua.w);
            b = make_float4(b.x / (1.0f + expf(-b.x)) * ub.x, b.y / (1.0f + expf(-b.y)) * ub.y,
                            b.z / (1.0f + expf(-b.z)) * ub.z, b.w / (1.0f + expf(-b.w)) * ub.w);
        }
        out.x = pack_h2(a.x, a.y), out.y = pack_h2(a.z, a.w), out.z = pack_h2(b.x, b.y), out.w = pack_h2(b.z, b.w);
    }
    reinterpret_cast<uint4 *>(y)[o] = out;
}

// rms_norm(x, eps) * weight (rms_norm.cu:13-49 then mul.cu:3-12) written straight into the panel: one workgroup per
// row, the row in registers (NV runs of eight values per thread), the arithmetic of galois_hip_rms_norm_mul_f32
// ((x * scale) * weight, rounded to fp16 at the end).  A thread's run is one 16-byte piece of the panel; the sixteen
// rows of a tile group are given to workgroups of one XCD (blockIdx % 8), so that the pieces of a line meet in
// one L2 before they are written back.
// SUM: the row is x + xb + xc first (xb, xc may be null; added in that order, as gemm_sum_pass adds two shares of k
// and a residual), and that sum is also written to xsum as f32 (xsum may be any of the three inputs: a thread reads
// its own elements before it writes them) -- the adding pass behind a product and the norm in front of the next one
// as one launch.
constexpr int kPanelNormThreads = 512;
template <int NV, bool SUM = false>
__global__ __launch_bounds__(kPanelNormThreads) void rms_norm_to_f16_tiles(const float *x, const float *__restrict__ w,
                                                                            _Float16 *__restrict__ y, int M, int K, float eps,
                                                                            int groups, int groups_per_xcd, const float *xb = nullptr,
                                                                            const float *xc = nullptr, float *xsum = nullptr) {
    constexpr int THREADS = kPanelNormThreads;
    __shared__ float part[THREADS / 64];
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int grp = xcd * groups_per_xcd + (j >> 4), r = j & 15;
    if (grp >= groups) return;
    const int m = grp * 16 + r;
    const bool live = m < M;  // rows past M are zeros in the panel
    const int nrun = K >> 3;
    float4 v[NV][2], g[NV][2];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = threadIdx.x + i * THREADS;
        const bool ok = live && c < nrun;
        const size_t at = (size_t)(live ? m : 0) * K + 8 * (size_t)(ok ? c : 0);
        const float4 *src = reinterpret_cast<const float4 *>(x + at);
        v[i][0] = ok ? src[0] : make_float4(0.f, 0.f, 0.f, 0.f);
        v[i][1] = ok ? src[1] : make_float4(0.f, 0.f, 0.f, 0.f);
        if (SUM) {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const float *more = t == 0 ? xb : xc;
                if (more && ok) {
                    const float4 p = reinterpret_cast<const float4 *>(more + at)[0], q = reinterpret_cast<const float4 *>(more + at)[1];
                    v[i][0] = make_float4(v[i][0].x + p.x, v[i][0].y + p.y, v[i][0].z + p.z, v[i][0].w + p.w);
                    v[i][1] = make_float4(v[i][1].x + q.x, v[i][1].y + q.y, v[i][1].z + q.z, v[i][1].w + q.w);
                }
            }
            if (ok) {
                __builtin_nontemporal_store(float4_t{v[i][0].x, v[i][0].y, v[i][0].z, v[i][0].w}, reinterpret_cast<float4_t *>(xsum + at));
                __builtin_nontemporal_store(float4_t{v[i][1].x, v[i][1].y, v[i][1].z, v[i][1].w}, reinterpret_cast<float4_t *>(xsum + at) + 1);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = min(threadIdx.x + i * THREADS, nrun - 1);
        g[i][0] = reinterpret_cast<const float4 *>(w)[2 * c];
        g[i][1] = reinterpret_cast<const float4 *>(w)[2 * c + 1];
    }
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
        for (int h = 0; h < 2; h++)
            ss += v[i][h].x * v[i][h].x + v[i][h].y * v[i][h].y + v[i][h].z * v[i][h].z + v[i][h].w * v[i][h].w;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < THREADS / 64; i++) tot += part[i];
    const float scale = 1.0f / sqrtf(tot / (float)K + eps);
    const size_t tile_row = (size_t)grp * (K >> 5);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = threadIdx.x + i * THREADS;
        if (c < nrun) {
            const float4 a = v[i][0], b = v[i][1], ga = g[i][0], gb = g[i][1];
            uint4 out;
            out.x = pack_h2((a.x * scale) * ga.x, (a.y * scale) * ga.y), out.y = pack_h2((a.z * scale) * ga.z, (a.w * scale) * ga.w);
            out.z = pack_h2((b.x * scale) * gb.x, (b.y * scale) * gb.y), out.w = pack_h2((b.z * scale) * gb.z, (b.w * scale) * gb.w);
            reinterpret_cast<uint4 *>(y)[(tile_row + (c >> 2)) * 64 + (c & 3) * 16 + r] = out;
        }
    }
}

// Four nibble bytes (one dword of qs) -> 4 + 4 fp16 weights:
// lo[0..1] = bytes 0..3 low nibbles (k = 4j .. 4j+3), hi[0..1] = high nibbles (k = 16+4j ..).
// (1024 + n) - 1032 is the exact integer n - 8; the product with d is rounded once.
__device__ __forceinline__ void deq_dword(uint32_t v, half2_t d2, uint32_t lo[2], uint32_t hi[2]) {
    const uint32_t l = v & 0x0F0F0F0Fu, h = (v >> 4) & 0x0F0F0F0Fu;
    const uint32_t magic = 0x64646464u;  // 0x64nn as fp16 is 1024 + nn
    const half2_t off = {(_Float16)1032.0f, (_Float16)1032.0f};
    // v_perm_b32 selectors: bytes 0..3 = second operand (nibbles), 4..7 = first operand (magic)
    const half2_t l01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(magic, l, 0x04010400u));
    const half2_t l23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(magic, l, 0x04030402u));
    const half2_t h01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(magic, h, 0x04010400u));
    const half2_t h23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(magic, h, 0x04030402u));
    lo[0] = __builtin_bit_cast(uint32_t, (l01 - off) * d2);
    lo[1] = __builtin_bit_cast(uint32_t, (l23 - off) * d2);
    hi[0] = __builtin_bit_cast(uint32_t, (h01 - off) * d2);
    hi[1] = __builtin_bit_cast(uint32_t, (h23 - off) * d2);
}

// ---- producer side ---------------------------------------------------------------------
// The weights are fetched four stages at a time as the 144 contiguous bytes (8 blocks) each
// tile row contributes: nine consecutive lanes read one row piece with 16-byte loads, so every
// request is made of whole lines.  The pieces are parked as raw bytes in LDS.

// Global loads whose use is a loop iteration (or four) away are issued through inline assembly and
// waited for by hand: loads retire in order, so "at most n younger loads outstanding" is the exact
// condition for an older one to have landed, whereas the compiler waits for such loads with vmcnt(0)
// right where they are issued (or parks them in scratch memory).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void gload16(u32x4_t &dst, const void *ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
}
#define GEMM_VMWAIT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")

// Up to GEMM_MAX_MATS weight matrices against the same panel in one launch (q | k | v, gate | up).  Their rows (the
// columns of the results) are numbered through as one concatenated matrix and tiled as such -- a tile may end in one
// matrix and go on in the next -- so three matrices of 4096 rows are exactly 128 tiles of 96 columns per 256-row
// panel: 256 workgroups at M = 512, where each of them alone has 86 (or 172 of 48 columns) for 256 CUs.
constexpr int GEMM_MAX_MATS = 4;
struct gemm_mats {
    const uint8_t *W[GEMM_MAX_MATS];
    float *Y[GEMM_MAX_MATS];
    int32_t N[GEMM_MAX_MATS];
    int32_t col0[GEMM_MAX_MATS];  // first concatenated column of each matrix; unused entries hold INT_MAX
    int32_t n_total;              // columns of the concatenation
    // SwiGLU pairing (96-column tiles only): W[0] = gate, W[1] = up, both N[0] rows.  Tile t holds rows 48 t .. 48 t + 47
    // of the gate matrix in its first 48 columns and the same rows of the up matrix in its last 48, so a consumer wave
    // has both products of an element in its registers and stores silu(gate) * up, as fp16, into the panel of the
    // [N[0], M] operand at swiglu_out.  n_total = 96 * ceil(N[0] / 48) then.
    _Float16 *swiglu_out;
};

// Row `c` of the concatenated weights (clamped to the last one): its bytes.
__device__ __forceinline__ const uint8_t *gemm_w_row(const gemm_mats &mats, int c, size_t wrow_bytes) {
    if (mats.swiglu_out) {
        const int t = c / 96, sub = c - t * 96, up = sub >= 48;
        const int r = min(t * 48 + sub - 48 * up, mats.N[0] - 1);
        return mats.W[up] + (size_t)r * wrow_bytes;
    }
    c = min(c, mats.n_total - 1);
    const uint8_t *W = mats.W[0];
    int first = 0;
#pragma unroll
    for (int j = 1; j < GEMM_MAX_MATS; j++) {
        const bool ge = c >= mats.col0[j];
        W = ge ? mats.W[j] : W, first = ge ? mats.col0[j] : first;
    }
    return W + (size_t)(c - first) * wrow_bytes;
}

template <int GN>
struct gemm_raw_regs {
    u32x4_t c[gemm_cfg<GN>::RAW_PER_THREAD];
};

// rowp[i]: where the thread's i-th 16-byte chunk of a piece lies in the first piece of its weight row (the row and
// the chunk are the same for every piece, so the matrix lookup happens once).
template <int GN>
__device__ __forceinline__ void gemm_raw_rows(const gemm_mats &mats, size_t wrow_bytes, int n0, int p,
                                              const uint8_t *(&rowp)[gemm_cfg<GN>::RAW_PER_THREAD]) {
#pragma unroll
    for (int i = 0; i < gemm_cfg<GN>::RAW_PER_THREAD; i++) {
        const int q = min(p + 256 * i, gemm_cfg<GN>::RAW_CHUNKS - 1);
        const int row = q / 9, c = q - row * 9;
        rowp[i] = gemm_w_row(mats, n0 + row, wrow_bytes) + c * 16;
    }
}

template <int GN>
__device__ __forceinline__ void gemm_load_raw(const uint8_t *const (&rowp)[gemm_cfg<GN>::RAW_PER_THREAD], int super,
                                              gemm_raw_regs<GN> &r) {
#pragma unroll
    for (int i = 0; i < gemm_cfg<GN>::RAW_PER_THREAD; i++) gload16(r.c[i], rowp[i] + (size_t)super * GRAW_STRIDE);
}

template <int GN>
__device__ __forceinline__ void gemm_store_raw(uint8_t *raw, int p, const gemm_raw_regs<GN> &r) {
#pragma unroll
    for (int i = 0; i < gemm_cfg<GN>::RAW_PER_THREAD; i++) {
        const int q = p + 256 * i;
        if (q < gemm_cfg<GN>::RAW_CHUNKS) *reinterpret_cast<u32x4_t *>(raw + q * 16) = r.c[i];
    }
}

// One stage of B: slot J (36 bytes) of every tile row out of a raw buffer, as 4 tasks per row:
// task (b, jp) = eight nibble bytes qs[8*jp .. 8*jp+7] of block b -> the 16-byte run k = 32b + 8jp ..
// (low nibbles) and the run k = 32b + 16 + 8jp .. (high nibbles).  The four lanes of a row write
// 64 distinct bytes per store and neighbouring rows are 160 bytes apart, so the 16-byte stores of
// eight consecutive lanes fall into 32 different banks.
// The raw bytes of a stage are read from LDS one stage ahead (gemm_stage_read) and turned into fp16
// after the barrier (gemm_stage_write), so that the read latency is not on the path between two barriers.
template <int GN>
struct gemm_stage_regs {
    uint32_t dbits[gemm_cfg<GN>::TASKS], w0[gemm_cfg<GN>::TASKS], w1[gemm_cfg<GN>::TASKS], w2[gemm_cfg<GN>::TASKS];
};

template <int J, int GN>
__device__ __forceinline__ void gemm_stage_read(gemm_stage_regs<GN> &r, const uint8_t *raw, int p) {
#pragma unroll
    for (int it = 0; it < gemm_cfg<GN>::TASKS; it++) {
        const int q = p + 256 * it;
        if ((it + 1) * 256 <= GN * 4 || q < GN * 4) {
            const int row = q >> 2, b = (q >> 1) & 1, jp = q & 1;
            const int o = row * GRAW_STRIDE + 36 * J + 18 * b;  // the block: d at o, qs at o + 2
            r.dbits[it] = *reinterpret_cast<const uint16_t *>(raw + o);
            const int qo = o + 2 + 8 * jp;                       // 4-byte aligned for b = 1, 2 mod 4 for b = 0
            const uint32_t *w = reinterpret_cast<const uint32_t *>(raw + (qo & ~3));
            r.w0[it] = w[0], r.w1[it] = w[1], r.w2[it] = w[2];   // w2 of the very last task lies in the 16-byte pad
        }
    }
}

template <int GN>
__device__ __forceinline__ void gemm_stage_write(const gemm_stage_regs<GN> &r, _Float16 *Bs, int p) {
#pragma unroll
    for (int it = 0; it < gemm_cfg<GN>::TASKS; it++) {
        const int q = p + 256 * it;
        if ((it + 1) * 256 <= GN * 4 || q < GN * 4) {
            const int row = q >> 2, b = (q >> 1) & 1, jp = q & 1;
            const uint32_t sh = b ? 0u : 16u;
            const uint32_t q0 = __builtin_amdgcn_alignbit(r.w1[it], r.w0[it], sh);
            const uint32_t q1 = __builtin_amdgcn_alignbit(r.w2[it], r.w1[it], sh);
            const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t)r.dbits[it]);
            const half2_t d2 = {d, d};
            uint32_t lo[4], hi[4];
            deq_dword(q0, d2, lo, hi);
            deq_dword(q1, d2, lo + 2, hi + 2);
            _Float16 *dst = Bs + row * GBSTRIDE + 32 * b + 8 * jp;
            *reinterpret_cast<uint4 *>(dst) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            *reinterpret_cast<uint4 *>(dst + 16) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        }
    }
}

// Barrier protocol (both kinds of wave meet every one): R after the first raw piece is parked,
// then barrier t after stage t is written, for t = 0 .. nslots-1.  Stage t goes to buffer t % 3.
template <int GN>
__device__ __forceinline__ void gemm_producer(_Float16 *smem, const gemm_mats &mats, int K, int n0, int sup0, int nsuper) {
    constexpr int GB_HALFS = gemm_cfg<GN>::B_HALFS, GRAW_BYTES = gemm_cfg<GN>::RAW_BYTES;
    const int p = threadIdx.x - 256;
    // the workgroup's share of k: pieces sup0 .. sup0 + nsuper - 1 of 256 weights (four stages) of every row
    const size_t wrow_bytes = (size_t)(K / 64) * 36;
    uint8_t *raw0 = reinterpret_cast<uint8_t *>(smem + GNBUF * GB_HALFS);
    uint8_t *raw1 = raw0 + GRAW_BYTES;

    gemm_raw_regs<GN> rr;
    const uint8_t *rowp[gemm_cfg<GN>::RAW_PER_THREAD];
    gemm_raw_rows<GN>(mats, wrow_bytes, n0, p, rowp);
#pragma unroll
    for (int i = 0; i < gemm_cfg<GN>::RAW_PER_THREAD; i++) rowp[i] += (size_t)sup0 * GRAW_STRIDE;
    gemm_load_raw<GN>(rowp, 0, rr);
    GEMM_VMWAIT(0);
    gemm_store_raw(raw0, p, rr);
    gemm_load_raw<GN>(rowp, min(1, nsuper - 1), rr);
    __syncthreads();  // R
    gemm_stage_regs<GN> s0, s1;
    gemm_stage_read<0>(s0, raw0, p);
    for (int sup = 0; sup < nsuper; sup++) {
        const uint8_t *raw = (sup & 1) ? raw1 : raw0;
        uint8_t *other = (sup & 1) ? raw0 : raw1;
        const int t = 4 * sup;
        gemm_stage_read<1>(s1, raw, p);
        gemm_stage_write(s0, smem + (t % GNBUF) * GB_HALFS, p);
        __syncthreads();
        gemm_stage_read<2>(s0, raw, p);
        gemm_stage_write(s1, smem + ((t + 1) % GNBUF) * GB_HALFS, p);
        __syncthreads();
        gemm_stage_read<3>(s1, raw, p);
        gemm_stage_write(s0, smem + ((t + 2) % GNBUF) * GB_HALFS, p);
        // park the next piece (requested four stages ago) in the other raw buffer, whose last readers
        // passed a barrier three stages ago, and request the one after it
        GEMM_VMWAIT(0);
        gemm_store_raw(other, p, rr);
        gemm_load_raw<GN>(rowp, min(sup + 2, nsuper - 1), rr);
        __syncthreads();
        gemm_stage_read<0>(s0, other, p);  // the next piece's first stage (read again, unused, after the last piece)
        gemm_stage_write(s1, smem + ((t + 3) % GNBUF) * GB_HALFS, p);
        __syncthreads();
    }
    // The last request is never consumed.  To the compiler an inline-asm load defines its destination at
    // once, so a dead destination could be handed to another value while the load is still in flight and
    // be overwritten when it lands.  Drain, then name every register so all stay allocated until here.
    GEMM_VMWAIT(0);
#pragma unroll
    for (int i = 0; i < gemm_cfg<GN>::RAW_PER_THREAD; i++) asm volatile("" ::"v"(rr.c[i]));
}

// ---- consumer side -----------------------------------------------------------------------
// The A fragments are requested through inline assembly and waited for by hand.  Loads retire in
// order, so "at most n younger loads outstanding" is the exact condition for an older one to have
// landed; left to the compiler, a load whose use is a loop iteration away is waited for with
// vmcnt(0), which would also drain the prefetches just issued.
struct gemm_a_regs {
    u32x4_t c[8];  // [ks * 4 + i]: rows i*16 + lane%16 of the wave's 64, k = ks*32 + (lane/16)*8 ..
};

// One fragment.  Address = scalar base xs (the panel advanced to the stage: 2 KB per stage) + per-lane
// 32-bit offset ro of the lane's piece in the first k-block of its 16-row group + immediate (second
// k-block, kh = 1: + 1 KB).
__device__ __forceinline__ void gemm_load_a1(u32x4_t &dst, const _Float16 *xs, uint32_t ro, int kh) {
    if (kh == 0)
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(ro), "s"(xs) : "memory");
    else
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(dst) : "v"(ro), "s"(xs) : "memory");
}

// Drains the load counter; naming the registers keeps all of them allocated until here.
#define GEMM_DRAIN_A(r)                                                                                      \
    asm volatile("s_waitcnt vmcnt(0)"                                                                        \
                 : "+v"((r).c[0]), "+v"((r).c[1]), "+v"((r).c[2]), "+v"((r).c[3]), "+v"((r).c[4]), "+v"((r).c[5]), \
                   "+v"((r).c[6]), "+v"((r).c[7])::"memory")

#define GEMM_LDB(dst, ptr) dst = *reinterpret_cast<const half8_t *>(ptr)
#define GEMM_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0)
template <int NF, int GN>
__device__ __forceinline__ void gemm_consumer(const _Float16 *smem, const _Float16 *__restrict__ Xh,
                                              const gemm_mats &mats, int K, int M, int m0, int n0, int wm, int ncol0,
                                              int nslots, size_t y_off) {
    // Xh: the panel advanced to the workgroup's first k-block; nslots: its stages; y_off: where its results go,
    // relative to Y (a workgroup that holds one share of k of several writes a partial result)
    constexpr int GB_HALFS = gemm_cfg<GN>::B_HALFS;
    const int lane = threadIdx.x & 63;
    float4_t acc[4][NF];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < NF; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    uint32_t ro[4];  // byte offsets in the tiled panel (the host checks that the panel is below 4 GB)
    const int m16_last = (M + 15) / 16 - 1;
#pragma unroll
    for (int i = 0; i < 4; i++)
        ro[i] = (uint32_t)min(m0 / 16 + wm * 4 + i, m16_last) * (uint32_t)(K / 32) * 1024u + lane * 16u;
    const int b_off = (ncol0 + (lane & 15)) * GBSTRIDE + (lane >> 4) * 8;

    // Stages of A fragments in flight: two for the wide tile (its accumulators leave room for no more), four for the
    // narrow one, whose stages are short enough to run into the latency of the requests (measured: 512 x 11008 x 4096
    // 70.7 -> 69.4 us, 512 x 4096 x 4096 31.4 -> 31.2 us).
    constexpr int DEPTH = (NF <= 3) ? 4 : 2;
    gemm_a_regs a0, a1, a2, a3;
    // requested in the order they are used: the waits below count younger requests
#pragma unroll
    for (int g = 0; g < 8; g++) gemm_load_a1(a0.c[g], Xh, ro[g & 3], g >> 2);
#pragma unroll
    for (int g = 0; g < 8; g++) gemm_load_a1(a1.c[g], Xh + 1024, ro[g & 3], g >> 2);
    if (DEPTH == 4) {
#pragma unroll
        for (int g = 0; g < 8; g++) gemm_load_a1(a2.c[g], Xh + 2048, ro[g & 3], g >> 2);
#pragma unroll
        for (int g = 0; g < 8; g++) gemm_load_a1(a3.c[g], Xh + 3072, ro[g & 3], g >> 2);
    }
    half8_t b0[NF], b1[NF];
    __syncthreads();  // R
    __syncthreads();  // stage 0 written
#pragma unroll
    for (int j = 0; j < NF; j++) GEMM_LDB(b0[j], smem + b_off + j * 16 * GBSTRIDE);

    // One stage = eight groups of NF matrix instructions; group g multiplies A fragment g (rows
    // (g % 4) * 16 .., k-half g / 4) of AC with the B fragments of that k-half, then requests the same
    // fragment of the stage DEPTH stages on into the registers it has just consumed.  The requests are spread
    // over the stage so that the four waves never queue more than the memory pipe takes without blocking
    // the issue of the matrix instructions; a fragment is needed 8 * DEPTH groups after its request, with
    // 8 * DEPTH - 1 younger requests outstanding.
    // The B reads are spread the same way: the second k-half of this stage during groups 0..2, the
    // first k-half of the next stage (after the barrier that publishes it) during groups 4..6.
    // cur / nxt are the LDS offsets of this stage's and the next stage's B buffers.
    int cur = b_off, nxt = b_off + GB_HALFS;
    constexpr int BPG = (NF + 2) / 3;  // B fragment reads per group
#define GEMM_GROUP(G, AC, BV)                                                                              \
    {                                                                                                      \
        if (DEPTH == 4) asm volatile("s_waitcnt vmcnt(31)" : "+v"((AC).c[G])::"memory");                   \
        else asm volatile("s_waitcnt vmcnt(15)" : "+v"((AC).c[G])::"memory");                              \
        __builtin_amdgcn_sched_barrier(0);                                                                 \
        _Pragma("unroll") for (int j = 0; j < NF; j++) acc[(G) & 3][j] =                                   \
            GEMM_MFMA(__builtin_bit_cast(half8_t, (AC).c[G]), BV[j], acc[(G) & 3][j]);                     \
        __builtin_amdgcn_sched_barrier(0);                                                                 \
        gemm_load_a1((AC).c[G], xs_next, ro[(G) & 3], (G) >> 2);                                           \
    }
#define GEMM_BREADS(G3, DST, OFF)                                                                          \
    _Pragma("unroll") for (int j = (G3) * BPG; j < NF && j < ((G3) + 1) * BPG; j++)                        \
        GEMM_LDB(DST[j], smem + (OFF) + j * 16 * GBSTRIDE);
#define GEMM_STAGE(S, AC, LAST)                                                                            \
    {                                                                                                      \
        const _Float16 *xs_next = Xh + min((S) + DEPTH, nslots - 1) * 1024;                                \
        GEMM_BREADS(0, b1, cur + 32) GEMM_GROUP(0, AC, b0)                                                 \
        GEMM_BREADS(1, b1, cur + 32) GEMM_GROUP(1, AC, b0)                                                 \
        GEMM_BREADS(2, b1, cur + 32) GEMM_GROUP(2, AC, b0)                                                 \
        GEMM_GROUP(3, AC, b0)                                                                              \
        if (!(LAST)) {                                                                                     \
            __syncthreads(); /* stage S+1 written */                                                           \
            GEMM_BREADS(0, b0, nxt)                                                                        \
        }                                                                                                  \
        GEMM_GROUP(4, AC, b1)                                                                              \
        if (!(LAST)) { GEMM_BREADS(1, b0, nxt) }                                                           \
        GEMM_GROUP(5, AC, b1)                                                                              \
        if (!(LAST)) { GEMM_BREADS(2, b0, nxt) }                                                           \
        GEMM_GROUP(6, AC, b1)                                                                              \
        GEMM_GROUP(7, AC, b1)                                                                              \
        cur = nxt;                                                                                         \
        nxt = (nxt == b_off + (GNBUF - 1) * GB_HALFS) ? b_off : nxt + GB_HALFS;                            \
    }
    int s = 0;
    if (DEPTH == 4) {
        for (; s < nslots - 4; s += 4) {
            GEMM_STAGE(s, a0, false)
            GEMM_STAGE(s + 1, a1, false)
            GEMM_STAGE(s + 2, a2, false)
            GEMM_STAGE(s + 3, a3, false)
        }
        GEMM_STAGE(s, a0, false)
        GEMM_STAGE(s + 1, a1, false)
        GEMM_STAGE(s + 2, a2, false)
        GEMM_STAGE(s + 3, a3, true)
    } else {
    for (; s < nslots - 2; s += 2) {
        GEMM_STAGE(s, a0, false)
        GEMM_STAGE(s + 1, a1, false)
    }
    GEMM_STAGE(s, a0, false)
    GEMM_STAGE(s + 1, a1, true)
    }
#undef GEMM_STAGE
#undef GEMM_GROUP
#undef GEMM_BREADS
    // the last two stages requested the last stage's fragments again (never used): drain before the registers die
    GEMM_DRAIN_A(a0);
    GEMM_DRAIN_A(a1);
    if (DEPTH == 4) {
        GEMM_DRAIN_A(a2);
        GEMM_DRAIN_A(a3);
    }

    // C layout of the 16x16 MFMA: column = lane % 16, row = 4 * (lane / 16) + e.
    if (NF == 6 && mats.swiglu_out) {
        // columns j and j + 3 of the wave's tile are the gate and the up product of one output column: silu(gate) * up
        // (silu_f32 then mul_f32, unary.cu:1-10, mul.cu:3-12, with the arithmetic of f32_to_f16_tiles<true>) goes
        // to the panel as fp16: element (m, n) lies in tile (m / 16, n / 32) of 1 KB, 16-byte piece ((n % 32) / 8) * 16
        // + m % 16, at n % 8.  Rows of the panel past M were zeros in the input panel, so their products are zeros.
        // The exponential and the reciprocal are the hardware's (v_exp_f32, v_rcp_f32: about one unit in the last place
        // of f32 each, far below the fp16 rounding that follows); four neighbouring lanes hold four neighbouring
        // columns of a row, which lane % 4 == 0 gathers over the quad and stores as one 8-byte piece.
        const int N = mats.N[0], m_pad = (M + 15) & ~15;
        unsigned char *out = reinterpret_cast<unsigned char *>(mats.swiglu_out);
#pragma unroll
        for (int j = 0; j < 3; j++) {
            const int n = (n0 / 96) * 48 + j * 16 + (lane & 15);
            const size_t col_at = (size_t)(n >> 5) * 1024 + (size_t)((n & 31) >> 3) * 256 + (size_t)(n & 7) * 2;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int m = m0 + wm * 64 + i * 16 + 4 * (lane >> 4) + e;
                    const float g = acc[i][j][e], u = acc[i][j + 3 < NF ? j + 3 : j][e];
                    const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.44269504088896340736f));
                    const uint32_t h = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)((g * sig) * u));
                    // quad_perm [1,0,3,2] then [2,3,0,1]: lane 4q ends up with the four halfs of its quad in column order
                    const uint32_t pair = h | ((uint32_t)__builtin_amdgcn_update_dpp(0, (int)h, 0xB1, 0xF, 0xF, false) << 16);
                    const uint32_t pair2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)pair, 0x4E, 0xF, 0xF, false);
                    if ((lane & 3) == 0 && m < m_pad && n < N)
                        *reinterpret_cast<uint2 *>(out + (size_t)(m >> 4) * (size_t)(N >> 5) * 1024 + col_at + (size_t)(m & 15) * 16) =
                            make_uint2(pair, pair2);
                }
        }
        return;
    }
    // A lane's column lies in one of the matrices of the launch: the result goes to that matrix's Y.
#pragma unroll
    for (int j = 0; j < NF; j++) {
        const int n = n0 + ncol0 + j * 16 + (lane & 15);
        float *Y = mats.Y[0];
        int N = mats.N[0], first = 0;
#pragma unroll
        for (int t = 1; t < GEMM_MAX_MATS; t++) {
            const bool ge = n >= mats.col0[t];
            Y = ge ? mats.Y[t] : Y, N = ge ? mats.N[t] : N, first = ge ? mats.col0[t] : first;
        }
        const int nl = n - first;
        Y += y_off;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int m = m0 + wm * 64 + i * 16 + 4 * (lane >> 4) + e;
                if (m < M && n < mats.n_total) Y[(size_t)m * N + nl] = acc[i][j][e];
            }
    }
}

template <int GN>
__global__ __launch_bounds__(512) void gemm_q4_0_mfma(const gemm_mats mats, const _Float16 *__restrict__ Xh, int K, int M,
                                                      int n_tiles, int m_tiles, int splits, size_t split_stride) {
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];  // [3] B stage | [2] raw | pad
    // XCD-aware tile order: blockIdx % 8 is the XCD; consecutive tiles (same X panel, same share of k) go to one XCD
    const int total = n_tiles * m_tiles * splits;
    const int per_xcd = (total + 7) >> 3;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= total) return;
    const int mts = tile / n_tiles, nt = tile - mts * n_tiles;
    const int sp = mts / m_tiles, mt = mts - sp * m_tiles;
    const int m0 = mt * GM, n0 = nt * GN;
    // share sp of k: whole pieces of 256 (four stages), as evenly as they divide; its results lie split_stride
    // floats after the previous share's
    const int nsuper_all = K / 256;
    const int sup0 = (int)((int64_t)sp * nsuper_all / splits), sup1 = (int)((int64_t)(sp + 1) * nsuper_all / splits);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave >= 4)
        gemm_producer<GN>(smem, mats, K, n0, sup0, sup1 - sup0);
    else  // four consumer waves stacked in M, each 64 rows x GN columns; a piece of 256 is 8 KB of a row group's panel
        gemm_consumer<GN / 16, GN>(smem, Xh + (size_t)sup0 * 4096, mats, K, M, m0, n0, wave, 0, (sup1 - sup0) * 4,
                                   (size_t)sp * split_stride);
}

// The pass behind a product with a residual: y = p (+ the second share of k, stride4 float4s on, when stride4 != 0)
// (+ r), four floats per thread.  y may be p (a product already in place) or r (the residual stream updated in place):
// every thread reads its own four elements before it writes them.  Measured against adding the residual where the
// product's tiles are stored: the separate pass is faster (512 x 4096 x 11008: 58.6 against 68.0 us), since the
// tiles' scattered 4-byte reads of the residual sit at the end of every workgroup with nothing left to hide them.
__global__ __launch_bounds__(256) void gemm_sum_pass(const float4 *p, const float4 *r, float4 *y, int64_t n4, int64_t stride4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    float4 o = p[i];
    if (stride4) {
        const float4 b = p[i + stride4];
        o = make_float4(o.x + b.x, o.y + b.y, o.z + b.z, o.w + b.w);
    }
    if (r) {
        const float4 c = r[i];
        o = make_float4(o.x + c.x, o.y + c.y, o.z + c.z, o.w + c.w);
    }
    __builtin_nontemporal_store(float4_t{o.x, o.y, o.z, o.w}, reinterpret_cast<float4_t *>(y + i));
}

// The same for a result whose size is not a multiple of four floats.
__global__ __launch_bounds__(256) void gemm_sum_tail(const float *p, const float *r, float *y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = p[i] + r[i];
}

// Launch of one tile width.
template <int GN>
int32_t gemm_launch(galois_hip_ctx *ctx, const gemm_mats &mats, const _Float16 *Xh, int K, int M, int splits = 1,
                    size_t split_stride = 0) {
    const int n_tiles = (mats.n_total + GN - 1) / GN;
    const int m_tiles = (M + GM - 1) / GM;
    const int total = n_tiles * m_tiles * splits;
    const int grid = ((total + 7) / 8) * 8;
    const size_t lds = gemm_cfg<GN>::LDS_BYTES;
    // the attribute lives with the function on the current device: set per launch (a table lookup), which is right
    // for every device and every thread without any flag of our own
    hipError_t e = hipFuncSetAttribute((const void *)gemm_q4_0_mfma<GN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipFuncSetAttribute(LDS size)");
    hipLaunchKernelGGL(gemm_q4_0_mfma<GN>, dim3(grid), dim3(512), lds, ctx->stream, mats, Xh, K, M, n_tiles, m_tiles, splits,
                       split_stride);
    return GALOIS_HIP_OK;
}

// Tile width by how many workgroups it gives the device.  Cost model: rounds of workgroups over the CUs
// times the relative cost of a k-stage (a 48-column stage has half the matrix instructions and half
// the dequantisation of a 96-column one but the same barriers and A requests: ~0.65).
// Numbers the columns of the first n_mats matrices through (col0, n_total).
void gemm_concat(gemm_mats &mats, int n_mats) {
    int64_t cols = 0;
    for (int j = 0; j < GEMM_MAX_MATS; j++) {
        mats.col0[j] = j < n_mats ? (int32_t)cols : 0x7FFFFFFF;
        if (j < n_mats) cols += mats.N[j];
    }
    mats.n_total = (int32_t)cols;
}

int32_t gemm_launch_any(galois_hip_ctx *ctx, gemm_mats mats, int n_mats, const _Float16 *Xh, int K, int M) {
    gemm_concat(mats, n_mats);
    const int64_t cols = mats.n_total;
    const int64_t m_tiles = (M + GM - 1) / GM;
    const int64_t wg96 = (cols + 95) / 96 * m_tiles, wg48 = (cols + 47) / 48 * m_tiles;
    const int64_t cus = ctx->n_cu > 0 ? ctx->n_cu : 256;
    const double cost96 = (double)((wg96 + cus - 1) / cus), cost48 = 0.65 * (double)((wg48 + cus - 1) / cus);
    return cost48 < cost96 ? gemm_launch<48>(ctx, mats, Xh, K, M) : gemm_launch<96>(ctx, mats, Xh, K, M);
}

// What the main kernel asks of its operands: whole 4-stage pieces of every weight row, 16-byte requests, and a panel
// whose byte offsets fit 32 bits.
bool gemm_panel_shape_ok(int64_t K, int64_t M) { return K > 0 && M > 0 && K % 256 == 0 && (M + 16) * K * 2 < ((int64_t)1 << 32); }

int32_t launch_to_panel(galois_hip_ctx *ctx, const float *x, const float *up, _Float16 *panel, int K, int M, bool swiglu) {
    const int64_t m_pad = ((int64_t)M + 15) / 16 * 16;
    const int64_t nchunks = m_pad * K / 8;
    const dim3 grid((unsigned)((nchunks + 255) / 256)), block(256);
    if (swiglu)
        hipLaunchKernelGGL(f32_to_f16_tiles<true>, grid, block, 0, ctx->stream, x, up, panel, M, K, nchunks);
    else
        hipLaunchKernelGGL(f32_to_f16_tiles<false>, grid, block, 0, ctx->stream, x, up, panel, M, K, nchunks);
    return GALOIS_HIP_OK;
}

}  // namespace

namespace {

// Whether one matrix against the panel is better multiplied as two shares of k, each a workgroup of 64 columns, than
// as whole-k tiles: the cost model of gemm_launch_any (rounds of workgroups x cost of a stage x stages; a 64-column
// stage on a full device at 0.75 of a 96-column one) plus the pass that adds the two partial results, which costs
// about fourteen stages per 2^21 results.  Measured at M = 512 on 256 CUs: 11008 -> 4096 70.3 -> 54.8 us,
// 4096 -> 4096 32.5 -> 30.2 us (both with the residual); the shapes the model leaves whole are slower when forced
// into shares.  margin > 1 asks for a clearer win (where the adding pass replaces nothing the caller would launch anyway),
// min_cost for a product large enough that the model's neglect of fixed costs does not matter.
bool gemm_two_shares_pay(const galois_hip_ctx *ctx, int K, int N, int M, double margin = 1.0, double min_cost = 0.0) {
    const int64_t m_tiles = (M + GM - 1) / GM, cus = ctx->n_cu > 0 ? ctx->n_cu : 256, stages = K / 64;
    const int64_t wg96 = ((int64_t)N + 95) / 96 * m_tiles, wg48 = ((int64_t)N + 47) / 48 * m_tiles, wg64x2 = ((int64_t)N + 63) / 64 * m_tiles * 2;
    const int64_t mn = (int64_t)M * N;
    const double c96 = (double)((wg96 + cus - 1) / cus) * stages, c48 = 0.65 * (double)((wg48 + cus - 1) / cus) * stages;
    const double c64x2 = 0.75 * (double)((wg64x2 + cus - 1) / cus) * (stages / 2 + 2) + 14.0 * (double)mn / (double)(1 << 21);
    return K >= 512 && mn % 4 == 0 && margin * c64x2 < c96 && margin * c64x2 < c48 && c96 >= min_cost && c48 >= min_cost;
}

// W . panel into dst as one result (shares = 1) or as two partial results M * N floats apart (shares = 2).
int32_t gemm_launch_shares(galois_hip_ctx *ctx, const void *W, const _Float16 *panel, float *dst, int K, int N, int M, int shares) {
    gemm_mats mats = {};
    mats.W[0] = (const uint8_t *)W, mats.Y[0] = dst, mats.N[0] = N;
    if (shares == 1) return gemm_launch_any(ctx, mats, 1, panel, K, M);
    gemm_concat(mats, 1);
    return gemm_launch<64>(ctx, mats, panel, K, M, 2, (size_t)M * N);
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
    if (gemm_panel_shape_ok(K, M) && gh_aligned(W, 16)) {
        // fp16 copy of X, tiled for the A fragments, in the context's workspace (grown on demand); behind it, for a
        // matrix that is clearly better multiplied as two shares of k (512 x 11008 x 4096: 65 -> 47 us + a 5.7 us adding
        // pass), room for the two partial results
        const int64_t m_pad = ((int64_t)M + 15) / 16 * 16, mn = (int64_t)M * N;
        const size_t panel_bytes = ((size_t)m_pad * K * sizeof(_Float16) + 255) & ~(size_t)255;
        const bool shares = mn < ((int64_t)1 << 31) && gh_aligned(Y, 16) && gemm_two_shares_pay(ctx, K, N, M, 1.1, 64.0);
        const size_t need = panel_bytes + (shares ? 2 * (size_t)mn * sizeof(float) : 0);
        if (ctx->ws_bytes < need) {
            GH_NOT_CAPTURING(ctx, "mul_mat_q4_0_f32: growing the workspace");
            // The outgrown block is kept until the context dies: work already queued, or a graph captured earlier,
            // has its address baked in.  Growing by at least half bounds what the retired blocks add up to.
            const size_t bytes = need > ctx->ws_bytes + ctx->ws_bytes / 2 ? need : ctx->ws_bytes + ctx->ws_bytes / 2;
            void *grown = nullptr;
            const hipError_t e = hipMalloc(&grown, bytes);
            if (e != hipSuccess) return gh_hip(ctx, e, "hipMalloc(workspace)");
            if (ctx->ws) ctx->ws_retired.push_back(ctx->ws);
            ctx->ws = grown;
            ctx->ws_bytes = bytes;
        }
        _Float16 *Xh = (_Float16 *)ctx->ws;
        launch_to_panel(ctx, X, nullptr, Xh, K, M, false);
        if (shares) {
            float *parts = reinterpret_cast<float *>(static_cast<unsigned char *>(ctx->ws) + panel_bytes);
            const int32_t st = gemm_launch_shares(ctx, W, Xh, parts, K, N, M, 2);
            if (st != GALOIS_HIP_OK) return st;
            hipLaunchKernelGGL(gemm_sum_pass, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, ctx->stream,
                               reinterpret_cast<const float4 *>(parts), static_cast<const float4 *>(nullptr),
                               reinterpret_cast<float4 *>(Y), mn / 4, mn / 4);
        } else {
            const int32_t st = gemm_launch_shares(ctx, W, Xh, Y, K, N, M, 1);
            if (st != GALOIS_HIP_OK) return st;
        }
    } else {
        const dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
        hipLaunchKernelGGL(gemm_q4_0_mfma_v1, grid, dim3(256), 0, ctx->stream, (const uint8_t *)W, X, Y, K, N, M);
    }
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_f32 launch");
}

// ---- the panel as an operand of its own: producers that write it, and the matmul that takes it ----

extern "C" int32_t galois_hip_f16_panel_bytes(int32_t K, int32_t M, int64_t *bytes) {
    if (!bytes) return GALOIS_HIP_E_NULL;
    *bytes = 0;
    if (!gemm_panel_shape_ok(K, M)) return GALOIS_HIP_E_SHAPE;
    *bytes = ((int64_t)M + 15) / 16 * 16 * K * (int64_t)sizeof(_Float16);
    return GALOIS_HIP_OK;
}

static int32_t panel_args(galois_hip_ctx *ctx, const void *a, const void *b, const void *panel, int32_t K, int32_t M,
                          const char *what) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, a && b && panel, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, gemm_panel_shape_ok(K, M), GALOIS_HIP_E_SHAPE,
               "f16 panel: ncols a positive multiple of 256, nrows positive, (nrows + 16) * ncols below 2^31");
    GH_REQUIRE(ctx, gh_aligned(a, 16) && gh_aligned(b, 16) && gh_aligned(panel, 16), GALOIS_HIP_E_ALIGN,
               "f16 panel: 16-byte aligned operands");
    return GALOIS_HIP_OK;
}

extern "C" int32_t galois_hip_f32_to_f16_panel(galois_hip_ctx *ctx, const float *x, void *panel, int32_t ncols, int32_t nrows) {
    const int32_t st = panel_args(ctx, x, x, panel, ncols, nrows, "f32_to_f16_panel");
    if (st != GALOIS_HIP_OK) return st;
    GH_BIND(ctx);
    launch_to_panel(ctx, x, nullptr, (_Float16 *)panel, ncols, nrows, false);
    GH_LAUNCH_CHECK(ctx, "f32_to_f16_panel launch");
}

extern "C" int32_t galois_hip_silu_mul_f16_panel(galois_hip_ctx *ctx, const float *gate, const float *up, void *panel,
                                                 int32_t ncols, int32_t nrows) {
    const int32_t st = panel_args(ctx, gate, up, panel, ncols, nrows, "silu_mul_f16_panel");
    if (st != GALOIS_HIP_OK) return st;
    GH_BIND(ctx);
    launch_to_panel(ctx, gate, up, (_Float16 *)panel, ncols, nrows, true);
    GH_LAUNCH_CHECK(ctx, "silu_mul_f16_panel launch");
}

extern "C" int32_t galois_hip_rms_norm_mul_f16_panel(galois_hip_ctx *ctx, const float *x, const float *weight, void *panel,
                                                     int32_t ncols, int32_t nrows, float eps) {
    const int32_t st = panel_args(ctx, x, weight, panel, ncols, nrows, "rms_norm_mul_f16_panel");
    if (st != GALOIS_HIP_OK) return st;
    const int nv = (ncols / 8 + kPanelNormThreads - 1) / kPanelNormThreads;
    GH_REQUIRE(ctx, nv <= 4, GALOIS_HIP_E_SHAPE, "rms_norm_mul_f16_panel: rows of at most 16384 columns");
    GH_BIND(ctx);
    const int groups = (nrows + 15) / 16, per_xcd = (groups + 7) / 8;
    const dim3 grid((unsigned)(8 * per_xcd * 16)), block(kPanelNormThreads);
    _Float16 *y = (_Float16 *)panel;
    if (nv <= 1)
        hipLaunchKernelGGL(rms_norm_to_f16_tiles<1>, grid, block, 0, ctx->stream, x, weight, y, nrows, ncols, eps, groups, per_xcd);
    else if (nv <= 2)
        hipLaunchKernelGGL(rms_norm_to_f16_tiles<2>, grid, block, 0, ctx->stream, x, weight, y, nrows, ncols, eps, groups, per_xcd);
    else
        hipLaunchKernelGGL(rms_norm_to_f16_tiles<4>, grid, block, 0, ctx->stream, x, weight, y, nrows, ncols, eps, groups, per_xcd);
    GH_LAUNCH_CHECK(ctx, "rms_norm_mul_f16_panel launch");
}

extern "C" int32_t galois_hip_mul_mat_q4_0_f16_panel(galois_hip_ctx *ctx, const galois_hip_gemm_item *items, int32_t n_items,
                                                     const void *panel, int32_t K, int32_t M) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, items && panel, GALOIS_HIP_E_NULL, "mul_mat_q4_0_f16_panel");
    GH_REQUIRE(ctx, n_items >= 1 && n_items <= GEMM_MAX_MATS, GALOIS_HIP_E_SHAPE, "mul_mat_q4_0_f16_panel: 1 to 4 matrices per call");
    GH_REQUIRE(ctx, gemm_panel_shape_ok(K, M), GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_f16_panel: K a positive multiple of 256, M positive, (M + 16) * K below 2^31");
    GH_REQUIRE(ctx, gh_aligned(panel, 16), GALOIS_HIP_E_ALIGN, "mul_mat_q4_0_f16_panel: 16-byte aligned panel");
    gemm_mats mats = {};
    int64_t cols = 0;
    for (int j = 0; j < n_items; j++) {
        GH_REQUIRE(ctx, items[j].W && items[j].Y, GALOIS_HIP_E_NULL, "mul_mat_q4_0_f16_panel");
        GH_REQUIRE(ctx, items[j].N > 0, GALOIS_HIP_E_SHAPE, "mul_mat_q4_0_f16_panel: N positive");
        GH_REQUIRE(ctx, gh_aligned(items[j].W, 16) && gh_aligned(items[j].Y, 4), GALOIS_HIP_E_ALIGN,
                   "mul_mat_q4_0_f16_panel: W 16-byte, Y 4-byte aligned");
        mats.W[j] = (const uint8_t *)items[j].W, mats.Y[j] = items[j].Y, mats.N[j] = items[j].N;
        cols += items[j].N;
    }
    GH_REQUIRE(ctx, cols < 0x7FFFFF00 && (cols + 47) / 48 * ((M + GM - 1) / GM) < 0x7FFFFF00, GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_f16_panel: too many columns");
    GH_BIND(ctx);
    const int32_t st = gemm_launch_any(ctx, mats, n_items, (const _Float16 *)panel, K, M);
    if (st != GALOIS_HIP_OK) return st;
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_f16_panel launch");
}


// One matrix against the panel with a residual added, and the k-split shape for matrices too narrow to fill the device.
extern "C" int32_t galois_hip_mul_mat_q4_0_f16_panel_add(galois_hip_ctx *ctx, const void *W, const void *panel, const float *residual,
                                                         float *Y, int32_t K, int32_t N, int32_t M, void *workspace,
                                                         int64_t workspace_bytes) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, W && panel && Y, GALOIS_HIP_E_NULL, "mul_mat_q4_0_f16_panel_add");
    GH_REQUIRE(ctx, gemm_panel_shape_ok(K, M) && N > 0 && (int64_t)M * N < ((int64_t)1 << 31), GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_f16_panel_add: K a positive multiple of 256, (M + 16) * K below 2^31, N positive, M * N below 2^31");
    GH_REQUIRE(ctx, gh_aligned(W, 16) && gh_aligned(panel, 16) && gh_aligned(Y, 16) && gh_aligned(residual, 16) && gh_aligned(workspace, 16),
               GALOIS_HIP_E_ALIGN, "mul_mat_q4_0_f16_panel_add: 16-byte aligned operands");
    GH_REQUIRE(ctx, workspace_bytes >= 0, GALOIS_HIP_E_SHAPE, "mul_mat_q4_0_f16_panel_add: workspace_bytes");
    GH_BIND(ctx);
    const int64_t mn = (int64_t)M * N;
    const dim3 sum_grid((unsigned)((mn / 4 + 255) / 256));
    if (gemm_two_shares_pay(ctx, K, N, M) && workspace && workspace_bytes >= 2 * mn * (int64_t)sizeof(float)) {
        const int32_t st = gemm_launch_shares(ctx, W, (const _Float16 *)panel, static_cast<float *>(workspace), K, N, M, 2);
        if (st != GALOIS_HIP_OK) return st;
        hipLaunchKernelGGL(gemm_sum_pass, sum_grid, dim3(256), 0, ctx->stream, static_cast<const float4 *>(workspace),
                           reinterpret_cast<const float4 *>(residual), reinterpret_cast<float4 *>(Y), mn / 4, mn / 4);
    } else {
        // the product needs a place of its own while the residual is still to be read: Y unless Y is the residual
        float *prod = Y;
        if (residual == Y) {
            GH_REQUIRE(ctx, workspace && workspace_bytes >= mn * (int64_t)sizeof(float), GALOIS_HIP_E_UNSUPPORTED,
                       "mul_mat_q4_0_f16_panel_add: Y may be the residual only with a workspace of M * N floats or more");
            prod = static_cast<float *>(workspace);
        }
        const int32_t st = gemm_launch_shares(ctx, W, (const _Float16 *)panel, prod, K, N, M, 1);
        if (st != GALOIS_HIP_OK) return st;
        if (residual) {
            if (mn % 4 == 0)
                hipLaunchKernelGGL(gemm_sum_pass, sum_grid, dim3(256), 0, ctx->stream, reinterpret_cast<const float4 *>(prod),
                                   reinterpret_cast<const float4 *>(residual), reinterpret_cast<float4 *>(Y), mn / 4, (int64_t)0);
            else
                hipLaunchKernelGGL(gemm_sum_tail, dim3((unsigned)((mn + 255) / 256)), dim3(256), 0, ctx->stream, prod, residual, Y, mn);
        }
    }
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_f16_panel_add launch");
}

// The product alone, as the shares it is computed in: what galois_hip_mul_mat_q4_0_f16_panel_add does before its adding
// pass, for callers whose next op can do the adding (galois_hip_add_rms_norm_mul_f16_panel).
extern "C" int32_t galois_hip_mul_mat_q4_0_f16_panel_shares(galois_hip_ctx *ctx, const void *W, const void *panel, float *shares,
                                                            int64_t shares_bytes, int32_t K, int32_t N, int32_t M, int32_t *n_shares) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, W && panel && shares && n_shares, GALOIS_HIP_E_NULL, "mul_mat_q4_0_f16_panel_shares");
    *n_shares = 0;
    GH_REQUIRE(ctx, gemm_panel_shape_ok(K, M) && N > 0 && (int64_t)M * N < ((int64_t)1 << 31), GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_f16_panel_shares: K a positive multiple of 256, (M + 16) * K below 2^31, N positive, M * N below 2^31");
    GH_REQUIRE(ctx, gh_aligned(W, 16) && gh_aligned(panel, 16) && gh_aligned(shares, 16), GALOIS_HIP_E_ALIGN,
               "mul_mat_q4_0_f16_panel_shares: 16-byte aligned operands");
    const int64_t mn = (int64_t)M * N;
    GH_REQUIRE(ctx, shares_bytes >= mn * (int64_t)sizeof(float), GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_f16_panel_shares: room for at least one result of M * N floats");
    GH_BIND(ctx);
    const int n = gemm_two_shares_pay(ctx, K, N, M) && shares_bytes >= 2 * mn * (int64_t)sizeof(float) ? 2 : 1;
    const int32_t st = gemm_launch_shares(ctx, W, (const _Float16 *)panel, shares, K, N, M, n);
    if (st != GALOIS_HIP_OK) return st;
    *n_shares = n;
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_f16_panel_shares launch");
}

// sum_out = a (+ b) (+ c), and rms_norm(sum_out, eps) * weight into the panel, one launch.
extern "C" int32_t galois_hip_add_rms_norm_mul_f16_panel(galois_hip_ctx *ctx, const float *a, const float *b, const float *c,
                                                         float *sum_out, const float *weight, void *panel, int32_t ncols,
                                                         int32_t nrows, float eps) {
    const int32_t st = panel_args(ctx, a, weight, panel, ncols, nrows, "add_rms_norm_mul_f16_panel");
    if (st != GALOIS_HIP_OK) return st;
    GH_REQUIRE(ctx, sum_out, GALOIS_HIP_E_NULL, "add_rms_norm_mul_f16_panel: sum_out");
    GH_REQUIRE(ctx, gh_aligned(b, 16) && gh_aligned(c, 16) && gh_aligned(sum_out, 16), GALOIS_HIP_E_ALIGN,
               "add_rms_norm_mul_f16_panel: 16-byte aligned operands");
    const int nv = (ncols / 8 + kPanelNormThreads - 1) / kPanelNormThreads;
    GH_REQUIRE(ctx, nv <= 4, GALOIS_HIP_E_SHAPE, "add_rms_norm_mul_f16_panel: rows of at most 16384 columns");
    GH_BIND(ctx);
    const int groups = (nrows + 15) / 16, per_xcd = (groups + 7) / 8;
    const dim3 grid((unsigned)(8 * per_xcd * 16)), block(kPanelNormThreads);
    _Float16 *y = (_Float16 *)panel;
    if (nv <= 1)
        hipLaunchKernelGGL((rms_norm_to_f16_tiles<1, true>), grid, block, 0, ctx->stream, a, weight, y, nrows, ncols, eps, groups, per_xcd, b, c, sum_out);
    else if (nv <= 2)
        hipLaunchKernelGGL((rms_norm_to_f16_tiles<2, true>), grid, block, 0, ctx->stream, a, weight, y, nrows, ncols, eps, groups, per_xcd, b, c, sum_out);
    else
        hipLaunchKernelGGL((rms_norm_to_f16_tiles<4, true>), grid, block, 0, ctx->stream, a, weight, y, nrows, ncols, eps, groups, per_xcd, b, c, sum_out);
    GH_LAUNCH_CHECK(ctx, "add_rms_norm_mul_f16_panel launch");
}

// gate | up and the SwiGLU between them and the down projection in one launch: the panel of silu(Wg . x) * (Wu . x).
extern "C" int32_t galois_hip_mul_mat_q4_0_swiglu_f16_panel(galois_hip_ctx *ctx, const void *W_gate, const void *W_up, const void *panel,
                                                            void *panel_out, int32_t K, int32_t N, int32_t M) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, W_gate && W_up && panel && panel_out, GALOIS_HIP_E_NULL, "mul_mat_q4_0_swiglu_f16_panel");
    GH_REQUIRE(ctx, gemm_panel_shape_ok(K, M) && gemm_panel_shape_ok(N, M), GALOIS_HIP_E_SHAPE,
               "mul_mat_q4_0_swiglu_f16_panel: K and N positive multiples of 256, (M + 16) * K and (M + 16) * N below 2^31");
    GH_REQUIRE(ctx, gh_aligned(W_gate, 16) && gh_aligned(W_up, 16) && gh_aligned(panel, 16) && gh_aligned(panel_out, 16), GALOIS_HIP_E_ALIGN,
               "mul_mat_q4_0_swiglu_f16_panel: 16-byte aligned operands");
    GH_REQUIRE(ctx, panel != panel_out, GALOIS_HIP_E_SHAPE, "mul_mat_q4_0_swiglu_f16_panel: the two panels are distinct");
    GH_BIND(ctx);
    gemm_mats mats = {};
    mats.W[0] = (const uint8_t *)W_gate, mats.W[1] = (const uint8_t *)W_up, mats.N[0] = mats.N[1] = N;
    for (int j = 0; j < GEMM_MAX_MATS; j++) mats.col0[j] = 0x7FFFFFFF;
    mats.n_total = 96 * ((N + 47) / 48);
    mats.swiglu_out = static_cast<_Float16 *>(panel_out);
    const int32_t st = gemm_launch<96>(ctx, mats, (const _Float16 *)panel, K, M);
    if (st != GALOIS_HIP_OK) return st;
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_swiglu_f16_panel launch");
}
