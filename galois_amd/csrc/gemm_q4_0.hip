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
//   - X is rounded to fp16 once by f32_to_f16_rows into a context-owned workspace, so a
//     tile row of 64 k-values is one 128-byte line and the 4 MB panel stays L2-resident.
//   - Workgroup tile 128 (M) x 176 (N), k-step 64 (two Q4_0 blocks = one 36-byte slot per
//     weight row, fetched with dwordx4 + dwordx4 + dword).  11008 = 62.5 x 176, so the
//     512 x 11008 prefill is 4 x 63 = 252 workgroups: one round on 256 CUs.
//   - 8 waves: 4 consumers as 2 (M) x 2 (N), wave tile 64 x 96 or 64 x 80 -> 4 x 6 (or 5)
//     tiles of v_mfma_f32_16x16x32_f16 with f32 accumulators in registers, and 4 producers
//     that load, dequantise and store; each SIMD hosts one wave of each kind.
//   - LDS double-buffered: while MFMA consumes stage s the producers fill the other buffer
//     with stage s+1 and have stages s+2, s+3 in flight from memory; one barrier per stage.
//   - blockIdx is mapped so that an XCD (blockIdx % 8) owns one 128-row panel of X and a
//     contiguous range of weight tiles: X stays in that XCD's L2, W streams once per panel.
constexpr int GM = 128, GN = 176, GK = 64;
constexpr int GSTRIDE = 72;                 // halfs per LDS row: 144-byte rows -> conflict-free 16-byte reads
constexpr int GA_HALFS = GM * GSTRIDE;      // 9216 halfs  (18,432 B)
constexpr int GB_HALFS = GN * GSTRIDE;      // 12672 halfs (25,344 B)
typedef float float4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void f32_to_f16_rows(const float *__restrict__ x, _Float16 *__restrict__ y,
                                                       int64_t n8) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const float4 a = reinterpret_cast<const float4 *>(x)[2 * i], b = reinterpret_cast<const float4 *>(x)[2 * i + 1];
    uint4 o;
    o.x = pack_h2(a.x, a.y), o.y = pack_h2(a.z, a.w), o.z = pack_h2(b.x, b.y), o.w = pack_h2(b.z, b.w);
    reinterpret_cast<uint4 *>(y)[i] = o;
}

// Four nibble bytes (one dword of qs, already aligned) -> 4 + 4 fp16 weights:
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

// One Q4_0 block (d bits + 4 aligned qs dwords) -> 32 fp16 values written to an LDS row.
__device__ __forceinline__ void deq_block_to_lds(uint32_t dbits, const uint32_t q[4], _Float16 *dst) {
    const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t)dbits);
    const half2_t d2 = {d, d};
    uint32_t lo[8], hi[8];
#pragma unroll
    for (int j = 0; j < 4; j++) deq_dword(q[j], d2, lo + 2 * j, hi + 2 * j);
    uint4 *p = reinterpret_cast<uint4 *>(dst);
    p[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    p[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
    p[2] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    p[3] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
}

// Producer side.  The upper 4 waves of the workgroup fetch and convert; the lower 4 waves only
// read fragments and issue MFMA.  Every SIMD therefore hosts one wave of each kind and the
// hardware overlaps the dequantisation arithmetic of one with the matrix instructions of the
// other without any hand scheduling.
//
// All global loads are whole-line: eight consecutive lanes fetch the eight 16-byte chunks of one
// 128-byte line of X; the weights are fetched four stages at a time as the 144 contiguous bytes
// (8 blocks) each tile row contributes, parked as raw bytes in LDS, and every stage a thread
// lifts its row's 36-byte slot back out, dequantises it and stores fp16.
constexpr int GRAW_STRIDE = 144;                 // raw bytes per tile row per super-stage (4 slots)
constexpr int GRAW_BYTES = GN * GRAW_STRIDE;     // 25,344 B per raw buffer
constexpr int GRAW_CHUNKS = GN * 9;              // 16-byte chunks per raw buffer
constexpr int GRAW_PER_THREAD = (GRAW_CHUNKS + 255) / 256;

// The producers' global loads are issued through inline assembly and waited for by hand.
// Loads retire in order, so "at most n younger loads outstanding" is the exact condition for an
// older load to have landed.  Left to the compiler, loads whose use is one or more loop
// iterations away are waited for with vmcnt(0), which also drains every prefetch issued since.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void gload16(u32x4_t &dst, const void *ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
}
#define GEMM_VMWAIT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")

struct gemm_x_regs {
    u32x4_t c[4];  // chunk j: row 32*j + p/8, 16-byte chunk p%8 of that row's 128-byte line
};

__device__ __forceinline__ void gemm_load_x(const _Float16 *xbase, int K, int M, int m0, int p, int s, gemm_x_regs &r) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = min(m0 + 32 * j + (p >> 3), M - 1);
        gload16(r.c[j], xbase + (size_t)row * K + (size_t)s * GK + (p & 7) * 8);
    }
}

__device__ __forceinline__ void gemm_store_x(_Float16 *As, int p, const gemm_x_regs &r) {
#pragma unroll
    for (int j = 0; j < 4; j++)
        *reinterpret_cast<u32x4_t *>(As + (32 * j + (p >> 3)) * GSTRIDE + (p & 7) * 8) = r.c[j];
}

__device__ __forceinline__ void gemm_keep_alive(const gemm_x_regs &r) {
#pragma unroll
    for (int j = 0; j < 4; j++) asm volatile("" ::"v"(r.c[j]));
}

struct gemm_raw_regs {
    u32x4_t c[GRAW_PER_THREAD];
};

__device__ __forceinline__ void gemm_load_raw(const uint8_t *W, size_t wrow_bytes, int N, int n0, int p, int super,
                                              gemm_raw_regs &r) {
#pragma unroll
    for (int i = 0; i < GRAW_PER_THREAD; i++) {
        // unconditional (clamped) so that the number of loads in flight is the same on every path:
        // the compiler can then wait for exactly the loads it needs instead of draining them all
        const int q = min(p + 256 * i, GRAW_CHUNKS - 1);
        const int row = q / 9, c = q - row * 9;
        gload16(r.c[i], W + (size_t)min(n0 + row, N - 1) * wrow_bytes + (size_t)super * GRAW_STRIDE + c * 16);
    }
}

__device__ __forceinline__ void gemm_store_raw(uint8_t *raw, int p, const gemm_raw_regs &r) {
#pragma unroll
    for (int i = 0; i < GRAW_PER_THREAD; i++) {
        const int q = p + 256 * i;
        if (q < GRAW_CHUNKS) *reinterpret_cast<u32x4_t *>(raw + q * 16) = r.c[i];
    }
}

// Slot J (0..3) of tile row `prow` out of a raw buffer: three aligned 16-byte reads cover the
// 36 bytes at offset 36*J; dequantise both blocks into the fp16 B tile.
template <int J>
__device__ __forceinline__ void gemm_dequant_slot(const uint8_t *raw, _Float16 *Bs, int prow) {
    constexpr int first = (36 * J) / 16;        // first 16-byte piece
    constexpr int skip = (36 * J) / 4 - 4 * first;  // dwords to skip inside it
    const uint4 *src = reinterpret_cast<const uint4 *>(raw + prow * GRAW_STRIDE) + first;
    const uint4 a = src[0], b = src[1], c = src[2];
    const uint32_t d[12] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w, c.x, c.y, c.z, c.w};
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; i++) w[i] = d[skip + i];
    // block A: qs bytes straddle the slot's dwords by two bytes; block B is aligned
    const uint32_t qa[4] = {__builtin_amdgcn_alignbit(w[1], w[0], 16), __builtin_amdgcn_alignbit(w[2], w[1], 16),
                            __builtin_amdgcn_alignbit(w[3], w[2], 16), __builtin_amdgcn_alignbit(w[4], w[3], 16)};
    deq_block_to_lds(w[0] & 0xFFFFu, qa, Bs + prow * GSTRIDE);
    const uint32_t qb[4] = {w[5], w[6], w[7], w[8]};
    deq_block_to_lds(w[4] >> 16, qb, Bs + prow * GSTRIDE + 32);
}

// LDS map: [2] fp16 stage buffers (A | B), then [2] raw weight buffers.
constexpr int GBUF_HALFS = GA_HALFS + GB_HALFS;
constexpr size_t GEMM_LDS_BYTES = 2 * (size_t)GBUF_HALFS * sizeof(_Float16) + 2 * (size_t)GRAW_BYTES;

__device__ __forceinline__ void gemm_producer(_Float16 *smem, const uint8_t *__restrict__ W,
                                              const _Float16 *__restrict__ Xh, int K, int N, int M, int m0, int n0) {
    const int p = threadIdx.x - 256;
    const int nslots = K / 64;            // stages; a multiple of 4 (K % 256 == 0)
    const int nsuper = nslots / 4;
    const size_t wrow_bytes = (size_t)nslots * 36;
    uint8_t *raw0 = reinterpret_cast<uint8_t *>(smem + 2 * GBUF_HALFS);
    uint8_t *raw1 = raw0 + GRAW_BYTES;
    const bool has_w = p < GN;

    // prologue: raw super-stage 0 parked, super-stage 1 requested; X stages 0..3 requested
    gemm_raw_regs rr;
    gemm_x_regs x0, x1, x2, x3;  // X ring: stage t lives in x[t % 4]
    gemm_load_raw(W, wrow_bytes, N, n0, p, 0, rr);
    gemm_load_x(Xh, K, M, m0, p, 0, x0);
    gemm_load_x(Xh, K, M, m0, p, 1, x1);
    gemm_load_x(Xh, K, M, m0, p, 2, x2);
    gemm_load_x(Xh, K, M, m0, p, 3, x3);
    static_assert(GRAW_PER_THREAD == 7, "the hand-written vmcnt values below count 7 raw + 4 X loads per batch");
    GEMM_VMWAIT(16);  // raw super-stage 0 landed (16 younger X loads may still fly)
    gemm_store_raw(raw0, p, rr);
    gemm_load_raw(W, wrow_bytes, N, n0, p, min(1, nsuper - 1), rr);
    __syncthreads();  // raw0 visible to every producer
    GEMM_VMWAIT(19);  // x0 landed (younger: x1..x3 and one raw batch)
    gemm_store_x(smem, p, x0);
    if (has_w) gemm_dequant_slot<0>(raw0, smem + GA_HALFS, p);
    gemm_load_x(Xh, K, M, m0, p, min(4, nslots - 1), x0);
    __syncthreads();  // stage 0 visible to the consumers

    // Step run while the consumers compute stage S: produce stage t = S+1 (slot J = t % 4 of its
    // super-stage) into buffer t&1 from X ring register XR, then request X stage t+4 into XR.
    // On the last slot of a super-stage the raw bytes of the next one (requested four stages
    // ago) are parked in the other raw buffer, whose previous content was last read long before,
    // and the one after that is requested.
#define GEMM_PRODUCE(S, J, XR)                                                                   \
    {                                                                                            \
        const int t = (S) + 1;                                                                   \
        const int sup = t >> 2;                                                                  \
        _Float16 *buf = smem + (t & 1) * GBUF_HALFS;                                             \
        GEMM_VMWAIT(19); /* XR was requested four steps ago: 3 x 4 X loads + 7 raw loads younger */ \
        gemm_store_x(buf, p, XR);                                                                \
        if (has_w) gemm_dequant_slot<J>((sup & 1) ? raw1 : raw0, buf + GA_HALFS, p);             \
        gemm_load_x(Xh, K, M, m0, p, min(t + 4, nslots - 1), XR);                                \
        if ((J) == 3) {                                                                          \
            GEMM_VMWAIT(16); /* rr was requested four steps ago: 4 x 4 X loads younger */        \
            gemm_store_raw(((sup + 1) & 1) ? raw1 : raw0, p, rr);                                \
            gemm_load_raw(W, wrow_bytes, N, n0, p, min(sup + 2, nsuper - 1), rr);                \
        }                                                                                        \
        __syncthreads();                                                                         \
    }
    // full groups of four steps: no conditionals, so every load has a fixed distance to its use
    int s = 0;
    for (; s + 4 < nslots; s += 4) {
        GEMM_PRODUCE(s, 1, x1)
        GEMM_PRODUCE(s + 1, 2, x2)
        GEMM_PRODUCE(s + 2, 3, x3)
        GEMM_PRODUCE(s + 3, 0, x0)
    }
    // last group: stages nslots-3 .. nslots-1 are produced, the final step only meets the barrier
    // (the J == 3 step parks a clamped, unused copy of the last super-stage: harmless)
    GEMM_PRODUCE(s, 1, x1)
    GEMM_PRODUCE(s + 1, 2, x2)
    GEMM_PRODUCE(s + 2, 3, x3)
    __syncthreads();
    // The last requests of every ring register are never consumed.  To the compiler an inline-asm
    // load defines its destination at once, so a dead destination could be handed to some other
    // value while the load is still in flight and be overwritten when it lands.  Drain the loads,
    // then name every ring register once more so that all of them stay allocated until here.
    GEMM_VMWAIT(0);
    gemm_keep_alive(x0);
    gemm_keep_alive(x1);
    gemm_keep_alive(x2);
    gemm_keep_alive(x3);
#pragma unroll
    for (int i = 0; i < GRAW_PER_THREAD; i++) asm volatile("" ::"v"(rr.c[i]));
#undef GEMM_PRODUCE
}

// Consumer side: a wave that owns NF 16-wide column tiles starting at ncol0 and rows wm*64..+63.
template <int NF>
__device__ __forceinline__ void gemm_consumer(const _Float16 *smem, float *__restrict__ Y, int K, int N, int M, int m0,
                                              int n0, int wm, int ncol0) {
    const int lane = threadIdx.x & 63;
    const int nslots = K / 64;
    constexpr int BUF = GBUF_HALFS;
    float4_t acc[4][NF];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < NF; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int a_off = (wm * 64 + (lane & 15)) * GSTRIDE + (lane >> 4) * 8;
    const int b_off = GA_HALFS + (ncol0 + (lane & 15)) * GSTRIDE + (lane >> 4) * 8;
    __syncthreads();  // producers: raw weights parked
    __syncthreads();  // producers: stage 0 ready
    for (int s = 0; s < nslots; s++) {
        const _Float16 *buf = smem + (s & 1) * BUF;
        // both k-halves of the stage are requested up front so the second half's LDS latency
        // hides behind the first half's matrix instructions
        half8_t a[2][4], b[2][NF];
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                a[ks][i] = *reinterpret_cast<const half8_t *>(buf + a_off + i * 16 * GSTRIDE + ks * 32);
#pragma unroll
            for (int j = 0; j < NF; j++)
                b[ks][j] = *reinterpret_cast<const half8_t *>(buf + b_off + j * 16 * GSTRIDE + ks * 32);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < NF; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[ks][i], b[ks][j], acc[i][j], 0, 0, 0);
        __syncthreads();
    }
    // C layout of the 16x16 MFMA: column = lane % 16, row = 4 * (lane / 16) + e
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < NF; j++) {
            const int n = n0 + ncol0 + j * 16 + (lane & 15);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int m = m0 + wm * 64 + i * 16 + 4 * (lane >> 4) + e;
                if (m < M && n < N) Y[(size_t)m * N + n] = acc[i][j][e];
            }
        }
}

__global__ __launch_bounds__(512) void gemm_q4_0_mfma(const uint8_t *__restrict__ W, const _Float16 *__restrict__ Xh,
                                                      float *__restrict__ Y, int K, int N, int M, int n_tiles,
                                                      int m_tiles) {
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[];  // [2][A | B]
    // XCD-aware tile order: blockIdx % 8 is the XCD; consecutive tiles (same X panel) go to one XCD
    const int total = n_tiles * m_tiles;
    const int per_xcd = (total + 7) >> 3;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= total) return;
    const int mt = tile / n_tiles, nt = tile - mt * n_tiles;
    const int m0 = mt * GM, n0 = nt * GN;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // consumer waves 2 (M) x 2 (N): the left column owns 6 column tiles (96 wide), the right one 5 (80)
    if (wave >= 4)
        gemm_producer(smem, W, Xh, K, N, M, m0, n0);
    else if ((wave & 1) == 0)
        gemm_consumer<6>(smem, Y, K, N, M, m0, n0, wave >> 1, 0);
    else
        gemm_consumer<5>(smem, Y, K, N, M, m0, n0, wave >> 1, 96);
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
    if (K % 256 == 0 && gh_aligned(W, 16)) {
        // fp16 copy of X in the context's workspace (grown on demand, kept until the context dies)
        const size_t need = (size_t)M * K * sizeof(_Float16);
        if (ctx->ws_bytes < need) {
            GH_NOT_CAPTURING(ctx, "mul_mat_q4_0_f32: growing the fp16 workspace");
            hipError_t e = hipStreamSynchronize(ctx->stream);
            if (e != hipSuccess) return gh_hip(ctx, e, "hipStreamSynchronize");
            if (ctx->ws) (void)hipFree(ctx->ws);
            ctx->ws = nullptr;
            ctx->ws_bytes = 0;
            e = hipMalloc(&ctx->ws, need);
            if (e != hipSuccess) return gh_hip(ctx, e, "hipMalloc(workspace)");
            ctx->ws_bytes = need;
        }
        _Float16 *Xh = (_Float16 *)ctx->ws;
        const int64_t n8 = (int64_t)M * K / 8;
        hipLaunchKernelGGL(f32_to_f16_rows, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, ctx->stream, X, Xh, n8);
        const int n_tiles = (N + GN - 1) / GN, m_tiles = (M + GM - 1) / GM;
        const int total = n_tiles * m_tiles;
        const int grid = ((total + 7) / 8) * 8;
        const size_t lds = GEMM_LDS_BYTES;
        static bool attr_set = false;
        if (!attr_set) {
            hipError_t e = hipFuncSetAttribute((const void *)gemm_q4_0_mfma, hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)lds);
            if (e != hipSuccess) return gh_hip(ctx, e, "hipFuncSetAttribute(LDS size)");
            attr_set = true;
        }
        hipLaunchKernelGGL(gemm_q4_0_mfma, dim3(grid), dim3(512), lds, ctx->stream, (const uint8_t *)W, Xh, Y, K, N, M,
                           n_tiles, m_tiles);
    } else {
        const dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
        hipLaunchKernelGGL(gemm_q4_0_mfma_v1, grid, dim3(256), 0, ctx->stream, (const uint8_t *)W, X, Y, K, N, M);
    }
    GH_LAUNCH_CHECK(ctx, "mul_mat_q4_0_f32 launch");
}
