// Causal attention of many query rows over a KV cache in one launch: the prefill counterpart of attn_decode.hip.
//
// Replaces, per layer of a prefill, the op sequence cpy(q -> [D, M, H]), matmul(K^T, q), scale, diag_mask_inf +
// soft_max, matmul(V, p), cpy(-> [D, H, M]) (CudaMatMul src/cuda.rs:867-992, scale src/cuda.rs:1597-1663,
// soft_max src/cuda.rs:1257-1356, cpy src/cuda.rs:1382-1595) for heads of 128.  Scores never reach memory.
//
// Shape of the work on gfx950:
//   - One workgroup of 8 waves per (head, 64 * QT consecutive queries).  A wave owns 16 * QT queries and keeps their
//     running maximum, running sum and the 16 x 128 output tile(s) in registers (the one-pass softmax: when the
//     maximum grows, sum and output are rescaled by exp2(old - new)).  Two waves own the same queries: keys are walked
//     in stages of 64, one wave multiplies the first 32-key block of every stage, the other the second, and at the end
//     the second hands its maximum, sum and output to the first through LDS -- half the chain of dependent blocks per
//     wave, and two waves per SIMD.
//   - The workgroup stages K rows and V rows through LDS as fp16 (an f32 cache is rounded on the way, the reference's
//     convert_fp32_to_fp16 in front of its gemm_ex), double-buffered: the global loads of stage s + 1 are in flight
//     while stage s is multiplied (they are unconditional -- keys past the end point at the last live row and are
//     zeroed on the way to LDS -- and stay raw in registers until then), one barrier per stage.
//   - Both products use v_mfma_f32_16x16x32_f16 with the QUERY on the column side:
//       S^T (16 keys x 16 queries) = K (A operand, rows = keys)  x  Q^T (B operand, 4 chunks of 32 dims),
//       O^T (16 dims x 16 queries) = V^T (A operand, rows = dims) x  P^T (B operand, 32 keys),
//     so a lane holds, for ONE query (lane % 16), four keys of each 16-key tile of S^T and four dims of each 16-dim tile
//     of O^T: the row maximum needs two cross-lane steps, the rescale none, and the probabilities a lane has just
//     computed are exactly its piece of the B operand of the second product (no shuffle, no LDS round trip).
//   - That fixes the order of the 32 keys along the second product's k axis: slot 8g + j holds key 4g + j of the first
//     16-key tile and slot 8g + 4 + j key 16 + 4g + j of the second.  V is written to LDS transposed ([dim][slot]) in
//     that order, two keys per 32-bit store, so an A fragment is one 16-byte read.  Rows of 80 bytes and a rotation of
//     the eight dims a thread owns keep those stores at two lanes per bank (the floor for 64 lanes) and the reads free
//     of conflicts; K rows of 272 bytes do the same for the first product's fragments.
//   - Causal structure: a workgroup stops at the last key its last query may see, a wave skips blocks that lie wholly
//     behind the mask for all its queries, the mask itself is applied only in blocks that straddle it.  The tiles with
//     the longest walks are scheduled first.  blockIdx % 8 (the XCD) depends only on the head when n_head % 8 == 0: a
//     head's keys stay in one L2.
#include "common.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int PA_D = 128;                  // head dim
constexpr int PA_BK = 32;                  // keys per block
constexpr int PA_THREADS = 512;
constexpr int PA_KROW = 272;               // bytes per key row of the K tile (256 + 16: fragment reads hit every bank once)
constexpr int PA_VROW = 80;                // bytes per dim row of the transposed V tile (32 slots of fp16 + 16)
constexpr int PA_KBYTES = PA_BK * PA_KROW;  // 8704
constexpr int PA_VBYTES = PA_D * PA_VROW;   // 10240
constexpr int PA_BLOCK = PA_KBYTES + PA_VBYTES;  // one block of 32 keys in LDS
constexpr int PA_STAGE = 2 * PA_BLOCK;            // a stage: two blocks, one per half of the workgroup
constexpr int PA_LDS = 2 * PA_STAGE;              // 75,776 bytes

struct pa_args {
    const float *q;     // [n][n_head * 128], rotated
    const void *kc;     // [>= n_past + n][n_head * 128] f32 or f16
    const void *vc;
    float *out;         // [n][n_head * 128] f32, or
    _Float16 *panel;    // the prefill matmul's fp16 panel of a [n_head * 128, n] operand
    int n, n_past, n_head, tiles;
    float qscale;       // scale * log2(e): the softmax runs in base 2
};

__device__ __forceinline__ uint32_t pa_pack(float a, float b) {
    half2_t h;
    h.x = (_Float16)a;
    h.y = (_Float16)b;
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ uint4 pa_pack8(const float4 a, const float4 b) {
    return make_uint4(pa_pack(a.x, a.y), pa_pack(a.z, a.w), pa_pack(b.x, b.y), pa_pack(b.z, b.w));
}

// The row of the transposed V tile that holds dim d: the eight rows of a group of eight dims are rotated by the
// group's index, so that the sixteen threads that store the same element of their eight dims hit different banks.
__device__ __forceinline__ int pa_vrow(int d) { return (d & ~7) | ((d + (d >> 3)) & 7); }

// One block's K and V pieces of a thread as they come from the cache (an f32 cache is rounded when the pieces go to
// LDS, after the block in between has been multiplied: the loads stay in flight meanwhile).
template <bool KV16>
struct pa_stage_regs;
template <>
struct pa_stage_regs<true> {
    uint4 k0, k1;  // key t / 8 of the block: dims (t % 8) * 8 .. + 7 and 64 + (t % 8) * 8 .. + 7   (t = tid % 256)
    uint4 va, vb;  // two neighbouring keys: dims (lane % 16) * 8 .. + 7
    __device__ __forceinline__ void load(uint4 &dst, const void *base, int64_t elem) {
        dst = *reinterpret_cast<const uint4 *>(static_cast<const _Float16 *>(base) + elem);
    }
    __device__ __forceinline__ uint4 half8(const uint4 &v) const { return v; }
};
template <>
struct pa_stage_regs<false> {
    struct f8 {
        float4 lo, hi;
    };
    f8 k0, k1, va, vb;
    __device__ __forceinline__ void load(f8 &dst, const void *base, int64_t elem) {
        const float4 *p = reinterpret_cast<const float4 *>(static_cast<const float *>(base) + elem);
        dst.lo = p[0], dst.hi = p[1];
    }
    __device__ __forceinline__ uint4 half8(const f8 &v) const { return pa_pack8(v.lo, v.hi); }
};

// Block `blk` (32 keys) of the cache: the 256 threads of one half of the workgroup fetch it (t = tid % 256).  Keys
// from kend on are not part of the walk (and may lie past the end of the cache): their loads are pointed at key
// kend - 1, so that every load is unconditional, and pa_store replaces what they bring by zeros.
__device__ __forceinline__ int pa_k_key(int blk, int t) { return blk * PA_BK + (t >> 3); }
__device__ __forceinline__ int pa_v_key(int blk, int t) {
    const int wv = t >> 6, w = (t & 63) >> 4;
    return blk * PA_BK + ((w & 2) ? 16 : 0) + 4 * wv + 2 * (w & 1);
}

template <bool KV16>
__device__ __forceinline__ void pa_fetch(pa_stage_regs<KV16> &s, const pa_args &a, int head, int blk, int kend, int t) {
    const int64_t E = (int64_t)a.n_head * PA_D;
    {
        const int key = min(pa_k_key(blk, t), kend - 1);
        const int64_t at = key * E + (int64_t)head * PA_D + (t & 7) * 8;
        s.load(s.k0, a.kc, at);
        s.load(s.k1, a.kc, at + 64);
    }
    {
        const int key = pa_v_key(blk, t);
        const int64_t col = (int64_t)head * PA_D + (t & 15) * 8;
        s.load(s.va, a.vc, min(key, kend - 1) * E + col);
        s.load(s.vb, a.vc, min(key + 1, kend - 1) * E + col);
    }
}

__device__ __forceinline__ uint4 pa_keep(const uint4 v, bool live) {
    return make_uint4(live ? v.x : 0u, live ? v.y : 0u, live ? v.z : 0u, live ? v.w : 0u);
}

template <bool KV16>
__device__ __forceinline__ void pa_store(const pa_stage_regs<KV16> &s, unsigned char *dst, int blk, int kend, int t) {
    {
        // keys past the last one in use are zeros: their probabilities are zero, and 0 * (whatever a cache holds
        // there) must not become NaN
        const bool live = pa_k_key(blk, t) < kend;
        unsigned char *row = dst + (t >> 3) * PA_KROW + (t & 7) * 16;
        *reinterpret_cast<uint4 *>(row) = pa_keep(s.half8(s.k0), live);
        *reinterpret_cast<uint4 *>(row + 128) = pa_keep(s.half8(s.k1), live);
    }
    {
        const int wv = t >> 6, lane = t & 63, w = lane >> 4, dg = lane & 15;
        const int key = pa_v_key(blk, t);
        unsigned char *vt = dst + PA_KBYTES + (4 * wv + w) * 4;  // the pair of slots 8 * wv + 2 * w, + 1
        const uint4 va = pa_keep(s.half8(s.va), key < kend), vb = pa_keep(s.half8(s.vb), key + 1 < kend);
        const uint32_t a[4] = {va.x, va.y, va.z, va.w}, b[4] = {vb.x, vb.y, vb.z, vb.w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t lo = (e & 1) ? (a[e >> 1] >> 16) : (a[e >> 1] & 0xffffu);
            const uint32_t hi = (e & 1) ? (b[e >> 1] & 0xffff0000u) : (b[e >> 1] << 16);
            *reinterpret_cast<uint32_t *>(vt + (dg * 8 + ((e + dg) & 7)) * PA_VROW) = lo | hi;
        }
    }
}

template <int QT, bool KV16, bool PANEL>
__global__ __launch_bounds__(PA_THREADS) void attn_prefill_kernel(const pa_args a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // two stages of two blocks: [K 32 x 272 | V^T 128 x 80]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int half = wave >> 2;   // which block of a stage this wave multiplies (and helps to fetch)
    const int wq = wave & 3;      // which queries of the workgroup it owns
    const int t = tid & 255;
    constexpr int BM = 64 * QT;
    const int head = blockIdx.x % a.n_head;
    const int tile = a.tiles - 1 - blockIdx.x / a.n_head;  // long walks first
    const int m0 = tile * BM;
    const int m_last = (m0 + BM < a.n ? m0 + BM : a.n) - 1;   // the workgroup's last live query
    const int kend = a.n_past + m_last + 1;                   // keys it may see
    const int nstage = (kend + 2 * PA_BK - 1) / (2 * PA_BK);
    const int64_t E = (int64_t)a.n_head * PA_D;
    const int mw0 = m0 + wq * 16 * QT;                        // the wave's first query

    // Q^T fragments, scaled: for query tile qt and chunk c, dims c * 32 + g * 8 .. + 7 of query mw0 + qt * 16 + r
    half8_t qf[QT][4];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        const int m = mw0 + qt * 16 + r;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m < a.n) {
                const float4 *p = reinterpret_cast<const float4 *>(a.q + m * E + (int64_t)head * PA_D + c * 32 + g * 8);
                float4 x = p[0], y = p[1];
                x.x *= a.qscale, x.y *= a.qscale, x.z *= a.qscale, x.w *= a.qscale;
                y.x *= a.qscale, y.y *= a.qscale, y.z *= a.qscale, y.w *= a.qscale;
                v = pa_pack8(x, y);
            }
            qf[qt][c] = __builtin_bit_cast(half8_t, v);
        }
    }

    float4_t acc[QT][8];
    float m_run[QT], l_run[QT];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        m_run[qt] = -INFINITY, l_run[qt] = 0.0f;
#pragma unroll
        for (int tt = 0; tt < 8; tt++) acc[qt][tt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }

    pa_stage_regs<KV16> st;
    pa_fetch<KV16>(st, a, head, half, kend, t);
    pa_store<KV16>(st, lds + half * PA_BLOCK, half, kend, t);
    __syncthreads();

    for (int sg = 0; sg < nstage; sg++) {
        const bool more = sg + 1 < nstage;
        if (more) pa_fetch<KV16>(st, a, head, (sg + 1) * 2 + half, kend, t);
        const unsigned char *ks = lds + (sg & 1) * PA_STAGE + half * PA_BLOCK, *vt = ks + PA_KBYTES;
        const int key0 = (sg * 2 + half) * PA_BK;
        // the wave's last query sees keys up to n_past + mw0 + 16 * QT - 1: blocks behind that are nothing to it
        if (key0 <= a.n_past + mw0 + 16 * QT - 1) {
            float4_t s[QT][2];
#pragma unroll
            for (int qt = 0; qt < QT; qt++) s[qt][0] = s[qt][1] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const half8_t kf = *reinterpret_cast<const half8_t *>(ks + (b * 16 + r) * PA_KROW + c * 64 + g * 16);
#pragma unroll
                    for (int qt = 0; qt < QT; qt++)
                        s[qt][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[qt][c], s[qt][b], 0, 0, 0);
                }
            half8_t pf[QT];
#pragma unroll
            for (int qt = 0; qt < QT; qt++) {
                float v[8] = {s[qt][0][0], s[qt][0][1], s[qt][0][2], s[qt][0][3], s[qt][1][0], s[qt][1][1], s[qt][1][2], s[qt][1][3]};
                // the mask: query m sees keys 0 .. n_past + m; only blocks that reach past the wave's first query need it
                if (key0 + PA_BK - 1 > a.n_past + mw0 + qt * 16) {
                    const int limit = a.n_past + mw0 + qt * 16 + r;
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const int key = key0 + (i >> 2) * 16 + g * 4 + (i & 3);
                        if (key > limit) v[i] = -INFINITY;
                    }
                }
                float mx = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                // a query that has seen no key yet (the second block of a stage can lie behind its mask) keeps -inf as
                // its maximum; the exponentials then take 0 as their reference and come out as exact zeros
                const float m_new = fmaxf(m_run[qt], mx);
                const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
                const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_ref);
                m_run[qt] = m_new;
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    v[i] = __builtin_amdgcn_exp2f(v[i] - m_ref);
                    sum += v[i];
                }
                l_run[qt] = l_run[qt] * alpha + sum;
                pf[qt] = __builtin_bit_cast(half8_t, make_uint4(pa_pack(v[0], v[1]), pa_pack(v[2], v[3]), pa_pack(v[4], v[5]),
                                                                pa_pack(v[6], v[7])));
#pragma unroll
                for (int tt = 0; tt < 8; tt++) acc[qt][tt] *= alpha;
            }
#pragma unroll
            for (int tt = 0; tt < 8; tt++) {
                const half8_t vf = *reinterpret_cast<const half8_t *>(vt + pa_vrow(tt * 16 + r) * PA_VROW + g * 16);
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
                    acc[qt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[qt], acc[qt][tt], 0, 0, 0);
            }
        }
        if (more) pa_store<KV16>(st, lds + ((sg + 1) & 1) * PA_STAGE + half * PA_BLOCK, (sg + 1) * 2 + half, kend, t);
        __syncthreads();
    }

    // The two waves that own the same queries (one walked the first block of every stage, the other the second) meet:
    // the second hands over maximum, sum and output through LDS (free after the last barrier), the first merges.
    float *xch = reinterpret_cast<float *>(lds) + wq * (QT * 34 * 64) + lane;
    if (half == 1) {
#pragma unroll
        for (int qt = 0; qt < QT; qt++) {
            float *x = xch + qt * 34 * 64;
            x[0] = m_run[qt], x[64] = l_run[qt];
#pragma unroll
            for (int tt = 0; tt < 8; tt++)
#pragma unroll
                for (int j = 0; j < 4; j++) x[(2 + tt * 4 + j) * 64] = acc[qt][tt][j];
        }
    }
    __syncthreads();
    if (half == 1) return;

#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        const float *x = xch + qt * 34 * 64;
        // the first wave has seen key 0, so the common maximum is finite
        const float m2 = x[0], m_all = fmaxf(m_run[qt], m2);
        const float a1 = __builtin_amdgcn_exp2f(m_run[qt] - m_all), a2 = __builtin_amdgcn_exp2f(m2 - m_all);
        float l = l_run[qt] * a1 + x[64] * a2;
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        const float inv = 1.0f / l;
        float4_t o[8];
#pragma unroll
        for (int tt = 0; tt < 8; tt++)
#pragma unroll
            for (int j = 0; j < 4; j++) o[tt][j] = (acc[qt][tt][j] * a1 + x[(2 + tt * 4 + j) * 64] * a2) * inv;
        const int m = mw0 + qt * 16 + r;
        if (PANEL) {
            // element (m, k) of the panel: tile (m / 16, k / 32) of 1 KB, 16-byte piece ((k % 32) / 8) * 16 + m % 16
            const int m_pad = (a.n + 15) & ~15;
            if (m < m_pad) {
                unsigned char *row = reinterpret_cast<unsigned char *>(a.panel) + ((int64_t)(m >> 4) * (E >> 5) + head * 4) * 1024 +
                                     (m & 15) * 16 + (g & 1) * 8;
#pragma unroll
                for (int tt = 0; tt < 8; tt++) {
                    uint2 w2 = make_uint2(0, 0);  // rows past n are zeros in a panel
                    if (m < a.n) w2 = make_uint2(pa_pack(o[tt][0], o[tt][1]), pa_pack(o[tt][2], o[tt][3]));
                    *reinterpret_cast<uint2 *>(row + (tt >> 1) * 1024 + ((tt & 1) * 2 + (g >> 1)) * 256) = w2;
                }
            }
        } else if (m < a.n) {
            float *row = a.out + m * E + (int64_t)head * PA_D + g * 4;
#pragma unroll
            for (int tt = 0; tt < 8; tt++) *reinterpret_cast<float4 *>(row + tt * 16) = make_float4(o[tt][0], o[tt][1], o[tt][2], o[tt][3]);
        }
    }
}

template <int QT, bool KV16, bool PANEL>
hipError_t pa_launch_one(galois_hip_ctx *ctx, const pa_args &a) {
    const hipError_t e = hipFuncSetAttribute((const void *)attn_prefill_kernel<QT, KV16, PANEL>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, PA_LDS);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((attn_prefill_kernel<QT, KV16, PANEL>), dim3((unsigned)(a.tiles * a.n_head)), dim3(PA_THREADS), PA_LDS,
                       ctx->stream, a);
    return hipSuccess;
}

template <int QT>
hipError_t pa_launch(galois_hip_ctx *ctx, const pa_args &a, bool kv16, bool panel) {
    if (kv16) return panel ? pa_launch_one<QT, true, true>(ctx, a) : pa_launch_one<QT, true, false>(ctx, a);
    return panel ? pa_launch_one<QT, false, true>(ctx, a) : pa_launch_one<QT, false, false>(ctx, a);
}

int32_t pa_entry(galois_hip_ctx *ctx, const float *q, const void *k_cache, const void *v_cache, bool kv16, float *out, void *out_panel,
                 int32_t n_head, int32_t head_dim, int32_t n_tokens, int32_t n_past, float scale) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, q && k_cache && v_cache && ((out != nullptr) != (out_panel != nullptr)), GALOIS_HIP_E_NULL,
               "attn_prefill: q, k_cache, v_cache and exactly one of out, out_panel");
    GH_REQUIRE(ctx, head_dim == PA_D, GALOIS_HIP_E_UNSUPPORTED, "attn_prefill: head_dim must be 128");
    GH_REQUIRE(ctx, n_head > 0 && n_tokens > 0 && n_past >= 0 && (int64_t)n_past + n_tokens < ((int64_t)1 << 30) && n_head <= 65536,
               GALOIS_HIP_E_SHAPE, "attn_prefill: n_head in 1 .. 65536, n_tokens positive, n_past not negative");
    GH_REQUIRE(ctx, gh_aligned(q, 16) && gh_aligned(k_cache, 16) && gh_aligned(v_cache, 16) && gh_aligned(out, 16) && gh_aligned(out_panel, 16),
               GALOIS_HIP_E_ALIGN, "attn_prefill: all pointers 16-byte aligned");
    GH_BIND(ctx);
    pa_args a;
    a.q = q, a.kc = k_cache, a.vc = v_cache, a.out = out, a.panel = static_cast<_Float16 *>(out_panel);
    a.n = n_tokens, a.n_past = n_past, a.n_head = n_head;
    a.qscale = scale * 1.44269504088896340736f;
    // 64 queries per workgroup, or 128 (a wave then multiplies every K and V fragment it reads from LDS with two query
    // tiles): the larger shape wins once the launch is bound by that traffic rather than by its dependent chains --
    // four workgroups of 64 per CU or more, or two when every walk is long (as many cached positions as new rows, so
    // that the causal walks differ by at most a factor of two).  Measured on 256 CUs, 32 heads, f32 cache, us for 64 /
    // 128 queries: 512 rows 15.7 / 22.4, 1024 rows 31.0 / 37.4, 2048 rows 112 / 82.6, 1024 rows behind 1024 positions
    // 83.7 / 72.0, 512 behind 1536 59.0 / 71.4; 8 heads x 4096 rows 100 / 124.
    const int64_t wg64 = ((int64_t)n_tokens + 63) / 64 * n_head, cus = ctx->n_cu > 0 ? ctx->n_cu : 256;
    const int qt = (wg64 >= 4 * cus || (wg64 >= 2 * cus && n_past >= n_tokens)) ? 2 : 1;
    a.tiles = (n_tokens + 64 * qt - 1) / (64 * qt);
    GH_REQUIRE(ctx, (int64_t)a.tiles * n_head < ((int64_t)1 << 31), GALOIS_HIP_E_SHAPE, "attn_prefill: too many workgroups");
    const hipError_t e = qt == 2 ? pa_launch<2>(ctx, a, kv16, out_panel != nullptr) : pa_launch<1>(ctx, a, kv16, out_panel != nullptr);
    if (e != hipSuccess) return gh_hip(ctx, e, "hipFuncSetAttribute(LDS size)");
    GH_LAUNCH_CHECK(ctx, "attn_prefill");
}

}  // namespace

extern "C" int32_t galois_hip_attn_prefill_f32(galois_hip_ctx *ctx, const float *q, const float *k_cache, const float *v_cache,
                                               float *out, void *out_panel, int32_t n_head, int32_t head_dim, int32_t n_tokens,
                                               int32_t n_past, float scale) {
    return pa_entry(ctx, q, k_cache, v_cache, false, out, out_panel, n_head, head_dim, n_tokens, n_past, scale);
}

extern "C" int32_t galois_hip_attn_prefill_f16kv(galois_hip_ctx *ctx, const float *q, const void *k_cache, const void *v_cache,
                                                 float *out, void *out_panel, int32_t n_head, int32_t head_dim, int32_t n_tokens,
                                                 int32_t n_past, float scale) {
    return pa_entry(ctx, q, k_cache, v_cache, true, out, out_panel, n_head, head_dim, n_tokens, n_past, scale);
}
