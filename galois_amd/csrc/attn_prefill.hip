// Causal attention of many query rows over a KV cache in one launch: the prefill counterpart of attn_decode.hip.
//
// Replaces, per layer of a prefill, the op sequence cpy(q -> [D, M, H]), matmul(K^T, q), scale, diag_mask_inf +
// soft_max, matmul(V, p), cpy(-> [D, H, M]) (CudaMatMul src/cuda.rs:867-992, scale src/cuda.rs:1597-1663,
// soft_max src/cuda.rs:1257-1356, cpy src/cuda.rs:1382-1595) for heads of 128.  Scores never reach memory.
//
// Shape of the work on gfx950:
//   - One workgroup of 4 waves per (head, 64 * QT consecutive queries); a wave owns 16 * QT queries for the whole walk
//     over the keys and keeps their running maximum, running sum and the 16 x 128 output tile(s) in registers
//     (the one-pass softmax: when the maximum grows, sum and output are rescaled by exp2(old - new)).
//   - Keys are walked in blocks of 32.  The workgroup stages a block's K rows and V rows through LDS as fp16 (an f32
//     cache is rounded here, the reference's convert_fp32_to_fp16 in front of its gemm_ex), double-buffered: the global
//     loads of block b + 1 are in flight while block b is multiplied, one barrier per block.
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
constexpr int PA_THREADS = 256;
constexpr int PA_KROW = 272;               // bytes per key row of the K tile (256 + 16: fragment reads hit every bank once)
constexpr int PA_VROW = 80;                // bytes per dim row of the transposed V tile (32 slots of fp16 + 16)
constexpr int PA_KBYTES = PA_BK * PA_KROW;  // 8704
constexpr int PA_VBYTES = PA_D * PA_VROW;   // 10240
constexpr int PA_STAGE = PA_KBYTES + PA_VBYTES;

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

// One block's K and V pieces of a thread, as fp16 (8 halfs per uint4).
struct pa_stage_regs {
    uint4 k0, k1;  // key tid / 8: dims (tid % 8) * 8 .. + 7 and 64 + (tid % 8) * 8 .. + 7
    uint4 va, vb;  // two neighbouring keys: dims (lane % 16) * 8 .. + 7
};

template <bool KV16>
__device__ __forceinline__ uint4 pa_load8(const void *base, int64_t elem, bool live) {
    if (!live) return make_uint4(0, 0, 0, 0);
    if (KV16) return *reinterpret_cast<const uint4 *>(static_cast<const _Float16 *>(base) + elem);
    const float4 *p = reinterpret_cast<const float4 *>(static_cast<const float *>(base) + elem);
    return pa_pack8(p[0], p[1]);
}

template <bool KV16>
__device__ __forceinline__ void pa_fetch(pa_stage_regs &s, const pa_args &a, int head, int kb, int kend, int tid) {
    const int64_t E = (int64_t)a.n_head * PA_D;
    {
        const int key = kb * PA_BK + (tid >> 3), piece = tid & 7;
        const int64_t at = key * E + (int64_t)head * PA_D + piece * 8;
        s.k0 = pa_load8<KV16>(a.kc, at, key < kend);
        s.k1 = pa_load8<KV16>(a.kc, at + 64, key < kend);
    }
    {
        const int wave = tid >> 6, lane = tid & 63, w = lane >> 4, dg = lane & 15;
        const int key = kb * PA_BK + ((w & 2) ? 16 : 0) + 4 * wave + 2 * (w & 1);
        const int64_t at = key * E + (int64_t)head * PA_D + dg * 8;
        // keys past the last one in use are zeros: their probabilities are zero, and 0 * (whatever the cache holds
        // there) must not become NaN
        s.va = pa_load8<KV16>(a.vc, at, key < kend);
        s.vb = pa_load8<KV16>(a.vc, at + E, key + 1 < kend);
    }
}

__device__ __forceinline__ void pa_store(const pa_stage_regs &s, unsigned char *stage, int tid) {
    {
        unsigned char *row = stage + (tid >> 3) * PA_KROW + (tid & 7) * 16;
        *reinterpret_cast<uint4 *>(row) = s.k0;
        *reinterpret_cast<uint4 *>(row + 128) = s.k1;
    }
    {
        const int wave = tid >> 6, lane = tid & 63, w = lane >> 4, dg = lane & 15;
        unsigned char *vt = stage + PA_KBYTES + (4 * wave + w) * 4;  // the pair of slots 8 * wave + 2 * w, + 1
        const uint32_t a[4] = {s.va.x, s.va.y, s.va.z, s.va.w}, b[4] = {s.vb.x, s.vb.y, s.vb.z, s.vb.w};
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
    __shared__ __align__(16) unsigned char lds[2 * PA_STAGE];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    constexpr int BM = 64 * QT;
    const int head = blockIdx.x % a.n_head;
    const int tile = a.tiles - 1 - blockIdx.x / a.n_head;  // long walks first
    const int m0 = tile * BM;
    const int m_last = (m0 + BM < a.n ? m0 + BM : a.n) - 1;   // the workgroup's last live query
    const int kend = a.n_past + m_last + 1;                   // keys it may see
    const int nblk = (kend + PA_BK - 1) / PA_BK;
    const int64_t E = (int64_t)a.n_head * PA_D;
    const int mw0 = m0 + wave * 16 * QT;                      // the wave's first query

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
        for (int t = 0; t < 8; t++) acc[qt][t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }

    pa_stage_regs st;
    pa_fetch<KV16>(st, a, head, 0, kend, tid);
    pa_store(st, lds, tid);
    __syncthreads();

    for (int kb = 0; kb < nblk; kb++) {
        const bool more = kb + 1 < nblk;
        if (more) pa_fetch<KV16>(st, a, head, kb + 1, kend, tid);
        const unsigned char *ks = lds + (kb & 1) * PA_STAGE, *vt = ks + PA_KBYTES;
        const int key0 = kb * PA_BK;
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
                // key 0 is visible to every query, so the maximum is finite from the first block on
                const float m_new = fmaxf(m_run[qt], mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_new);
                m_run[qt] = m_new;
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    v[i] = __builtin_amdgcn_exp2f(v[i] - m_new);
                    sum += v[i];
                }
                l_run[qt] = l_run[qt] * alpha + sum;
                pf[qt] = __builtin_bit_cast(half8_t, make_uint4(pa_pack(v[0], v[1]), pa_pack(v[2], v[3]), pa_pack(v[4], v[5]),
                                                                pa_pack(v[6], v[7])));
#pragma unroll
                for (int t = 0; t < 8; t++) acc[qt][t] *= alpha;
            }
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const half8_t vf = *reinterpret_cast<const half8_t *>(vt + pa_vrow(t * 16 + r) * PA_VROW + g * 16);
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
                    acc[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[qt], acc[qt][t], 0, 0, 0);
            }
        }
        if (more) pa_store(st, lds + ((kb + 1) & 1) * PA_STAGE, tid);
        __syncthreads();
    }

#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        float l = l_run[qt];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        const float inv = 1.0f / l;
        const int m = mw0 + qt * 16 + r;
        if (PANEL) {
            // element (m, k) of the panel: tile (m / 16, k / 32) of 1 KB, 16-byte piece ((k % 32) / 8) * 16 + m % 16
            const int m_pad = (a.n + 15) & ~15;
            if (m < m_pad) {
                unsigned char *row = reinterpret_cast<unsigned char *>(a.panel) + ((int64_t)(m >> 4) * (E >> 5) + head * 4) * 1024 +
                                     (m & 15) * 16 + (g & 1) * 8;
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    uint2 o = make_uint2(0, 0);  // rows past n are zeros in a panel
                    if (m < a.n) o = make_uint2(pa_pack(acc[qt][t][0] * inv, acc[qt][t][1] * inv), pa_pack(acc[qt][t][2] * inv, acc[qt][t][3] * inv));
                    *reinterpret_cast<uint2 *>(row + (t >> 1) * 1024 + ((t & 1) * 2 + (g >> 1)) * 256) = o;
                }
            }
        } else if (m < a.n) {
            float *row = a.out + m * E + (int64_t)head * PA_D + g * 4;
#pragma unroll
            for (int t = 0; t < 8; t++)
                *reinterpret_cast<float4 *>(row + t * 16) =
                    make_float4(acc[qt][t][0] * inv, acc[qt][t][1] * inv, acc[qt][t][2] * inv, acc[qt][t][3] * inv);
        }
    }
}

template <int QT>
void pa_launch(galois_hip_ctx *ctx, const pa_args &a, bool kv16, bool panel) {
    const dim3 grid((unsigned)(a.tiles * a.n_head)), block(PA_THREADS);
    if (kv16) {
        if (panel) hipLaunchKernelGGL((attn_prefill_kernel<QT, true, true>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((attn_prefill_kernel<QT, true, false>), grid, block, 0, ctx->stream, a);
    } else {
        if (panel) hipLaunchKernelGGL((attn_prefill_kernel<QT, false, true>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((attn_prefill_kernel<QT, false, false>), grid, block, 0, ctx->stream, a);
    }
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
    // 64 queries per workgroup while that does not leave more than four rounds of workgroups per CU; 128 beyond
    const int64_t wg64 = ((int64_t)n_tokens + 63) / 64 * n_head;
    const int qt = wg64 > (int64_t)ctx->n_cu * 4 ? 2 : 1;
    a.tiles = (n_tokens + 64 * qt - 1) / (64 * qt);
    GH_REQUIRE(ctx, (int64_t)a.tiles * n_head < ((int64_t)1 << 31), GALOIS_HIP_E_SHAPE, "attn_prefill: too many workgroups");
    if (qt == 2) pa_launch<2>(ctx, a, kv16, out_panel != nullptr);
    else pa_launch<1>(ctx, a, kv16, out_panel != nullptr);
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
