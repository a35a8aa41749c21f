// Attention of one decode step over an f32 KV cache, as one streaming pass.
//
// In galois's op vocabulary a decode step's attention is rope_custom(q), rope_custom(k), cpy(k -> cache row),
// cpy(v -> cache row), matmul(K^T, q), scale, soft_max, matmul(V, p) (launchers src/cuda.rs:1257-1356, 1382-1595,
// 698-782, 1597-1663).  Issued one by one these are nine launches that read the 64 MB of one layer's cache at
// a third of the HBM rate, most of the time being launch gaps.  Here the same arithmetic runs in one launch:
//
//   attn_decode_partial: a workgroup owns 128 consecutive keys of one head.  It rotates its head's q (every
//     workgroup of the head does, it is 128 floats), and the workgroup that owns position n_past also rotates
//     the new k and writes k and v into row n_past of the caches.  Scores = scale * (k . q) go to LDS; the
//     workgroup takes their maximum m, p = exp(score - m), the sum of p and the partial output sum p * v, and
//     writes (m, sum, partial output) to the context's scratch block, then counts itself on the head's counter;
//   the workgroup that counts a head's last split rescales the head's partials to the global maximum, adds them
//     in split order and divides by the total: out = softmax(scores) . V exactly as the three separate ops
//     define it, up to the order of the f32 additions (the result does not depend on which workgroup merges).
//
// A lane owns 4 consecutive floats of a head; head_dim / 4 lanes cover one key, so a wave-load of 16 bytes per
// lane reads 64 / (head_dim / 4) whole cache rows of the head (512 contiguous bytes each for head_dim 128).
#include "attn_decode_body.h"

namespace {

constexpr int AT_THREADS = 256;

template <int LPR, typename CT>
__global__ __launch_bounds__(AT_THREADS) void attn_decode_partial(const float *__restrict__ q, const float *__restrict__ k,
                                                                  const float *__restrict__ v, CT *__restrict__ kc,
                                                                  CT *__restrict__ vc, float *__restrict__ part,
                                                                  unsigned *__restrict__ done, float *__restrict__ out, int H, int L,
                                                                  const int32_t *__restrict__ pos, float freq_scale,
                                                                  float theta_scale, float scale, int64_t key_stride,
                                                                  int64_t head_stride) {
    attn_decode_wg<LPR, CT, AT_THREADS, false>(q, k, v, kc, vc, part, done, out, H, L, pos, freq_scale, theta_scale, scale,
                                               (int)blockIdx.y, (int)blockIdx.x, (int)gridDim.x, nullptr, 0u, key_stride,
                                               head_stride);
}

// Scratch of the entry point that allocates nothing: per-head counters, then the split records.  One copy per
// device, held from the moment the library's code is loaded there until the process ends.
constexpr int64_t AT_STATIC_HEADS = 1024;
constexpr int64_t AT_STATIC_FLOATS = 1 << 18;  // records: n_head * splits * (head_dim + 4) floats, 1 MB
}  // namespace
static __device__ __align__(256) unsigned char scratch[AT_STATIC_HEADS * sizeof(unsigned) + AT_STATIC_FLOATS * sizeof(float)];
namespace {

// static_scratch: the partial results and counters live in the device's copy of `scratch` (ctx->attn_static)
// instead of the blocks the context allocated.
template <typename CT>
int32_t attn_decode_launch(galois_hip_ctx *ctx, const float *q, const float *k, const float *v, CT *k_cache, CT *v_cache,
                           float *out, int32_t n_head, int32_t head_dim, int32_t n_past, const int32_t *pos,
                           float freq_scale, float theta_scale, float scale, int32_t head_major_n_ctx, const char *what,
                           bool static_scratch = false) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, q && k && v && k_cache && v_cache && out && pos, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, n_head > 0 && n_head <= 65535 && n_past >= 0 && n_past < 0x7FFFFF00, GALOIS_HIP_E_SHAPE,
               "attn_decode: n_head in 1..65535, n_past >= 0");
    GH_REQUIRE(ctx, head_dim == 64 || head_dim == 128, GALOIS_HIP_E_UNSUPPORTED, "attn_decode: head_dim 64 or 128");
    GH_REQUIRE(ctx, gh_aligned(q, 16) && gh_aligned(k, 16) && gh_aligned(v, 16) && gh_aligned(k_cache, 16) &&
                        gh_aligned(v_cache, 16) && gh_aligned(out, 16) && gh_aligned(pos, 4),
               GALOIS_HIP_E_ALIGN, "attn_decode: 16-byte aligned vectors and caches");
    GH_REQUIRE(ctx, head_major_n_ctx == 0 || head_major_n_ctx > n_past, GALOIS_HIP_E_SHAPE,
               "attn_decode: head_major_n_ctx is 0 or the capacity of a [n_head][n_ctx][head_dim] cache, above n_past");
    const int64_t key_stride = head_major_n_ctx ? head_dim : (int64_t)n_head * head_dim;
    const int64_t head_stride = head_major_n_ctx ? (int64_t)head_major_n_ctx * head_dim : head_dim;
    const int L = n_past + 1;
    const int S = (L + AT_KEYS - 1) / AT_KEYS;
    float *part;
    unsigned *done;  // one counter per head, zero between calls
    if (static_scratch) {
        GH_REQUIRE(ctx, ctx->attn_static != nullptr, GALOIS_HIP_E_UNSUPPORTED, "attn_decode: the device's static scratch was not found");
        GH_REQUIRE(ctx, S == 1 || (S <= AT_MAX_SPLITS && n_head <= AT_STATIC_HEADS &&
                                   (int64_t)n_head * S * (head_dim + 4) <= AT_STATIC_FLOATS),
                   GALOIS_HIP_E_SHAPE, "attn_decode_f32_static: at most 1024 heads and n_head * ceil((n_past + 1) / 128) * "
                                       "(head_dim + 4) <= 262144 floats of partial results (the static 1 MB block)");
        done = (unsigned *)ctx->attn_static;
        part = (float *)((unsigned char *)ctx->attn_static + AT_STATIC_HEADS * sizeof(unsigned));
    } else {
        GH_REQUIRE(ctx, S == 1 || (S <= AT_MAX_SPLITS && (int64_t)n_head * S * (head_dim + 4) <= GH_PARTIAL_FLOATS && ctx->scratch != nullptr && ctx->attn_done != nullptr),
                   GALOIS_HIP_E_UNSUPPORTED, "attn_decode: n_head * ceil((n_past + 1) / 128) * (head_dim + 4) floats of partial "
                                             "results must fit the context's 4 MB scratch block");
        part = (float *)ctx->scratch;
        done = ctx->attn_done;
    }
    GH_BIND(ctx);
    const dim3 grid((unsigned)S, (unsigned)n_head), block(AT_THREADS);
    if (head_dim == 128)
        hipLaunchKernelGGL((attn_decode_partial<32, CT>), grid, block, 0, ctx->stream, q, k, v, k_cache, v_cache, part, done,
                           out, n_head, L, pos, freq_scale, theta_scale, scale, key_stride, head_stride);
    else
        hipLaunchKernelGGL((attn_decode_partial<16, CT>), grid, block, 0, ctx->stream, q, k, v, k_cache, v_cache, part, done,
                           out, n_head, L, pos, freq_scale, theta_scale, scale, key_stride, head_stride);
    GH_LAUNCH_CHECK(ctx, what);
}

}  // namespace

// Called by galois_hip_create with the context's device current: where this device keeps its copy of `scratch`.
// (In host code the array's name is a handle for this lookup, not a device address.)
int32_t gh_attn_static_init(galois_hip_ctx *ctx) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return gh_hip(ctx, e, "hipGetSymbolAddress(attention scratch)");
    ctx->attn_static = p;
    return GALOIS_HIP_OK;
}

extern "C" int32_t galois_hip_attn_decode_f32_static(galois_hip_ctx *ctx, const float *q, const float *k, const float *v,
                                                     float *k_cache, float *v_cache, float *out, int32_t n_head,
                                                     int32_t head_dim, int32_t n_past, const int32_t *pos,
                                                     float freq_scale, float theta_scale, float scale, int32_t head_major_n_ctx) {
    return attn_decode_launch<float>(ctx, q, k, v, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale,
                                     theta_scale, scale, head_major_n_ctx, "attn_decode_f32_static", true);
}

extern "C" int32_t galois_hip_attn_decode_f32(galois_hip_ctx *ctx, const float *q, const float *k, const float *v,
                                              float *k_cache, float *v_cache, float *out, int32_t n_head,
                                              int32_t head_dim, int32_t n_past, const int32_t *pos, float freq_scale,
                                              float theta_scale, float scale, int32_t head_major_n_ctx) {
    return attn_decode_launch<float>(ctx, q, k, v, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale,
                                     theta_scale, scale, head_major_n_ctx, "attn_decode_f32");
}

extern "C" int32_t galois_hip_attn_decode_f16kv(galois_hip_ctx *ctx, const float *q, const float *k, const float *v,
                                                void *k_cache, void *v_cache, float *out, int32_t n_head,
                                                int32_t head_dim, int32_t n_past, const int32_t *pos, float freq_scale,
                                                float theta_scale, float scale, int32_t head_major_n_ctx) {
    return attn_decode_launch<_Float16>(ctx, q, k, v, (_Float16 *)k_cache, (_Float16 *)v_cache, out, n_head, head_dim,
                                        n_past, pos, freq_scale, theta_scale, scale, head_major_n_ctx, "attn_decode_f16kv");
}
