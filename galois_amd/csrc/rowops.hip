// Single-pass row kernels for gfx950: RMSNorm (+ fused weight), RoPE, softmax (+ causal).
// Each reads its input once from HBM and writes its output once; rows live in registers.
#include "common.h"

namespace {

// Results leave through streaming (non-temporal) stores: nothing in these launches reads them again, and lines that
// are not left dirty in the L2 caches do not have to be written back when the kernel ends (measured on the three
// kernels at the benchmark's sizes: 4.64 -> 4.20, 4.19 -> 4.04 and 9.93 -> 8.79 us; non-temporal LOADS cost 7-20 %).
typedef float rv4 __attribute__((ext_vector_type(4)));
typedef float rv2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void st4(float *p, float4 v) {
    __builtin_nontemporal_store(rv4{v.x, v.y, v.z, v.w}, reinterpret_cast<rv4 *>(p));
}
__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ void st2(float *p, float2 v) {
    __builtin_nontemporal_store(rv2{v.x, v.y}, reinterpret_cast<rv2 *>(p));
}
__device__ __forceinline__ float2 ld2(const float *p) { return *reinterpret_cast<const float2 *>(p); }

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm(1,0,3,2)
    v += dpp_mov<0x4E>(v);   // quad_perm(2,3,0,1)
    v += dpp_mov<0x141>(v);  // row_half_mirror
    v += dpp_mov<0x140>(v);  // row_mirror
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_mov<0xB1>(v));
    v = fmaxf(v, dpp_mov<0x4E>(v));
    v = fmaxf(v, dpp_mov<0x141>(v));
    v = fmaxf(v, dpp_mov<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// ------------------------------------------------------------------ RMSNorm
// rms_norm_f32 (galois-kernels/src/rms_norm.cu:13-49) with the optional broadcast
// weight of mul_f32 (mul.cu:3-12) fused in.  One workgroup per row; the row is read once into registers
// (NV float4 per thread), reduced, scaled and written with streaming stores.  Measured on 512 rows of 4096:
// 512 threads per row 4.05 us, 256 threads 4.19 us, two rows per workgroup sharing the weight 4.57 us.
constexpr int kNormThreads = 256;    // of the generic kernel
constexpr int kNormRowThreads = 512;

template <int NV>
__global__ __launch_bounds__(kNormRowThreads) void rms_norm_rows(const float *__restrict__ x, const float *__restrict__ w,
                                                                 float *__restrict__ y, int ncols, float eps) {
    constexpr int THREADS = kNormRowThreads;
    __shared__ float part[THREADS / 64];
    const size_t base = (size_t)blockIdx.x * ncols;
    const int nvec = ncols >> 2;
    float4 v[NV], g[NV];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = threadIdx.x + i * THREADS;
        v[i] = c < nvec ? ld4(x + base + 4 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    // the weight is requested behind the row, before the reduction, so that nothing waits for it afterwards
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = threadIdx.x + i * THREADS;
        g[i] = (w && c < nvec) ? reinterpret_cast<const float4 *>(w)[c] : make_float4(1.f, 1.f, 1.f, 1.f);
    }
#pragma unroll
    for (int i = 0; i < NV; i++) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < THREADS / 64; i++) tot += part[i];
    const float scale = 1.0f / sqrtf(tot / (float)ncols + eps);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = threadIdx.x + i * THREADS;
        if (c < nvec) {
            float4 o = make_float4(v[i].x * scale, v[i].y * scale, v[i].z * scale, v[i].w * scale);
            if (w) o.x *= g[i].x, o.y *= g[i].y, o.z *= g[i].z, o.w *= g[i].w;
            st4(y + base + 4 * c, o);
        }
    }
}

// Any ncols / alignment: the row is read twice (the second read hits L2).
__global__ __launch_bounds__(kNormThreads) void rms_norm_rows_generic(const float *__restrict__ x,
                                                                      const float *__restrict__ w,
                                                                      float *__restrict__ y, int ncols, float eps) {
    __shared__ float part[kNormThreads / 64];
    const size_t base = (size_t)blockIdx.x * ncols;
    float ss = 0.0f;
    for (int c = threadIdx.x; c < ncols; c += kNormThreads) ss += x[base + c] * x[base + c];
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormThreads / 64; i++) tot += part[i];
    const float scale = 1.0f / sqrtf(tot / (float)ncols + eps);
    for (int c = threadIdx.x; c < ncols; c += kNormThreads) {
        float o = x[base + c] * scale;
        if (w) o *= w[c];
        y[base + c] = o;
    }
}

int32_t launch_rms_norm(galois_hip_ctx *ctx, const float *x, const float *w, float *dst, int32_t ncols,
                        int32_t nrows, float eps, const char *what) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && dst, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, ncols > 0 && nrows > 0, GALOIS_HIP_E_SHAPE, what);
    GH_REQUIRE(ctx, gh_aligned(x, 4) && gh_aligned(dst, 4) && gh_aligned(w, 4), GALOIS_HIP_E_ALIGN, what);
    GH_BIND(ctx);
    const bool vec = ncols % 4 == 0 && gh_aligned(x, 16) && gh_aligned(dst, 16) && gh_aligned(w, 16);
    const int nv = (ncols / 4 + kNormRowThreads - 1) / kNormRowThreads;
    const dim3 grid(nrows), block(kNormRowThreads);
    if (vec && nv <= 1)
        hipLaunchKernelGGL(rms_norm_rows<1>, grid, block, 0, ctx->stream, x, w, dst, ncols, eps);
    else if (vec && nv <= 2)
        hipLaunchKernelGGL(rms_norm_rows<2>, grid, block, 0, ctx->stream, x, w, dst, ncols, eps);
    else if (vec && nv <= 4)
        hipLaunchKernelGGL(rms_norm_rows<4>, grid, block, 0, ctx->stream, x, w, dst, ncols, eps);
    else if (vec && nv <= 8)
        hipLaunchKernelGGL(rms_norm_rows<8>, grid, block, 0, ctx->stream, x, w, dst, ncols, eps);
    else
        hipLaunchKernelGGL(rms_norm_rows_generic, grid, dim3(kNormThreads), 0, ctx->stream, x, w, dst, ncols, eps);
    GH_LAUNCH_CHECK(ctx, what);
}

// ------------------------------------------------------------------ RoPE
// rope_f32 (galois-kernels/src/rope.cu:3-28): adjacent pairs, one position per group of
// p_delta_rows consecutive rows.  One workgroup per position group; a lane computes
// sin/cos for its pair index once and reuses it for every row (head) of the group, so
// the transcendental cost is shared by all heads.  theta follows the reference formula
// in f32: pos * freq_scale * powf(theta_scale, pair).
constexpr int kRopeThreads = 256;

// Rows of up to 256 columns, 16-byte aligned: a lane owns two adjacent pairs (16 bytes), half a wave covers a row of
// 128 columns, so a wave-load is whole rows in 16-byte pieces (512 positions x 32 heads x 128: 3.59 us against 4.04 us
// for the 8-byte pieces of rope_rows below, which serves every other shape).
template <int LPR>  // lanes per row: ncols / 4 rounded up to 16, 32 or 64
__global__ __launch_bounds__(kRopeThreads) void rope_rows4(const float *__restrict__ x, float *__restrict__ y, int ncols,
                                                           int nrows, const int32_t *__restrict__ pos, float freq_scale,
                                                           int p_delta_rows, float theta_scale) {
    constexpr int RPW = 64 / LPR;                  // rows per wave-load
    constexpr int RS = (kRopeThreads / 64) * RPW;  // rows per workgroup-load
    constexpr int RU = 4;
    const int group = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / LPR, c4 = lane % LPR;   // row within the wave-load, 16-byte piece within the row
    const bool live = c4 * 4 < ncols;
    const int row_lo = group * p_delta_rows;
    const int row_hi = min(row_lo + p_delta_rows, nrows);
    const float p0 = (float)pos[group] * freq_scale;
    int r = row_lo + wave * RPW + sub;
    float4 first[RU];
    const bool have_first = r - sub + (RU - 1) * RS + RPW - 1 < row_hi;  // wave-uniform: all RU loads are whole
    if (have_first && live) {
#pragma unroll
        for (int u = 0; u < RU; u++) first[u] = ld4(x + (size_t)(r + u * RS) * ncols + 4 * c4);
    }
    float s0, c0, s1, c1;
    sincosf(p0 * powf(theta_scale, (float)(2 * c4)), &s0, &c0);
    sincosf(p0 * powf(theta_scale, (float)(2 * c4 + 1)), &s1, &c1);
    auto rot = [&](float4 v) {
        return make_float4(__builtin_fmaf(v.x, c0, -(v.y * s0)), __builtin_fmaf(v.x, s0, v.y * c0),
                           __builtin_fmaf(v.z, c1, -(v.w * s1)), __builtin_fmaf(v.z, s1, v.w * c1));
    };
    if (!live) return;
    bool use_first = have_first;
    for (; r - sub + (RU - 1) * RS + RPW - 1 < row_hi; r += RU * RS) {
        float4 v[RU];
#pragma unroll
        for (int u = 0; u < RU; u++) v[u] = use_first ? first[u] : ld4(x + (size_t)(r + u * RS) * ncols + 4 * c4);
        use_first = false;
#pragma unroll
        for (int u = 0; u < RU; u++) st4(y + (size_t)(r + u * RS) * ncols + 4 * c4, rot(v[u]));
    }
    for (; r < row_hi; r += RS) st4(y + (size_t)r * ncols + 4 * c4, rot(ld4(x + (size_t)r * ncols + 4 * c4)));
}


// rope_custom of the q and the k rows of many tokens and the append of k and v to the cache rows of those tokens, one
// launch: one workgroup per token; sin / cos of a lane's two pairs are computed once (the formula of rope_rows4) and
// serve the token's q rows and k rows alike.  q goes rotated to qo (f32); k rotated to kd and, when v is given, v
// unchanged to vd: f32, or f16 rounded to nearest even (cpy_f32_f16, cpy.cu:79-156, into an f16 cache).
template <int LPR, bool KV16>
__global__ __launch_bounds__(kRopeThreads) void rope_qk_append_rows4(const float *__restrict__ q, const float *__restrict__ k,
                                                                     const float *__restrict__ v, float *__restrict__ qo,
                                                                     void *__restrict__ kd, void *__restrict__ vd, int head_dim,
                                                                     int n_head, const int32_t *__restrict__ pos,
                                                                     float freq_scale, float theta_scale) {
    constexpr int RPW = 64 / LPR;                  // rows per wave-load
    constexpr int RS = (kRopeThreads / 64) * RPW;  // rows per workgroup-load
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / LPR, c4 = lane % LPR;
    if (c4 * 4 >= head_dim) return;
    const size_t tok = (size_t)blockIdx.x * n_head * head_dim;
    const float p0 = (float)pos[blockIdx.x] * freq_scale;
    float s0, c0, s1, c1;
    sincosf(p0 * powf(theta_scale, (float)(2 * c4)), &s0, &c0);
    sincosf(p0 * powf(theta_scale, (float)(2 * c4 + 1)), &s1, &c1);
    auto rot = [&](float4 x) {
        return make_float4(__builtin_fmaf(x.x, c0, -(x.y * s0)), __builtin_fmaf(x.x, s0, x.y * c0),
                           __builtin_fmaf(x.z, c1, -(x.w * s1)), __builtin_fmaf(x.z, s1, x.w * c1));
    };
    auto put = [&](void *dst, size_t at, float4 x) {
        if (KV16) {
            // the rotation's f32 results first, then their rounding to f16, as the two ops would do it: left to the
            // compiler the multiply-add and the conversion become one instruction with a single rounding
            asm volatile("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w));
            typedef _Float16 h4 __attribute__((ext_vector_type(4)));
            __builtin_nontemporal_store(h4{(_Float16)x.x, (_Float16)x.y, (_Float16)x.z, (_Float16)x.w},
                                        reinterpret_cast<h4 *>(static_cast<_Float16 *>(dst) + at));
        } else {
            st4(static_cast<float *>(dst) + at, x);
        }
    };
    for (int r = wave * RPW + sub; r < n_head; r += RS) {
        const size_t at = tok + (size_t)r * head_dim + 4 * c4;
        const float4 a = ld4(q + at), b = ld4(k + at);
        float4 c = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v) c = ld4(v + at);
        st4(qo + at, rot(a));
        put(kd, at, rot(b));
        if (v) put(vd, at, c);
    }
}

__global__ __launch_bounds__(kRopeThreads) void rope_rows(const float *__restrict__ x, float *__restrict__ y,
                                                          int ncols, int nrows, const int32_t *__restrict__ pos,
                                                          float freq_scale, int p_delta_rows, float theta_scale) {
    const int group = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int npairs = ncols >> 1;
    const int row_lo = group * p_delta_rows;
    const int row_hi = min(row_lo + p_delta_rows, nrows);
    const float p0 = (float)pos[group] * freq_scale;
    for (int pi = lane; pi < npairs; pi += 64) {
        int r = row_lo + wave;
        // RU rows in flight per lane; the first RU are requested before the angle's sine and cosine are computed
        // (a few hundred instructions), so the arithmetic runs while they are in flight
        constexpr int RU = 4, RS = kRopeThreads / 64;
        float2 first[RU];
        const bool have_first = r + (RU - 1) * RS < row_hi;  // wave-uniform
        if (have_first) {
#pragma unroll
            for (int u = 0; u < RU; u++) first[u] = ld2(x + (size_t)(r + u * RS) * ncols + 2 * pi);
        }
        const float theta = p0 * powf(theta_scale, (float)pi);
        float sn, cs;
        sincosf(theta, &sn, &cs);
        bool use_first = have_first;
        for (; r + (RU - 1) * RS < row_hi; r += RU * RS) {
            float2 v[RU];
#pragma unroll
            for (int u = 0; u < RU; u++)
                v[u] = use_first ? first[u] : ld2(x + (size_t)(r + u * RS) * ncols + 2 * pi);
            use_first = false;
#pragma unroll
            for (int u = 0; u < RU; u++)
                st2(y + (size_t)(r + u * RS) * ncols + 2 * pi,
                    make_float2(__builtin_fmaf(v[u].x, cs, -(v[u].y * sn)), __builtin_fmaf(v[u].x, sn, v[u].y * cs)));
        }
        for (; r < row_hi; r += kRopeThreads / 64) {
            const float2 v = reinterpret_cast<const float2 *>(x + (size_t)r * ncols)[pi];
            reinterpret_cast<float2 *>(y + (size_t)r * ncols)[pi] =
                make_float2(__builtin_fmaf(v.x, cs, -(v.y * sn)), __builtin_fmaf(v.x, sn, v.y * cs));
        }
    }
}

// ------------------------------------------------------------------ softmax
// soft_max_f32 (galois-kernels/src/softmax.cu:3-48): f32 row softmax, -inf inputs are
// masked.  One wave per row, the row held in registers (NV float4 per lane): one read,
// one write.  `causal` computes the mask from indices instead: row r keeps columns
// <= n_past + (r % rows_per_head); masked inputs are not read and their outputs are 0.
constexpr int kSoftThreads = 256;

template <int NV>
__global__ __launch_bounds__(kSoftThreads) void soft_max_rows(const float *__restrict__ x, float *__restrict__ y,
                                                              int ncols, int nrows, int causal, int rows_per_head,
                                                              int n_past) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (kSoftThreads / 64) + (threadIdx.x >> 6);
    if (row >= nrows) return;
    const int nvalid = causal ? min(ncols, n_past + (row % rows_per_head) + 1) : ncols;
    const size_t base = (size_t)row * ncols;
    const float ninf = -__builtin_inff();
    float4 v[NV];
    float mx = ninf;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = (lane + i * 64) * 4;
        if (c < nvalid) {
            v[i] = ld4(x + base + c);
            if (c + 1 >= nvalid) v[i].y = ninf;
            if (c + 2 >= nvalid) v[i].z = ninf;
            if (c + 3 >= nvalid) v[i].w = ninf;
        } else {
            v[i] = make_float4(ninf, ninf, ninf, ninf);
        }
        mx = fmaxf(mx, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        v[i].x = expf(v[i].x - mx);
        v[i].y = expf(v[i].y - mx);
        v[i].z = expf(v[i].z - mx);
        v[i].w = expf(v[i].w - mx);
        sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = (lane + i * 64) * 4;
        if (c < ncols)
            st4(y + base + c, make_float4(v[i].x * inv, v[i].y * inv, v[i].z * inv, v[i].w * inv));
    }
}

// Any ncols / alignment: one workgroup per row, three passes (re-reads hit L2).
__global__ __launch_bounds__(kSoftThreads) void soft_max_rows_generic(const float *__restrict__ x,
                                                                      float *__restrict__ y, int ncols, int causal,
                                                                      int rows_per_head, int n_past) {
    __shared__ float part[kSoftThreads / 64];
    const int row = blockIdx.x;
    const int nvalid = causal ? min(ncols, n_past + (row % rows_per_head) + 1) : ncols;
    const size_t base = (size_t)row * ncols;
    float mx = -__builtin_inff();
    for (int c = threadIdx.x; c < nvalid; c += kSoftThreads) mx = fmaxf(mx, x[base + c]);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = part[0];
#pragma unroll
    for (int i = 1; i < kSoftThreads / 64; i++) mx = fmaxf(mx, part[i]);
    __syncthreads();
    float sum = 0.0f;
    for (int c = threadIdx.x; c < nvalid; c += kSoftThreads) sum += expf(x[base + c] - mx);
    sum = wave_sum(sum);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sum;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < kSoftThreads / 64; i++) tot += part[i];
    const float inv = 1.0f / tot;
    for (int c = threadIdx.x; c < ncols; c += kSoftThreads)
        y[base + c] = c < nvalid ? expf(x[base + c] - mx) * inv : 0.0f;
}

int32_t launch_soft_max(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols, int32_t nrows, int causal,
                        int32_t rows_per_head, int32_t n_past, const char *what) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && dst, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, ncols > 0 && nrows > 0, GALOIS_HIP_E_SHAPE, what);
    GH_REQUIRE(ctx, !causal || (rows_per_head > 0 && n_past >= 0), GALOIS_HIP_E_SHAPE, what);
    GH_REQUIRE(ctx, gh_aligned(x, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN, what);
    GH_BIND(ctx);
    const bool vec = ncols % 4 == 0 && gh_aligned(x, 16) && gh_aligned(dst, 16);
    const int nv = (ncols / 4 + 63) / 64;
    const dim3 grid((nrows + kSoftThreads / 64 - 1) / (kSoftThreads / 64)), block(kSoftThreads);
#define GH_SOFT(NV) \
    hipLaunchKernelGGL(soft_max_rows<NV>, grid, block, 0, ctx->stream, x, dst, ncols, nrows, causal, rows_per_head, n_past)
    if (vec && nv <= 1)
        GH_SOFT(1);
    else if (vec && nv <= 2)
        GH_SOFT(2);
    else if (vec && nv <= 4)
        GH_SOFT(4);
    else if (vec && nv <= 8)
        GH_SOFT(8);
    else if (vec && nv <= 16)
        GH_SOFT(16);
    else
        hipLaunchKernelGGL(soft_max_rows_generic, dim3(nrows), block, 0, ctx->stream, x, dst, ncols, causal,
                           rows_per_head, n_past);
#undef GH_SOFT
    GH_LAUNCH_CHECK(ctx, what);
}

}  // namespace

extern "C" {

int32_t galois_hip_rms_norm_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols, int32_t nrows,
                                float eps) {
    return launch_rms_norm(ctx, x, nullptr, dst, ncols, nrows, eps, "rms_norm_f32");
}

int32_t galois_hip_rms_norm_mul_f32(galois_hip_ctx *ctx, const float *x, const float *weight, float *dst,
                                    int32_t ncols, int32_t nrows, float eps) {
    if (ctx && !weight) return gh_fail(ctx, GALOIS_HIP_E_NULL, "rms_norm_mul_f32: weight");
    return launch_rms_norm(ctx, x, weight, dst, ncols, nrows, eps, "rms_norm_mul_f32");
}

int32_t galois_hip_rope_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols, int32_t nrows,
                            const int32_t *pos, float freq_scale, int32_t p_delta_rows, float theta_scale) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, x && dst && pos, GALOIS_HIP_E_NULL, "rope_f32");
    GH_REQUIRE(ctx, ncols > 0 && ncols % 2 == 0 && nrows > 0 && p_delta_rows > 0, GALOIS_HIP_E_SHAPE,
               "rope_f32: ncols must be even and positive, nrows and p_delta_rows positive");
    GH_REQUIRE(ctx, gh_aligned(x, 8) && gh_aligned(dst, 8) && gh_aligned(pos, 4), GALOIS_HIP_E_ALIGN, "rope_f32");
    GH_BIND(ctx);
    const int groups = (nrows + p_delta_rows - 1) / p_delta_rows;
    if (ncols % 4 == 0 && ncols <= 256 && gh_aligned(x, 16) && gh_aligned(dst, 16)) {
#define GH_ROPE4(LPR) \
    hipLaunchKernelGGL(rope_rows4<LPR>, dim3(groups), dim3(kRopeThreads), 0, ctx->stream, x, dst, ncols, nrows, pos, \
                       freq_scale, p_delta_rows, theta_scale)
        if (ncols <= 64) GH_ROPE4(16);
        else if (ncols <= 128) GH_ROPE4(32);
        else GH_ROPE4(64);
#undef GH_ROPE4
        GH_LAUNCH_CHECK(ctx, "rope_f32 launch");
    }
    hipLaunchKernelGGL(rope_rows, dim3(groups), dim3(kRopeThreads), 0, ctx->stream, x, dst, ncols, nrows, pos,
                       freq_scale, p_delta_rows, theta_scale);
    GH_LAUNCH_CHECK(ctx, "rope_f32 launch");
}

int32_t galois_hip_rope_qk_append(galois_hip_ctx *ctx, const float *q, const float *k, const float *v, float *q_out, void *k_rows,
                                  void *v_rows, int32_t kv_f16, int32_t head_dim, int32_t n_head, int32_t n_tokens,
                                  const int32_t *pos, float freq_scale, float theta_scale) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, q && k && q_out && k_rows && pos && ((v != nullptr) == (v_rows != nullptr)), GALOIS_HIP_E_NULL,
               "rope_qk_append: q, k, q_out, k_rows, pos; v and v_rows together or neither");
    GH_REQUIRE(ctx, head_dim > 0 && head_dim % 4 == 0 && head_dim <= 256 && n_head > 0 && n_tokens > 0, GALOIS_HIP_E_SHAPE,
               "rope_qk_append: head_dim a multiple of 4 up to 256, n_head and n_tokens positive");
    GH_REQUIRE(ctx, gh_aligned(q, 16) && gh_aligned(k, 16) && gh_aligned(v, 16) && gh_aligned(q_out, 16) && gh_aligned(k_rows, 16) &&
                        gh_aligned(v_rows, 16) && gh_aligned(pos, 4), GALOIS_HIP_E_ALIGN, "rope_qk_append: 16-byte aligned tensors");
    GH_BIND(ctx);
#define GH_ROPE_QK(LPR)                                                                                                      \
    do {                                                                                                                     \
        if (kv_f16)                                                                                                          \
            hipLaunchKernelGGL((rope_qk_append_rows4<LPR, true>), dim3(n_tokens), dim3(kRopeThreads), 0, ctx->stream, q, k, v, q_out, \
                               k_rows, v_rows, head_dim, n_head, pos, freq_scale, theta_scale);                              \
        else                                                                                                                 \
            hipLaunchKernelGGL((rope_qk_append_rows4<LPR, false>), dim3(n_tokens), dim3(kRopeThreads), 0, ctx->stream, q, k, v, q_out, \
                               k_rows, v_rows, head_dim, n_head, pos, freq_scale, theta_scale);                              \
    } while (0)
    if (head_dim <= 64) GH_ROPE_QK(16);
    else if (head_dim <= 128) GH_ROPE_QK(32);
    else GH_ROPE_QK(64);
#undef GH_ROPE_QK
    GH_LAUNCH_CHECK(ctx, "rope_qk_append launch");
}

int32_t galois_hip_soft_max_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols, int32_t nrows) {
    return launch_soft_max(ctx, x, dst, ncols, nrows, 0, 1, 0, "soft_max_f32");
}

int32_t galois_hip_soft_max_causal_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols,
                                       int32_t rows_per_head, int32_t nrows, int32_t n_past) {
    return launch_soft_max(ctx, x, dst, ncols, nrows, 1, rows_per_head, n_past, "soft_max_causal_f32");
}

}  // extern "C"
