// The decode attention's workgroup: split s of head h over an f32 or f16 KV cache.  Included by the attention
// kernel proper (attn_decode.hip) and by the launch that also carries the q | k | v products (gemv_q4_0.hip).
#pragma once
#include "common.h"

namespace {

constexpr int AT_KEYS = 128;  // keys per workgroup (measured: 64 and, for an f16 cache, 256 are slower)

template <int CTRL>
__device__ __forceinline__ float at_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over aligned groups of LANES lanes (16 or 32); every lane of a group ends with its total.
template <int LANES>
__device__ __forceinline__ float at_group_sum(float v) {
    v += at_dpp<0xB1>(v);   // quad_perm(1,0,3,2)
    v += at_dpp<0x4E>(v);   // quad_perm(2,3,0,1)
    v += at_dpp<0x141>(v);  // row_half_mirror
    v += at_dpp<0x140>(v);  // row_mirror
    if (LANES >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

__device__ __forceinline__ float at_wave_max(float v) {
    v = fmaxf(v, at_dpp<0xB1>(v));
    v = fmaxf(v, at_dpp<0x4E>(v));
    v = fmaxf(v, at_dpp<0x141>(v));
    v = fmaxf(v, at_dpp<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

__device__ __forceinline__ float at_wave_sum(float v) {
    v += at_dpp<0xB1>(v);
    v += at_dpp<0x4E>(v);
    v += at_dpp<0x141>(v);
    v += at_dpp<0x140>(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// Rotation of the lane's two adjacent pairs (rope.cu:3-28, mode 0): pair i of the head by
// theta = pos * freq_scale * theta_scale^i.
struct at_rot {
    float c0, s0, c1, s1;
    // the same sequence of roundings as rope_rows (one product, then a fused multiply-add), spelled out so that the
    // compiler cannot contract the two kernels differently: the appended cache row equals rope_f32's output
    __device__ __forceinline__ float4 apply(float4 x) const {
        return make_float4(__builtin_fmaf(x.x, c0, -(x.y * s0)), __builtin_fmaf(x.x, s0, x.y * c0),
                           __builtin_fmaf(x.z, c1, -(x.w * s1)), __builtin_fmaf(x.z, s1, x.w * c1));
    }
};

// Device-coherent accesses to the split records: relaxed atomics of device scope are plain loads and stores that
// bypass the caches private to a CU or an XCD, so a record written on one XCD is read correctly on another
// without any cache being flushed.
__device__ __forceinline__ void at_store(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float at_load(const float *p) {
    return __hip_atomic_load(const_cast<float *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge of a head's splits, run by the workgroup that finishes the head's last split: thread d < D owns output
// element d.  The split maxima and sums are fetched by S threads at once and the weights exp(m_s - M) shared
// through LDS; the partial outputs are then read eight splits at a time.
constexpr int AT_MAX_SPLITS = 1024;
template <int AT_THREADS>
__device__ __forceinline__ void at_combine(const float *rec, float *__restrict__ out_h, int D, int S, float *w,
                                           float (*red)[AT_THREADS / 64]) {
    constexpr int WAVES = AT_THREADS / 64;
    const int d = threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (S <= 16) {
        // Few splits (up to 2048 keys): every thread fetches all maxima, sums and its own element of every partial
        // output in one go -- one trip to memory instead of three dependent ones, and no barrier.  Same order of
        // additions as the general path below.
        float ms[16], ss[16], os[16];
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const float *r = rec + (size_t)min(s, S - 1) * (D + 4);
            ms[s] = at_load(r), ss[s] = at_load(r + 1), os[s] = at_load(r + 4 + min(d, D - 1));
        }
        float M = ms[0];
#pragma unroll
        for (int s = 1; s < 16; s++) M = fmaxf(M, s < S ? ms[s] : M);
        float den = 0.0f, num = 0.0f;
#pragma unroll
        for (int s = 0; s < 16; s++)
            if (s < S) {
                const float ws = expf(ms[s] - M);
                den = __builtin_fmaf(ws, ss[s], den);
                num = __builtin_fmaf(ws, os[s], num);
            }
        if (d < D) out_h[d] = num / den;
        return;
    }
    float mx = -__builtin_inff();
    for (int s = d; s < S; s += AT_THREADS) {
        const float ms = at_load(rec + (size_t)s * (D + 4));
        w[s] = ms;
        mx = fmaxf(mx, ms);
    }
    mx = at_wave_max(mx);
    if (lane == 0) red[0][wave] = mx;
    __syncthreads();
    float M = red[0][0];
#pragma unroll
    for (int i = 1; i < WAVES; i++) M = fmaxf(M, red[0][i]);
    float den = 0.0f;
    for (int s = d; s < S; s += AT_THREADS) {
        const float ws = expf(w[s] - M);
        w[s] = ws;
        den = __builtin_fmaf(ws, at_load(rec + (size_t)s * (D + 4) + 1), den);
    }
    den = at_wave_sum(den);
    if (lane == 0) red[1][wave] = den;
    __syncthreads();
    den = red[1][0];
#pragma unroll
    for (int i = 1; i < WAVES; i++) den += red[1][i];
    if (d < D) {
        float num = 0.0f;
        for (int s0 = 0; s0 < S; s0 += 8) {
            float o[8];
#pragma unroll
            for (int j = 0; j < 8; j++) o[j] = at_load(rec + (size_t)min(s0 + j, S - 1) * (D + 4) + 4 + d);
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (s0 + j < S) num = __builtin_fmaf(w[s0 + j], o[j], num);
        }
        out_h[d] = num / den;
    }
}

// The lane's four consecutive cache elements, f32 or f16 (the reference keeps f16 caches on the GPU: cpy_f32_f16,
// src/cuda.rs:1382-1595, then gemm_ex with F16 operands, src/cuda.rs:881-992).  Rows appended to an f16 cache are
// rounded to nearest even, and this step's scores and outputs use the rounded row, as the op sequence would.
typedef _Float16 at_half4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 at_load4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ at_half4 at_load4(const _Float16 *p) { return *reinterpret_cast<const at_half4 *>(p); }
__device__ __forceinline__ float4 at_f32(float4 v) { return v; }
__device__ __forceinline__ float4 at_f32(at_half4 h) { return make_float4((float)h.x, (float)h.y, (float)h.z, (float)h.w); }
template <typename CT> struct at_raw { typedef float4 type; };
template <> struct at_raw<_Float16> { typedef at_half4 type; };
__device__ __forceinline__ float4 at_load4_rounded(float4 v) {  // v as an f16 cache returns it
    return make_float4((float)(_Float16)v.x, (float)(_Float16)v.y, (float)(_Float16)v.z, (float)(_Float16)v.w);
}
__device__ __forceinline__ float4 at_store4(float *p, float4 v) {
    *reinterpret_cast<float4 *>(p) = v;
    return v;
}
__device__ __forceinline__ float4 at_store4(_Float16 *p, float4 v) {
    const at_half4 h = {(_Float16)v.x, (_Float16)v.y, (_Float16)v.z, (_Float16)v.w};
    *reinterpret_cast<at_half4 *>(p) = h;
    return make_float4((float)h.x, (float)h.y, (float)h.z, (float)h.w);
}

// Bounded wait for a counter that other workgroups of the same launch advance (device-coherent reads).  The bound is
// never reached when the producers are dispatched ahead of the waiters; if it is, the caller poisons its result and
// raises the context's status word.
__device__ __forceinline__ bool at_wait_ge(const unsigned *p, unsigned target, int spin_limit) {
    for (int it = 0; it < spin_limit; it++) {
        if ((int)(__hip_atomic_load(const_cast<unsigned *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) >= 0) {
            asm volatile("" ::: "memory");  // what the producers wrote is read after this point
            return true;
        }
        __builtin_amdgcn_s_sleep(8);
    }
    return false;
}
__device__ __forceinline__ float4 at_load4_coherent(const float *p) {
    return make_float4(at_load(p), at_load(p + 1), at_load(p + 2), at_load(p + 3));
}

// The work of one workgroup: split s of head h (S splits per head).  Record of one (head, split) in the scratch
// block: m, sum, 2 unused floats, then head_dim partial outputs.
// Cache element (position l, head h, d) lies at l * key_stride + h * head_stride + d: (H * D, D) for caches kept
// [n_ctx][n_head * head_dim], (D, n_ctx * D) for caches kept [n_head][n_ctx][head_dim], where a workgroup's 128 keys
// are one contiguous 64 KB instead of 128 pieces of 512 bytes.
// FUSED: q, k and v are written by other workgroups of the same launch (the q | k | v products); ready[h],
// ready[H + h], ready[2 H + h] count the workgroups that have stored their rows of head h's q, k, v, and reach
// `target` when the head's rows are complete.  The cache rows are requested first, then the workgroup waits for q
// (and, if it holds position n_past, for k and v), which it reads with device-coherent loads.  The workgroup that
// merges a head returns the three counters to zero.  A wait that runs out (spin_limit polls) is agreed on by the whole
// workgroup: the head's record -- and with it the head's output, whichever workgroup merges it -- becomes NaN in
// every element, and *status (pinned host memory the context reads after its next wait for the stream) is set.
template <int LPR, typename CT, int AT_THREADS, bool FUSED>
__device__ __forceinline__ void attn_decode_wg(const float *__restrict__ q, const float *__restrict__ k,
                                               const float *__restrict__ v, CT *__restrict__ kc, CT *__restrict__ vc,
                                               float *__restrict__ part, unsigned *__restrict__ done,
                                               float *__restrict__ out, int H, int L, const int32_t *__restrict__ pos,
                                               float freq_scale, float theta_scale, float scale, int h, int s, int S,
                                               unsigned *ready, unsigned target, int64_t key_stride, int64_t head_stride,
                                               int spin_limit = 0, unsigned *status = nullptr) {
    constexpr int D = LPR * 4, RPL = 64 / LPR, WAVES = AT_THREADS / 64;
    constexpr int KEYS = AT_KEYS;
    constexpr int KPW = KEYS / WAVES;     // keys per wave
    constexpr int U = KPW / RPL;          // wave-loads per wave, all in flight
    constexpr bool F16 = sizeof(CT) == 2;
    __shared__ float sc[KEYS];
    __shared__ float4 ored[WAVES][LPR];
    __shared__ float sred[WAVES];
    __shared__ float cw[AT_MAX_SPLITS];
    __shared__ float cred[2][WAVES];
    __shared__ unsigned last_flag;
    __shared__ unsigned gave_up[WAVES];  // FUSED: per wave, whether any of its lanes gave up a wait
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / LPR, kl = lane % LPR;
    const int l0 = s * KEYS, l1 = min(L, l0 + KEYS), nl = l1 - l0;
    const size_t hoff = (size_t)h * D + kl * 4;                    // in q, k, v, out
    const size_t coff = (size_t)h * (size_t)head_stride + kl * 4;  // in the caches: element (l, h, d) at l * key_stride + h * head_stride + d
    const size_t E = (size_t)key_stride;

    const int lnew = L - 1;  // the position being appended
    const int kbase = l0 + wave * KPW + sub;

    // ---- every request of the workgroup goes out first: its keys and values as the cache holds them (row n_past
    // is not in the cache yet: what is read for it is replaced below by this step's k and v), then k, v and q;
    // the rotation is computed while they are in flight
    // FUSED: the counters are read ahead of the cache rows (loads return in order), so their values are known while
    // the rows are still in flight; in the usual case the producers finished long ago and nothing is waited for
    unsigned seen_q = 0, seen_k = 0, seen_v = 0;
    if (FUSED) {
        seen_q = __hip_atomic_load(ready + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (l1 - 1 == L - 1) {
            seen_k = __hip_atomic_load(ready + H + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            seen_v = __hip_atomic_load(ready + 2 * H + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    typename at_raw<CT>::type kv[U], vv[U];
#pragma unroll
    for (int u = 0; u < U; u++) kv[u] = at_load4(kc + (size_t)min(kbase + u * RPL, l1 - 1) * E + coff);
#pragma unroll
    for (int u = 0; u < U; u++) vv[u] = at_load4(vc + (size_t)min(kbase + u * RPL, l1 - 1) * E + coff);
    float4 knew_raw, vnew, qraw;
    if (!FUSED) {
        knew_raw = *reinterpret_cast<const float4 *>(k + hoff);
        vnew = *reinterpret_cast<const float4 *>(v + hoff);
        qraw = *reinterpret_cast<const float4 *>(q + hoff);
    }
    // this position's rotation for the lane's pairs 2 kl and 2 kl + 1
    at_rot rot;
    {
        const float p0 = (float)pos[0] * freq_scale;
        sincosf(p0 * powf(theta_scale, (float)(2 * kl)), &rot.s0, &rot.c0);
        sincosf(p0 * powf(theta_scale, (float)(2 * kl + 1)), &rot.s1, &rot.c1);
    }
    bool arrived = true;
    if (FUSED) {
        arrived = (int)(seen_q - target) >= 0 || at_wait_ge(ready + h, target, spin_limit);
        asm volatile("" ::: "memory");
        qraw = at_load4_coherent(q + hoff);
        knew_raw = vnew = make_float4(0.f, 0.f, 0.f, 0.f);
        if (l1 - 1 == lnew) {  // the workgroup that holds the new position
            arrived &= (int)(seen_k - target) >= 0 || at_wait_ge(ready + H + h, target, spin_limit);
            arrived &= (int)(seen_v - target) >= 0 || at_wait_ge(ready + 2 * H + h, target, spin_limit);
            asm volatile("" ::: "memory");
            knew_raw = at_load4_coherent(k + hoff);
            vnew = at_load4_coherent(v + hoff);
        }
    }
    if (FUSED) {  // published by the barrier behind the scores; read where the record is written
        const bool wave_gave_up = __builtin_amdgcn_ballot_w64(!arrived) != 0;
        if (lane == 0) {
            gave_up[wave] = wave_gave_up;
            if (wave_gave_up) __hip_atomic_fetch_or(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
    const float4 qv = rot.apply(qraw);
    float4 knew = rot.apply(knew_raw);
    if (F16) {  // what an f16 cache will hold
        // the rotation's f32 result is rounded again to f16, as a cpy of rope_custom's output is; without the
        // barrier the compiler folds rotation and conversion into one mixed-precision fma (one rounding)
        asm volatile("" : "+v"(knew.x), "+v"(knew.y), "+v"(knew.z), "+v"(knew.w));
        knew = at_load4_rounded(knew);
        vnew = at_load4_rounded(vnew);
    }

    // ---- scores of the workgroup's keys
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int l = kbase + u * RPL;
        float4 kf = at_f32(kv[u]);
        if (min(l, l1 - 1) == lnew) {  // the new key; the lanes that own it write both cache rows
            kf = knew;
            if (l == lnew) {
                at_store4(kc + (size_t)lnew * E + coff, knew);
                at_store4(vc + (size_t)lnew * E + coff, vnew);
            }
        }
        float acc = kf.x * qv.x;
        acc = __builtin_fmaf(kf.y, qv.y, acc);
        acc = __builtin_fmaf(kf.z, qv.z, acc);
        acc = __builtin_fmaf(kf.w, qv.w, acc);
        acc = at_group_sum<LPR>(acc);
        if (kl == 0) sc[wave * KPW + u * RPL + sub] = acc * scale;
    }
    __syncthreads();

    // ---- softmax numerators relative to the workgroup's own maximum
    float m = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < KEYS; i += 64) m = fmaxf(m, lane + i < nl ? sc[lane + i] : -__builtin_inff());
    m = at_wave_max(m);
    __syncthreads();  // every wave has read the scores
#pragma unroll
    for (int i = 0; i < KEYS; i += AT_THREADS) {
        const int j = (int)threadIdx.x + i;
        if (j < KEYS) sc[j] = j < nl ? expf(sc[j] - m) : 0.0f;
    }
    __syncthreads();

    // ---- partial output: sum of p * v over the workgroup's keys (p is 0 for keys past the end)
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const float p = sc[wave * KPW + u * RPL + sub];
        const float4 vf = min(kbase + u * RPL, l1 - 1) == lnew ? vnew : at_f32(vv[u]);
        acc.x = __builtin_fmaf(vf.x, p, acc.x);
        acc.y = __builtin_fmaf(vf.y, p, acc.y);
        acc.z = __builtin_fmaf(vf.z, p, acc.z);
        acc.w = __builtin_fmaf(vf.w, p, acc.w);
    }
    // the RPL keys of a wave-load sit LPR lanes apart
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off, 64);
        acc.y += __shfl_xor(acc.y, off, 64);
        acc.z += __shfl_xor(acc.z, off, 64);
        acc.w += __shfl_xor(acc.w, off, 64);
    }
    if (lane < LPR) ored[wave][lane] = acc;
    float psum = 0.0f;
#pragma unroll
    for (int i = 0; i < KEYS; i += 64) psum += lane + i < nl ? sc[lane + i] : 0.0f;
    psum = at_wave_sum(psum);
    if (lane == 0) sred[wave] = psum;  // every wave holds the same total; wave 0's is used
    __syncthreads();
    if (wave == 0 && lane < LPR) {
        float4 o = ored[0][lane];
#pragma unroll
        for (int w = 1; w < WAVES; w++) {
            const float4 t = ored[w][lane];
            o.x += t.x, o.y += t.y, o.z += t.z, o.w += t.w;
        }
        float tot = sred[0];
        if (FUSED) {  // a producer never arrived for some lane of the workgroup: the head's output is poisoned
            unsigned any = 0;
#pragma unroll
            for (int w = 0; w < WAVES; w++) any |= gave_up[w];
            if (any) tot = __builtin_nanf("");
        }
        if (S == 1) {  // a single split is the whole softmax
            const float inv = 1.0f / tot;
            *reinterpret_cast<float4 *>(out + (size_t)h * D + lane * 4) = make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
        } else {
            // The record goes out as device-coherent stores (they bypass the XCD-local caches) and is waited for
            // before the split is counted; a device-wide fence here would write back and invalidate the whole L2
            // once per workgroup (measured: the kernel takes almost three times as long).
            float *rec = part + ((size_t)h * S + s) * (D + 4);
            if (lane == 0) at_store(rec, m), at_store(rec + 1, tot);
            at_store(rec + 4 + lane * 4, o.x), at_store(rec + 5 + lane * 4, o.y);
            at_store(rec + 6 + lane * 4, o.z), at_store(rec + 7 + lane * 4, o.w);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }
    if (S == 1) {
        if (FUSED && threadIdx.x == 0) ready[h] = 0, ready[H + h] = 0, ready[2 * H + h] = 0;  // every thread is past its waits
        return;
    }
    // The workgroup that counts the head's last split merges all of them (no second launch).  The counter
    // returns to zero for the next call.
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned prev = atomicAdd(done + h, 1u);
        last_flag = prev == (unsigned)(S - 1);
        if (last_flag) {
            done[h] = 0;
            if (FUSED) ready[h] = 0, ready[H + h] = 0, ready[2 * H + h] = 0;
        }
    }
    __syncthreads();
    if (!last_flag) return;
    at_combine<AT_THREADS>(part + (size_t)h * S * (D + 4), out + (size_t)h * D, D, S, cw, cred);
}

}  // namespace
