// Q4_0 x f32 matrix-vector product for decode: an HBM-bandwidth kernel for gfx950.
//
// Replaces dequantize_mul_mat_vec_q4_0 (galois-kernels/src/matmul.cu:45-117) and its
// launcher (src/cuda.rs:1011-1034): dst[row] = sum_col (q-8)*d * y[col].
//
// Layout of the work.  Two consecutive 18-byte blocks form a 36-byte "slot" that is
// 4-byte aligned whenever K % 64 == 0, so a lane fetches one slot of one row with
// dwordx4 + dwordx4 + dword loads and the 64 lanes of a wave cover 2304 contiguous
// bytes (4096 weights) of that row.  The weight nibbles are never unpacked: a dword of
// eight nibbles, XORed with 0x88888888 (which turns q into the 4-bit two's complement
// of q-8), goes straight into v_dot8_i32_i4 against a dword holding one signed 4-bit
// digit of eight activations.  The activations are converted once per workgroup into
// block-scaled fixed point, split into L such digit planes (gemv_xprep.h) and kept in
// registers for every row the wave owns.  Per block the integer sum is exact; it is
// converted to f32 once and multiplied by the block's power-of-two activation scale
// and the f16 weight scale d.
#include "common.h"
#include "gemv_xprep.h"
#include "attn_decode_body.h"

namespace {

constexpr int kChunkSlots = 192;  // slots staged per pass over LDS (12288 activations)

struct __attribute__((aligned(4))) q4_slot {
    uint32_t w[9];  // [d0 | qs0[0..1]] [qs0 2..5] [6..9] [10..13] [qs0 14..15 | d1] [qs1 0..3] .. [qs1 12..15]
};

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes of a wave; every lane ends with the total.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm(1,0,3,2)
    v += dpp_mov<0x4E>(v);   // quad_perm(2,3,0,1)
    v += dpp_mov<0x141>(v);  // row_half_mirror
    v += dpp_mov<0x140>(v);  // row_mirror
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

__device__ __forceinline__ void load_slot(q4_slot &q, const uint8_t *p) {
    const uint32_t *s = reinterpret_cast<const uint32_t *>(p);
#pragma unroll
    for (int i = 0; i < 9; i++) q.w[i] = s[i];  // plain loads: the three loads of a lane share cache lines
}

// LDS image of one prepared slot: L planes x 8 dwords, then the two block scales and the two scales of the
// blocks' corrections (0 = the block has none).  The correction planes (gemv_xprep.h) of all slots follow the
// slots: corr_dwords per slot.
template <int L>
struct slot_lds {
    static constexpr int dwords = 8 * L + 4;  // stride = 4 (mod 8): 16-byte reads of 8 lanes hit 32 distinct banks
    static constexpr int corr_dwords = 8 * xprep::CORR_L;
    static constexpr int bytes_per_slot = (dwords + corr_dwords) * 4;  // what a launch reserves per slot
};

// Sum over the 64 lanes of a wave with DPP only; the total lands in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v += dpp_mov<0x111>(v);  // row_shr:1
    v += dpp_mov<0x112>(v);  // row_shr:2
    v += dpp_mov<0x114>(v);  // row_shr:4
    v += dpp_mov<0x118>(v);  // row_shr:8  -> lane 15 of each row holds the row total
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));  // row_bcast:15
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));  // row_bcast:31
    return v;
}

template <int CTRL>
__device__ __forceinline__ uint32_t quad_max(uint32_t v) {
    return max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true));
}

// Eight activations of one (slot, weight-dword group) task, in the nibble order of their weight dword, to LDS:
// the L planes, the block's scale, and -- when the fixed point leaves too much of the block behind -- the
// correction planes of the residuals with their scale.  The four threads of a quad hold one block.
// refetch(y8) produces the eight activations once more: the rare path takes them from where they came from
// rather than keep them in registers past the planes, which would cost the common path its occupancy.
template <int L, class Refetch>
__device__ __forceinline__ void prep_store(const float (&x8)[8], uint32_t *slot_dst, uint32_t *corr_dst, int g,
                                           Refetch refetch) {
    // max of |x| on the bit patterns: for non-negative floats the unsigned order is the numeric
    // order, with inf and NaN on top, so a non-finite activation is never lost
    uint32_t amax = 0;
    float sum_x = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        amax = max(amax, __builtin_bit_cast(uint32_t, x8[j]) & 0x7FFFFFFFu);
        sum_x += __builtin_fabsf(x8[j]);
    }
    amax = quad_max<0xB1>(amax), sum_x += dpp_mov<0xB1>(sum_x);  // quad_perm(1,0,3,2)
    amax = quad_max<0x4E>(amax), sum_x += dpp_mov<0x4E>(sum_x);  // quad_perm(2,3,0,1)
    float mult, scale;
    xprep::block_scales<L>(amax, &mult, &scale);
    uint32_t planes[L];
    xprep::make_planes<L>(x8, mult, planes);
#pragma unroll
    for (int l = 0; l < L; l++) slot_dst[l * 8 + g] = planes[l];
    float scale2 = 0.0f;
    if (xprep::needs_correction(sum_x, amax, scale)) {  // the same in the four threads of the block; rare
        const bool no_grid = scale == 0.0f;  // every activation counts as below the top binade
        float r8[8];
        refetch(r8);
        uint32_t rmax = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t xb = __builtin_bit_cast(uint32_t, r8[j]) & 0x7FFFFFFFu;
            r8[j] = (no_grid || xprep::below_top_binade(xb, amax)) ? xprep::residual(r8[j], mult, scale) : 0.0f;
            rmax = max(rmax, __builtin_bit_cast(uint32_t, r8[j]) & 0x7FFFFFFFu);
        }
        rmax = quad_max<0xB1>(rmax);
        rmax = quad_max<0x4E>(rmax);
        float mult2;
        xprep::block_scales<xprep::CORR_L>(rmax, &mult2, &scale2);
        uint32_t planes2[xprep::CORR_L];
        xprep::make_planes<xprep::CORR_L>(r8, mult2, planes2);
#pragma unroll
        for (int l = 0; l < xprep::CORR_L; l++) corr_dst[l * 8 + g] = planes2[l];
    }
    if ((g & 3) == 0) {
        slot_dst[8 * L + (g >> 2)] = __builtin_bit_cast(uint32_t, scale);
        slot_dst[8 * L + 2 + (g >> 2)] = __builtin_bit_cast(uint32_t, scale2);
    }
}

// The eight activations of task (slot, g) of a vector in global memory, in the order prep_store takes them.
__device__ __forceinline__ void fetch_task(const float *xs /* the slot's 64 activations */, int g, float2 (&v)[4]) {
#pragma unroll
    for (int t = 0; t < 4; t += 2) {
        // nibble pairs t, t+1 of group g: weights (b, b+1) low nibbles and (16+b, 17+b) high nibbles
        const int b = xprep::group_x_index(g, 2 * t);  // even by construction
        v[t] = *reinterpret_cast<const float2 *>(xs + b);
        v[t + 1] = *reinterpret_cast<const float2 *>(xs + b + 16);
    }
}

// nibble order of the weight dword: byte b low, byte b high, byte b+1 low, byte b+1 high, ...
#define GH_TASK_X8(v) {(v)[0].x, (v)[1].x, (v)[0].y, (v)[1].y, (v)[2].x, (v)[3].x, (v)[2].y, (v)[3].y}

// Activation preparation, split in two so that the activation loads can be issued before
// the first weight loads (loads return in order, so whatever must be consumed first has to
// be requested first) and the arithmetic runs while the weights are in flight.
// One thread per (slot, weight-dword group); a quad of threads covers one block.
template <int L, int THREADS, int PG>  // PG: groups per thread, an upper bound fixed at dispatch
struct xprep_state {
    float2 v[PG][4];

    __device__ __forceinline__ void load(const float *__restrict__ xg, int c0, int cs) {
#pragma unroll
        for (int p = 0; p < PG; p++) {
            const int idx = threadIdx.x + p * THREADS;
            if (idx < cs * 8) fetch_task(xg + (size_t)(c0 + (idx >> 3)) * 64, idx & 7, v[p]);
        }
    }

    __device__ __forceinline__ void compute(uint32_t *lds, const float *__restrict__ xg, int c0, int cs) const {
        uint32_t *corr = lds + cs * slot_lds<L>::dwords;
#pragma unroll
        for (int p = 0; p < PG; p++) {
            const int idx = threadIdx.x + p * THREADS;
            if (idx < cs * 8) {
                const int slot = idx >> 3, g = idx & 7;
                const float x8[8] = GH_TASK_X8(v[p]);
                prep_store<L>(x8, lds + slot * slot_lds<L>::dwords, corr + slot * slot_lds<L>::corr_dwords, g,
                              [&](float (&y8)[8]) {
                                  float2 w[4];
                                  fetch_task(xg + (size_t)(c0 + slot) * 64, g, w);
                                  const float t8[8] = GH_TASK_X8(w);
#pragma unroll
                                  for (int j = 0; j < 8; j++) y8[j] = t8[j];
                              });
            }
        }
    }
};

__device__ __forceinline__ int sdot8_first(uint32_t a, uint32_t b) {
    int d;
    asm("v_dot8_i32_i4 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}

// Integer dot of one block's four nibble dwords with the block's four dwords of each of its L planes:
// sum_l 16^l * dot8.  One accumulator per plane, issued round-robin: back-to-back v_dot8 into the same
// register serialise on the dot pipeline's latency, independent ones issue every cycle.
template <int L>
__device__ __forceinline__ int block_dot(const uint32_t (&nd)[4], const uint32_t (&xh)[L][4]) {
    int t[L];
#pragma unroll
    for (int l = 0; l < L; l++) t[l] = sdot8_first(nd[0], xh[l][0]);
#pragma unroll
    for (int i = 1; i < 4; i++)
#pragma unroll
        for (int l = 0; l < L; l++) t[l] = __builtin_amdgcn_sdot8((int)nd[i], (int)xh[l][i], t[l], false);
    int r = t[L - 1];
#pragma unroll
    for (int l = L - 2; l >= 0; l--) r = (r << 4) + t[l];
    return r;
}

// One slot of R rows: acc[r] += the dot product of row r's 64 weights (q[r]) with the slot's activations, read from
// the slot's LDS image (slot_lds) one block at a time, so that only half a slot's planes are held at once; a block
// with a correction (few, if any) also takes the same weights against its correction planes.
template <int L, int R>
__device__ __forceinline__ void slot_rows(const q4_slot (&q)[R], const uint32_t *slot_src, const uint32_t *corr_src,
                                          float *acc /* [R] */) {
    constexpr int CL = xprep::CORR_L;
    const uint32_t sign = 0x88888888u;
    const uint4 sc = *reinterpret_cast<const uint4 *>(slot_src + 8 * L);  // scales of A, B; of their corrections (0 = none)
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
        uint32_t xh[L][4];
#pragma unroll
        for (int l = 0; l < L; l++) {
            const uint4 v = *reinterpret_cast<const uint4 *>(slot_src + l * 8 + 4 * blk);
            xh[l][0] = v.x, xh[l][1] = v.y, xh[l][2] = v.z, xh[l][3] = v.w;
        }
        const float s = __builtin_bit_cast(float, blk ? sc.y : sc.x);
        const uint32_t cbits = blk ? sc.w : sc.z;
        uint32_t nd[R][4];
        float d[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (blk == 0) {
                // block A's qs start 2 bytes into the slot: each of its dwords is the top half of one word and the
                // low half of the next
                d[r] = f16_bits_to_f32(q[r].w[0] & 0xFFFFu);
#pragma unroll
                for (int i = 0; i < 4; i++) nd[r][i] = __builtin_amdgcn_alignbit(q[r].w[i + 1], q[r].w[i], 16) ^ sign;
            } else {
                d[r] = f16_bits_to_f32(q[r].w[4] >> 16);
#pragma unroll
                for (int i = 0; i < 4; i++) nd[r][i] = q[r].w[5 + i] ^ sign;
            }
            acc[r] = __builtin_fmaf(d[r] * s, (float)block_dot<L>(nd[r], xh), acc[r]);
        }
        if (cbits != 0) {
            uint32_t xc[CL][4];
#pragma unroll
            for (int l = 0; l < CL; l++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(corr_src + l * 8 + 4 * blk);
                xc[l][0] = v.x, xc[l][1] = v.y, xc[l][2] = v.z, xc[l][3] = v.w;
            }
            const float s2 = __builtin_bit_cast(float, cbits);
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] = __builtin_fmaf(d[r] * s2, (float)block_dot<CL>(nd[r], xc), acc[r]);
        }
    }
}

// Fast path: K % 64 == 0, W 4-byte aligned, x 8-byte aligned.
// Each wave owns R*G consecutive rows; a workgroup owns WAVES*R*G rows.  No explicit
// register double-buffering: several workgroups share a CU and overlap each other's
// loads, activation preparation and arithmetic.
// PG bounds the activation groups one thread prepares per pass; OCC is the number of waves
// per SIMD the register allocation must leave room for.
// MULTIPASS: K exceeds one LDS pass (kChunkSlots slots); the single-pass instantiation has
// no outer loop, which keeps the compiler from ordering loads across a back edge.
template <int L, int R, int G, int WAVES, int PG, int OCC, bool MULTIPASS>
__global__ __launch_bounds__(WAVES * 64, OCC) void gemv_q4_0_dot8(const uint8_t *__restrict__ W,
                                                             const float *__restrict__ xg, float *__restrict__ y,
                                                             int nslots, int N) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr int SD = slot_lds<L>::dwords;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * WAVES + wave) * (R * G);
    const size_t row_bytes = (size_t)nslots * sizeof(q4_slot);

    float acc[G][R];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[g][r] = 0.0f;

    for (int c0 = 0; c0 < (MULTIPASS ? nslots : 1); c0 += kChunkSlots) {
        const int cs = MULTIPASS ? min(kChunkSlots, nslots - c0) : nslots;
        if (MULTIPASS && c0 > 0) __syncthreads();
        xprep_state<L, WAVES * 64, PG> xp;
        xp.load(xg, c0, cs);
        // first weights of this pass go in flight behind the activations
        q4_slot q0[R];
        {
            const int s = min(c0 + lane, nslots - 1);
#pragma unroll
            for (int r = 0; r < R; r++)
                load_slot(q0[r], W + (size_t)min(row0 + r, N - 1) * row_bytes + (size_t)s * sizeof(q4_slot));
        }
        // nothing that waits for the activations may be scheduled ahead of the weight requests
        __builtin_amdgcn_sched_barrier(0);
        xp.compute(lds, xg, c0, cs);
        __syncthreads();

        const uint32_t *corr = lds + cs * SD;
        for (int sl = lane; sl - lane < cs; sl += 64) {  // uniform trip count; lanes past the end idle
            const bool act = sl < cs;
            const int s_ld = min(sl, cs - 1);
#pragma unroll
            for (int g = 0; g < G; g++) {
                q4_slot q[R];
                if (g == 0 && sl == lane) {
#pragma unroll
                    for (int r = 0; r < R; r++) q[r] = q0[r];
                } else {
#pragma unroll
                    for (int r = 0; r < R; r++)  // rows past N are loaded from row N-1 and never stored
                        load_slot(q[r], W + (size_t)min(row0 + g * R + r, N - 1) * row_bytes +
                                            (size_t)(c0 + s_ld) * sizeof(q4_slot));
                }
                if (act) slot_rows<L, R>(q, lds + s_ld * SD, corr + s_ld * slot_lds<L>::corr_dwords, acc[g]);
            }
        }
    }

    // every total lands in lane 63; lane 63-j picks up row j so the wave stores its rows at once
    float out = 0.0f;
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float t = wave_sum_to_lane63(acc[g][r]);
            const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, t), 63));
            if (lane == g * R + r) out = b;
        }
    if (lane < R * G && row0 + lane < N) y[row0 + lane] = out;
}

// Generic path: any K % 32 == 0 and any 2-byte-aligned W / 4-byte-aligned x.
// One wave per row, one block per lane per step, 2-byte loads, plain f32 arithmetic.
__global__ __launch_bounds__(256) void gemv_q4_0_generic(const uint16_t *__restrict__ W, const float *__restrict__ x,
                                                        float *__restrict__ y, int nblocks, int N) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint16_t *wr = W + (size_t)row * nblocks * 9;
    float acc = 0.0f;
    for (int b = lane; b < nblocks; b += 64) {
        const uint16_t *p = wr + (size_t)b * 9;
        const float d = f16_bits_to_f32(p[0]);
        const float *xb = x + (size_t)b * 32;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t v = p[1 + j];  // bytes 2j, 2j+1
            s = __builtin_fmaf((float)((int)(v & 0xF) - 8), xb[2 * j], s);
            s = __builtin_fmaf((float)((int)((v >> 4) & 0xF) - 8), xb[2 * j + 16], s);
            s = __builtin_fmaf((float)((int)((v >> 8) & 0xF) - 8), xb[2 * j + 1], s);
            s = __builtin_fmaf((float)((int)((v >> 12) & 0xF) - 8), xb[2 * j + 17], s);
        }
        acc = __builtin_fmaf(d, s, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

// ---------------------------------------------------------------------------------------
// Group kernel: up to GG_MAX matrix-vector products in one launch.
//
// A launch costs about as much as streaming 15-20 MB of weights.  Here the grids of several
// products are laid end to end: a workgroup finds its matrix from its block index and then
// does what a workgroup of gemv_q4_0_dot8 does (single pass, K <= 12288); the hardware hands
// workgroups to CUs as they free up, which balances matrices of different shapes.
//
// Fused around the product, so that a decode step needs no separate launches for them:
//   - RMSNorm (+ weight) of the activation vector while it is prepared (rms_norm.cu:13-49
//     followed by mul.cu:3-12): every workgroup reads the whole vector anyway;
//   - a residual added to the result (add.cu:3-12);
//   - a second matrix on the same activations whose result is multiplied with silu of the
//     first's (unary.cu:1-10 then mul.cu:3-12): the SwiGLU gate / up pair.
constexpr int GG_MAX = 8;
constexpr int GG_MAX_SLOTS = kChunkSlots;  // K <= 12288: one LDS pass

// Kernel arguments, one array per field.  What a workgroup needs before it can request memory (matrix,
// activations, shape) is fetched for all GG_MAX products at once and picked with scalar selects, so a
// workgroup waits for one scalar load round trip, not for one per level of indexing.
struct gg_args {
    int32_t blk0[GG_MAX];         // first block of each matrix; unused entries hold INT_MAX
    const uint8_t *W[GG_MAX];
    const uint8_t *W2[GG_MAX];    // up matrix of a SwiGLU pair, or null
    const float *x[GG_MAX];
    int32_t N[GG_MAX];
    int32_t nslots[GG_MAX];
    const float *norm_w[GG_MAX];  // NORM 1: RMSNorm weight; NORM 2: the partial sums of squares of the activations
    float *dst[GG_MAX];
    const float *residual[GG_MAX];  // or null
    float eps[GG_MAX];
    float *dst2[GG_MAX];          // OUT2: second copy of the result, multiplied by scale2, or null
    const float *scale2[GG_MAX];
    float *ssq_out[GG_MAX];       // OUT2: sum of squares of the result, one float per workgroup (16 rows), or null
};

// A wave owns R slots per lane: R rows, or R / 2 rows of a gate / up pair; a workgroup WAVES times that.
// PG: activation groups (8 values) one thread prepares at most.
// NORM 1: the vector is normalised (rms_norm) and multiplied by a weight first.  NORM 2: the vector arrives already
// multiplied by the weight and the sums of squares of the unweighted vector arrive as per-16-row partials (written
// by the launch that produced the vector, OUT2): w . (inv * xg) = inv * (w . xg), so the product runs on the vector as
// it is and the result is multiplied by inv = rsqrt(mean + eps) at the end -- no second vector to fetch and no
// barrier before the preparation.
// OUT2: the launch also writes result * scale2 and the workgroup's sum of squares of the result.
// MAXI: products the selects look at (4 keeps all of their operands in scalar registers at once).
// COHERENT: the results go out as device-coherent stores, for readers in the same launch on other XCDs.
// item / item_block: which product the workgroup served and its index among that product's workgroups.
// CHUNKED: a vector longer than THREADS * PG / 8 slots is worked through in chunks of that many slots -- prepare a
// chunk, meet, multiply it, meet, prepare the next -- so that the kernel keeps the registers and the LDS of the
// short-vector build whatever the longest vector of the launch: measured on the four LLaMA-7B products in one
// launch, the one K = 11008 matrix made all 3200 workgroups run the build that holds three tasks per thread and
// 52 KB of planes (three workgroups per CU instead of four), 24.4 us against 23.1 us for the same bytes at K = 4096.
// Not for the normalising preparation, which needs the whole vector's sum of squares before it scales anything.
template <int L, int R, int WAVES, int PG, int NORM_MODE, int MAXI, bool OUT2, bool COHERENT, bool CHUNKED = false>
__device__ __forceinline__ void gemv_group_wg(const gg_args &a, uint32_t *lds, int &item, int &item_block) {
    static_assert(!(CHUNKED && NORM_MODE == 1), "the normalising preparation is not chunked");
    constexpr int CH = WAVES * 64 * PG / 8;  // slots per chunk
    __shared__ float red[WAVES];
    __shared__ float red2[WAVES];
    constexpr int SD = slot_lds<L>::dwords;
    constexpr int THREADS = WAVES * 64;
    constexpr bool NORM = NORM_MODE == 1;    // normalise here
    constexpr bool NORM2 = NORM_MODE == 2;   // scale the result by inv from the partial sums of squares
    constexpr bool NARG = NORM_MODE != 0;    // the norm_w / eps arguments are used
    const int lane = threadIdx.x & 63;
    // CHUNKED: the wave index as a scalar, so that row addresses are scalar too and do not hold vector registers
    // through every phase of every chunk
    const int wave = CHUNKED ? __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) : (int)(threadIdx.x >> 6);

    // Every product's fields are fetched before any is chosen (the empty asm makes each an opaque value; left
    // alone, the compiler turns a select of two arguments into a second, dependent load from a selected address).
    int32_t k_blk0[MAXI], k_N[MAXI], k_ns[MAXI];
    uint64_t k_W[MAXI], k_W2[MAXI], k_x[MAXI], k_nw[NARG ? MAXI : 1];  // pointers as bits: an address that has been
                                                // through an asm is no longer known to be global memory and is cast back below
    float k_eps[NARG ? MAXI : 1];
#pragma unroll
    for (int k = 0; k < MAXI; k++) {
        k_blk0[k] = a.blk0[k], k_N[k] = a.N[k], k_ns[k] = a.nslots[k];
        k_W[k] = (uint64_t)a.W[k], k_W2[k] = (uint64_t)a.W2[k], k_x[k] = (uint64_t)a.x[k];
        if (NARG) k_nw[k] = (uint64_t)a.norm_w[k], k_eps[k] = a.eps[k];
    }
#pragma unroll
    for (int k = 0; k < MAXI; k++) {
        asm volatile("" : "+s"(k_blk0[k]));
        asm volatile("" : "+s"(k_N[k]));
        asm volatile("" : "+s"(k_ns[k]));
        asm volatile("" : "+s"(k_W[k]));
        asm volatile("" : "+s"(k_W2[k]));
        asm volatile("" : "+s"(k_x[k]));
        if (NARG) {
            asm volatile("" : "+s"(k_nw[k]));
            asm volatile("" : "+s"(k_eps[k]));
        }
    }
    int ii = 0, first_blk = 0;
    uint64_t W_bits = k_W[0], W2_bits = k_W2[0], x_bits = k_x[0], nw_bits = NARG ? k_nw[0] : 0;
    float eps = NARG ? k_eps[0] : 0.0f;
    int N = k_N[0], ns = k_ns[0];
#pragma unroll
    for (int k = 1; k < MAXI; k++) {
        const bool ge = (int)blockIdx.x >= k_blk0[k];
        ii = ge ? k : ii, first_blk = ge ? k_blk0[k] : first_blk;
        W_bits = ge ? k_W[k] : W_bits, W2_bits = ge ? k_W2[k] : W2_bits, x_bits = ge ? k_x[k] : x_bits;
        N = ge ? k_N[k] : N, ns = ge ? k_ns[k] : ns;
        if (NARG) nw_bits = ge ? k_nw[k] : nw_bits, eps = ge ? k_eps[k] : eps;
    }
    typedef const __attribute__((address_space(1))) uint8_t *global_bytes;
    typedef const __attribute__((address_space(1))) float *global_floats;
    const uint8_t *const W = (const uint8_t *)(global_bytes)W_bits, *const W2 = (const uint8_t *)(global_bytes)W2_bits;
    const float *const xg_all = (const float *)(global_floats)x_bits;
    item = ii, item_block = (int)blockIdx.x - first_blk;
    const bool dual = W2 != nullptr;
    const int rw = dual ? R / 2 : R;  // rows per wave and group
    // the workgroup's waves cover WAVES * rw consecutive rows: neighbouring waves read neighbouring rows
    const int row0 = ((int)blockIdx.x - first_blk) * (WAVES * rw) + wave * rw;
    const size_t row_bytes = (size_t)ns * sizeof(q4_slot);  // of the whole row

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;

    // ---- activation preparation: task = (slot, weight-dword group).  Loads retire in order, so the activations
    // are requested first and the first weights right behind them: the preparation then runs while the weights
    // are in flight.
    q4_slot q0[R];
    uint64_t dst_bits = 0, res_bits = 0, dst2_bits = 0, scale2_bits = 0, ssq_bits = 0;
    float scale2_first = 0.0f;  // OUT2: scale_weight of this lane's row
    float inv2 = 1.0f;
    const int ns_all = ns;  // the row's slots; below, ns is the chunk's
    const int nchunks = CHUNKED ? (ns_all + CH - 1) / CH : 1;
    constexpr int MAX_CHUNKS = CHUNKED ? (GG_MAX_SLOTS + CH - 1) / CH : 1;
    // unrolled: as a loop the compiler hoists the chunk-independent address arithmetic into registers that then live
    // through every phase (76 registers instead of 59)
#pragma unroll
    for (int chunk = 0; chunk < MAX_CHUNKS; chunk++) {
    if (CHUNKED && chunk >= nchunks) break;
    if (CHUNKED && chunk > 0) __builtin_amdgcn_sched_barrier(0);  // the next chunk's requests stay behind this point: their
                                                                  // registers are not free before the multiplication is done
    const int c0 = CHUNKED ? chunk * CH : 0;                     // first slot of the chunk
    const int ns = CHUNKED ? min(CH, ns_all - c0) : ns_all;      // slots in it
    const float *const xg = xg_all + (size_t)c0 * 64;
    const bool first = !CHUNKED || chunk == 0;
    // CHUNKED: the thread index passes through an empty asm in every chunk, so that what is derived from it (addresses in
    // the vector, in LDS, in the row) is computed where it is used instead of living in registers from chunk to chunk
    int tid_c = (int)threadIdx.x;
    if (CHUNKED) asm volatile("" : "+v"(tid_c));
    const int lane = tid_c & 63;
    {
        const float *wg = NORM ? (const float *)(global_floats)nw_bits : nullptr;
        float2 v[PG][4], nw[NORM ? PG : 1][4];
        // Normalising preparation of a short vector (K <= 4096): the vector and the norm weight are fetched with
        // fully coalesced 16-byte loads (a thread's eight values in weight-nibble order lie in four places, and
        // fetching both arrays that way costs as much as a quarter of the weight stream), their product is staged
        // in LDS behind the planes, and each thread gathers its eight values from there after the barrier the sum
        // of squares needs anyway.
        constexpr bool STAGED = NORM && PG == 1;
        float4 sx[2], sg[2];
        if (STAGED) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int i4 = min(tid_c + j * THREADS, ns * 16 - 1);
                sx[j] = reinterpret_cast<const float4 *>(xg)[i4];
                sg[j] = reinterpret_cast<const float4 *>(wg)[i4];
            }
        }
#pragma unroll
        for (int p = 0; p < PG; p++) {
            const int idx = tid_c + p * THREADS;
            if (!STAGED && idx < ns * 8) {
                fetch_task(xg + (idx >> 3) * 64, idx & 7, v[p]);
                if (NORM) fetch_task(wg + (idx >> 3) * 64, idx & 7, nw[NORM ? p : 0]);
            }
        }
        float psq = 0.0f;
        if (NORM2 && first) {  // one partial per 16 elements of the whole vector: ns_all * 4 of them
            const float *sq = (const float *)(global_floats)nw_bits;
            constexpr int PQ = (GG_MAX_SLOTS * 4 + THREADS - 1) / THREADS;
            float t[PQ];
#pragma unroll
            for (int p = 0; p < PQ; p++) t[p] = sq[min(tid_c + p * THREADS, ns_all * 4 - 1)];
#pragma unroll
            for (int p = 0; p < PQ; p++) psq += tid_c + p * THREADS < ns_all * 4 ? t[p] : 0.0f;
        }
        // q[j] = slot `lane` of row row0 + j of W; for a gate / up pair q[j] = row row0 + j of W (j < R/2) or of W2.
        // Rows past N are loaded from row N - 1 and never stored.
        {
            const int s = min(lane, ns - 1);
#pragma unroll
            for (int j = 0; j < R; j++) {
                const uint8_t *base = (dual && j >= R / 2) ? W2 : W;
                const int row = min(row0 + ((dual && j >= R / 2) ? j - R / 2 : j), N - 1);
                load_slot(q0[j], base + (size_t)row * row_bytes + (size_t)(c0 + s) * sizeof(q4_slot));
            }
        }
        // nothing that waits for the activations may be scheduled ahead of the weight requests
        __builtin_amdgcn_sched_barrier(0);
        // Where the results go, fetched now (indexed argument loads) so that nothing waits for them at the end.
        if (first) {
            dst_bits = (uint64_t)a.dst[ii], res_bits = (uint64_t)a.residual[ii];
            asm volatile("" : "+s"(dst_bits));
            asm volatile("" : "+s"(res_bits));
            if (OUT2) {
                dst2_bits = (uint64_t)a.dst2[ii], scale2_bits = (uint64_t)a.scale2[ii], ssq_bits = (uint64_t)a.ssq_out[ii];
                asm volatile("" : "+s"(dst2_bits));
                asm volatile("" : "+s"(scale2_bits));
                asm volatile("" : "+s"(ssq_bits));
            }
        }
        if (NORM2 && first) {  // the partial sums reach every wave through the barrier that publishes the planes
            psq = wave_sum(psq);
            if (lane == 0) red[wave] = psq;
        }
        float inv_norm = 1.0f;
        if (NORM) {
            float ss = 0.0f;
            float *stage = reinterpret_cast<float *>(lds + ns * SD);
            if (STAGED) {
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int i4 = tid_c + j * THREADS;
                    if (i4 < ns * 16) {
                        ss += sx[j].x * sx[j].x + sx[j].y * sx[j].y + sx[j].z * sx[j].z + sx[j].w * sx[j].w;
                        reinterpret_cast<float4 *>(stage)[i4] =
                            make_float4(sx[j].x * sg[j].x, sx[j].y * sg[j].y, sx[j].z * sg[j].z, sx[j].w * sg[j].w);
                    }
                }
            } else {
#pragma unroll
                for (int p = 0; p < PG; p++)
                    if (tid_c + p * THREADS < ns * 8) {
#pragma unroll
                        for (int t = 0; t < 4; t++) ss += v[p][t].x * v[p][t].x + v[p][t].y * v[p][t].y;
                    }
            }
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
            __syncthreads();
            float tot = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; w++) tot += red[w];
            const float inv = rsqrtf(tot / (float)(ns * 64) + eps);
            if (STAGED) {
                if (tid_c < ns * 8) {
                    fetch_task(stage + (tid_c >> 3) * 64, tid_c & 7, v[0]);
#pragma unroll
                    for (int t = 0; t < 4; t++) v[0][t] = make_float2(v[0][t].x * inv, v[0][t].y * inv);
                }
            } else {
#pragma unroll
                for (int p = 0; p < PG; p++)
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        v[p][t].x = (inv * v[p][t].x) * nw[NORM ? p : 0][t].x;
                        v[p][t].y = (inv * v[p][t].y) * nw[NORM ? p : 0][t].y;
                    }
            }
            inv_norm = inv;
        }
        // the corrections live behind the slots (and behind the staged activations, which other threads may still read)
        uint32_t *const corr = lds + ns * SD + (STAGED ? ns * 64 : 0);
#pragma unroll
        for (int p = 0; p < PG; p++) {
            const int idx = tid_c + p * THREADS;
            if (idx < ns * 8) {
                const int slot = idx >> 3, g = idx & 7;
                const float x8[8] = GH_TASK_X8(v[p]);
                prep_store<L>(x8, lds + slot * SD, corr + slot * slot_lds<L>::corr_dwords, g, [&](float (&y8)[8]) {
                    // the same values by the same arithmetic as above
                    float2 w[4];
                    if (STAGED) {
                        fetch_task(reinterpret_cast<const float *>(lds + ns * SD) + slot * 64, g, w);
#pragma unroll
                        for (int t = 0; t < 4; t++) w[t] = make_float2(w[t].x * inv_norm, w[t].y * inv_norm);
                    } else {
                        fetch_task(xg + slot * 64, g, w);
                        if (NORM) {
                            float2 gw[4];
                            fetch_task(wg + slot * 64, g, gw);
#pragma unroll
                            for (int t = 0; t < 4; t++)
                                w[t] = make_float2((inv_norm * w[t].x) * gw[t].x, (inv_norm * w[t].y) * gw[t].y);
                        }
                    }
                    const float t8[8] = GH_TASK_X8(w);
#pragma unroll
                    for (int j = 0; j < 8; j++) y8[j] = t8[j];
                });
            }
        }
    }
    __syncthreads();
    if (OUT2 && first) {  // the scale values ride behind the weights, requested once the preparation's registers are free
        const float *sp = scale2_bits ? (const float *)(global_floats)scale2_bits + min(row0 + (lane < rw ? lane : 0), N - 1) : xg;
        scale2_first = *sp;
    }
    if (NORM2 && first) {
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) tot += red[w];
        // the same value in every lane: kept in a scalar register (the kernel has no vector register to spare)
        inv2 = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, rsqrtf(tot / (float)(ns_all * 64) + eps))));
    }

    // The rows of this wave.  The first slots are the ones requested before the preparation.
    {
        const uint32_t *corr = lds + ns * SD + ((NORM && PG == 1) ? ns * 64 : 0);
        if (CHUNKED) {  // a chunk is at most one slot per lane: the one requested before its preparation
            if (lane < ns) slot_rows<L, R>(q0, lds + lane * SD, corr + lane * slot_lds<L>::corr_dwords, acc);
        } else
        for (int sl = lane; sl - lane < ns; sl += 64) {  // uniform trip count; lanes past the end idle
            const bool act = sl < ns;
            const int s_ld = min(sl, ns - 1);
            q4_slot q[R];
            if (sl == lane) {
#pragma unroll
                for (int j = 0; j < R; j++) q[j] = q0[j];
            } else {
#pragma unroll
                for (int j = 0; j < R; j++) {
                    const uint8_t *base = (dual && j >= R / 2) ? W2 : W;
                    const int row = min(row0 + ((dual && j >= R / 2) ? j - R / 2 : j), N - 1);
                    load_slot(q[j], base + (size_t)row * row_bytes + (size_t)(c0 + s_ld) * sizeof(q4_slot));
                }
            }
            if (act) slot_rows<L, R>(q, lds + s_ld * SD, corr + s_ld * slot_lds<L>::corr_dwords, acc);
        }
    }
    if (CHUNKED && chunk + 1 < nchunks) __syncthreads();  // every wave is done with this chunk's planes
    }  // chunks

    float sq_out = 0.0f;  // OUT2: squares of this lane's results
    {
        // every total lands in lane 63; lane j picks up row j so the wave stores its rows at once
        float out = 0.0f;
        if (dual) {
#pragma unroll
            for (int j = 0; j < R / 2; j++) {
                float gt = wave_sum_to_lane63(acc[j]), up = wave_sum_to_lane63(acc[R / 2 + j]);
                gt = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gt), 63));
                up = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, up), 63));
                if (NORM2) gt *= inv2, up *= inv2;
                if (lane == j) out = gt / (1.0f + expf(-gt)) * up;
            }
        } else {
#pragma unroll
            for (int j = 0; j < R; j++) {
                float t = wave_sum_to_lane63(acc[j]);
                t = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, t), 63));
                if (NORM2) t *= inv2;
                if (lane == j) out = t;
            }
        }
        if (lane < rw && row0 + lane < N) {
            typedef __attribute__((address_space(1))) float *global_out;
            const float *res = (const float *)(global_floats)res_bits;
            if (res) out += res[row0 + lane];
            if (COHERENT)
                __hip_atomic_store((float *)(global_out)dst_bits + row0 + lane, out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else
                ((float *)(global_out)dst_bits)[row0 + lane] = out;
            if (OUT2) {
                if (dst2_bits)
                    ((float *)(global_out)dst2_bits)[row0 + lane] = out * scale2_first;
                sq_out = __builtin_fmaf(out, out, sq_out);
            }
        }
    }
    if (OUT2 && ssq_bits) {  // wave-uniform; every wave of the workgroup gets here
        sq_out = wave_sum(sq_out);
        if (lane == 0) red2[wave] = sq_out;
        __syncthreads();
        if (threadIdx.x == 0) {
            float tot = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; w++) tot += red2[w];
            typedef __attribute__((address_space(1))) float *global_out;
            ((float *)(global_out)ssq_bits)[(int)blockIdx.x - first_blk] = tot;
        }
    }
}

template <int L, int R, int WAVES, int PG, int OCC, int NORM_MODE, int MAXI, bool OUT2, bool CHUNKED = false>
__global__ __launch_bounds__(WAVES * 64, OCC) void gemv_q4_0_group(const gg_args a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    int item, item_block;
    gemv_group_wg<L, R, WAVES, PG, NORM_MODE, MAXI, OUT2, false, CHUNKED>(a, lds, item, item_block);
}

template <int L, int R, int G, int WAVES, int OCC>
void launch_dot8(galois_hip_ctx *ctx, const void *vx, const float *x, float *dst, int nslots, int N) {
    const int rows_per_wg = WAVES * R * G;
    const dim3 grid((N + rows_per_wg - 1) / rows_per_wg), block(WAVES * 64);
    const int pass_slots = min(nslots, kChunkSlots);
    const size_t lds = (size_t)pass_slots * slot_lds<L>::bytes_per_slot;
    constexpr int PGMAX = (kChunkSlots * 8 + WAVES * 64 - 1) / (WAVES * 64);
    constexpr int PGSMALL = (64 * 8 + WAVES * 64 - 1) / (WAVES * 64);  // K <= 4096
    const uint8_t *W = (const uint8_t *)vx;
    if (nslots <= 64)
        hipLaunchKernelGGL((gemv_q4_0_dot8<L, R, G, WAVES, PGSMALL, OCC, false>), grid, block, lds, ctx->stream, W,
                           x, dst, nslots, N);
    else if (nslots <= kChunkSlots)
        hipLaunchKernelGGL((gemv_q4_0_dot8<L, R, G, WAVES, PGMAX, OCC, false>), grid, block, lds, ctx->stream, W, x,
                           dst, nslots, N);
    else
        hipLaunchKernelGGL((gemv_q4_0_dot8<L, R, G, WAVES, PGMAX, (OCC > 3 ? 3 : OCC), true>), grid, block, lds,
                           ctx->stream, W, x, dst, nslots, N);  // the loop over passes keeps more alive
}

// Host side of the group kernel: checks, the block range of every matrix, launch.
// mode: 0 plain, 1 normalising, 2 pre-weighted activations + partial sums of squares; out2: second outputs.
// The second outputs exist for plain launches of at most four products (what produces a residual stream).
template <int L, int R, int WAVES, int OCC, int MAXI>
void launch_group_cfg(galois_hip_ctx *ctx, const gg_args &a, unsigned blocks, int max_slots, int mode, bool out2) {
    const dim3 grid(blocks), block(WAVES * 64);
    const size_t lds = (size_t)max_slots * slot_lds<L>::bytes_per_slot;
    constexpr int PGMAX = (kChunkSlots * 8 + WAVES * 64 - 1) / (WAVES * 64);
    constexpr int PGSMALL = (64 * 8 + WAVES * 64 - 1) / (WAVES * 64);  // K <= 4096
    constexpr int OCCN = OCC > 4 ? 4 : OCC;  // the normalising preparation of a long vector needs more registers
#define GG_LAUNCH(PG_, OCC_, MODE_, OUT2_, LDS_) \
    hipLaunchKernelGGL((gemv_q4_0_group<L, R, WAVES, PG_, OCC_, MODE_, MAXI, OUT2_>), grid, block, LDS_, ctx->stream, a)
    if (max_slots <= 64) {
        if (mode == 1 && PGSMALL == 1)  // room behind the planes for the staged, weighted activations (64 floats per slot)
            GG_LAUNCH(PGSMALL, OCC, 1, false, lds + (size_t)max_slots * 64 * sizeof(float));
        else if (mode == 1)
            GG_LAUNCH(PGSMALL, OCC, 1, false, lds);
        else if (mode == 2)
            GG_LAUNCH(PGSMALL, OCC, 2, false, lds);
        else if (out2 && MAXI == 4)
            GG_LAUNCH(PGSMALL, OCC, 0, (MAXI == 4), lds);
        else
            GG_LAUNCH(PGSMALL, OCC, 0, false, lds);
    } else if (WAVES == 8 && mode != 1) {
        // many rows and a long vector somewhere in the launch: chunks of 64 slots, so that every workgroup keeps the
        // registers and the LDS of the short-vector build
        const size_t lds_chunk = (size_t)64 * slot_lds<L>::bytes_per_slot;
#define GG_LAUNCH_CHUNKED(MODE_, OUT2_)                                                                                \
    hipLaunchKernelGGL((gemv_q4_0_group<L, R, WAVES, PGSMALL, OCC, MODE_, MAXI, OUT2_, true>), grid, block, lds_chunk, \
                       ctx->stream, a)
        if (mode == 2)
            GG_LAUNCH_CHUNKED(2, false);
        else if (out2 && MAXI == 4)
            GG_LAUNCH_CHUNKED(0, (MAXI == 4));
        else
            GG_LAUNCH_CHUNKED(0, false);
#undef GG_LAUNCH_CHUNKED
    } else {
        if (mode == 1)
            GG_LAUNCH(PGMAX, OCCN, 1, false, lds);
        else if (mode == 2)
            GG_LAUNCH(PGMAX, OCC, 2, false, lds);
        else if (out2 && MAXI == 4)
            GG_LAUNCH(PGMAX, OCC, 0, (MAXI == 4), lds);
        else
            GG_LAUNCH(PGMAX, OCC, 0, false, lds);
    }
#undef GG_LAUNCH
}

template <int L, int R, int WAVES, int OCC>
void launch_group_cfg(galois_hip_ctx *ctx, const gg_args &a, int n_items, unsigned blocks, int max_slots, int mode, bool out2) {
    if (n_items <= 4)
        launch_group_cfg<L, R, WAVES, OCC, 4>(ctx, a, blocks, max_slots, mode, out2);
    else
        launch_group_cfg<L, R, WAVES, OCC, GG_MAX>(ctx, a, blocks, max_slots, mode, out2);
}

// What a group launch needs besides the kernel arguments.
struct gg_plan {
    int32_t max_slots = 0;
    int mode = 0;       // 0 plain, 1 normalising, 2 pre-weighted activations + partial sums of squares
    bool out2 = false;
    bool small = false;  // few rows per CU: 16 waves x 1 slot
    int64_t blocks = 0;
};

// Checks the items and fills the kernel arguments and the plan.  wg_slots: 0 = the shape is chosen here (16 slots
// per workgroup either way); otherwise the caller's kernel has workgroups of that many slots (a launch that also
// carries other work).
int32_t prepare_group(galois_hip_ctx *ctx, const galois_hip_gemv_item *items, int32_t n_items, const char *what, gg_args &a,
                      gg_plan &plan, int wg_slots) {
    GH_REQUIRE(ctx, items != nullptr, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, n_items >= 1 && n_items <= GG_MAX, GALOIS_HIP_E_SHAPE, "gemv group: 1 to 8 products per call");
    memset(&a, 0, sizeof(a));
    int32_t max_slots = 0;
    int64_t rows = 0;
    int mode = 0;
    bool out2 = false;
    for (int i = 0; i < GG_MAX; i++) a.blk0[i] = 0x7FFFFFFF;
    for (int i = 0; i < n_items; i++) {
        const galois_hip_gemv_item &s = items[i];
        GH_REQUIRE(ctx, s.vx && s.y && s.dst, GALOIS_HIP_E_NULL, what);
        GH_REQUIRE(ctx, s.ncols > 0 && s.nrows > 0 && s.ncols % 64 == 0 && s.ncols / 64 <= GG_MAX_SLOTS, GALOIS_HIP_E_SHAPE,
                   "gemv group: ncols must be a positive multiple of 64, at most 12288; nrows positive");
        GH_REQUIRE(ctx, gh_aligned(s.vx, 4) && gh_aligned(s.vx_up, 4) && gh_aligned(s.y, 8) && gh_aligned(s.norm_weight, 8) &&
                            gh_aligned(s.residual, 4) && gh_aligned(s.dst, 4),
                   GALOIS_HIP_E_ALIGN, "gemv group: matrices 4-byte, activations and norm weights 8-byte, vectors 4-byte aligned");
        GH_REQUIRE(ctx, !(s.norm_weight && s.sumsq_in), GALOIS_HIP_E_UNSUPPORTED,
                   "gemv group: norm_weight (normalise here) and sumsq_in (activations already weighted) exclude each other");
        const int m = s.norm_weight ? 1 : (s.sumsq_in ? 2 : 0);
        if (i == 0) mode = m;
        GH_REQUIRE(ctx, m == mode, GALOIS_HIP_E_UNSUPPORTED,
                   "gemv group: the products of a call all normalise their activations the same way or not at all");
        GH_REQUIRE(ctx, (s.dst_scaled == nullptr) == (s.scale_weight == nullptr), GALOIS_HIP_E_NULL,
                   "gemv group: dst_scaled and scale_weight go together");
        if (s.dst_scaled || s.sumsq_out) {
            GH_REQUIRE(ctx, m == 0 && !s.vx_up && n_items <= 4, GALOIS_HIP_E_UNSUPPORTED,
                       "gemv group: dst_scaled / sumsq_out are written by plain products (no norm, no pair) in calls of at most four");
            GH_REQUIRE(ctx, gh_aligned(s.dst_scaled, 4) && gh_aligned(s.scale_weight, 4) && gh_aligned(s.sumsq_out, 4),
                       GALOIS_HIP_E_ALIGN, "gemv group: 4-byte aligned vectors");
            out2 = true;
        }
        GH_REQUIRE(ctx, gh_aligned(s.sumsq_in, 4), GALOIS_HIP_E_ALIGN, "gemv group: 4-byte aligned vectors");
        a.W[i] = (const uint8_t *)s.vx, a.W2[i] = (const uint8_t *)s.vx_up, a.dst[i] = s.dst, a.residual[i] = s.residual;
        a.x[i] = s.y, a.norm_w[i] = m == 2 ? s.sumsq_in : s.norm_weight, a.eps[i] = s.norm_eps, a.N[i] = s.nrows;
        a.nslots[i] = s.ncols / 64;
        a.dst2[i] = s.dst_scaled, a.scale2[i] = s.scale_weight, a.ssq_out[i] = s.sumsq_out;
        if (a.nslots[i] > max_slots) max_slots = a.nslots[i];
        rows += (int64_t)s.nrows * (s.vx_up ? 2 : 1);
    }
    // Workgroup shape by rows per CU, as for the one-product kernel: few rows -> 16 waves x 1 slot so every SIMD has
    // work; more rows -> 8 waves x 2 slots, four workgroups resident per CU.  A gate / up pair needs 2 slots per lane.
    // One 16-slot row group per workgroup: measured, working through two or four groups per workgroup (which would
    // amortise the activation preparation) loses more to the coarser split of the launch than it saves at every
    // LLaMA-7B shape.
    bool any_dual = false;
    for (int i = 0; i < n_items; i++) any_dual |= items[i].vx_up != nullptr;
    const bool small = !wg_slots && !any_dual && (rows + ctx->n_cu - 1) / ctx->n_cu <= 16;
    const int slots_per_wg = wg_slots ? wg_slots : 16;  // WAVES * R of both shapes
    int64_t blocks = 0;
    for (int i = 0; i < n_items; i++) {
        const int64_t rows_per_wg = items[i].vx_up ? slots_per_wg / 2 : slots_per_wg;
        a.blk0[i] = (int32_t)blocks;
        blocks += (items[i].nrows + rows_per_wg - 1) / rows_per_wg;
        GH_REQUIRE(ctx, blocks < 0x7FFFFFFF, GALOIS_HIP_E_SHAPE, "gemv group: too many rows");
    }
    plan.max_slots = max_slots, plan.mode = mode, plan.out2 = out2, plan.small = small, plan.blocks = blocks;
    return GALOIS_HIP_OK;
}

int32_t launch_group(galois_hip_ctx *ctx, const galois_hip_gemv_item *items, int32_t n_items, const char *what) {
    gg_args a;
    gg_plan plan;
    const int32_t st = prepare_group(ctx, items, n_items, what, a, plan, 0);
    if (st != GALOIS_HIP_OK) return st;
    GH_BIND(ctx);
    if (plan.small)
        launch_group_cfg<5, 1, 16, 4>(ctx, a, n_items, (unsigned)plan.blocks, plan.max_slots, plan.mode, plan.out2);
    else
        launch_group_cfg<5, 2, 8, 6>(ctx, a, n_items, (unsigned)plan.blocks, plan.max_slots, plan.mode, plan.out2);
    GH_LAUNCH_CHECK(ctx, what);
}

// ---------------------------------------------------------------------------------------
// The q | k | v products and the decode attention in one launch.
//
// Issued as two launches the attention starts when the last product row is out, pays a launch gap, and then spends
// its first microseconds requesting the cache; its own end is a chain of dependent round trips (split records,
// counter, merge) during which the memory system idles.  Here the grid is the products' workgroups followed by the
// attention's: workgroups are handed out in index order, so the attention workgroups take the slots the products
// free, request their cache rows while the last products still stream, and wait (bounded) only for the 128 floats
// of their head's q -- the workgroups of the last split, which holds position n_past, also for k and v; whatever a
// workgroup waits for belongs to workgroups ahead of it in the grid, which are running or done.  A product workgroup
// stores its 16 rows with device-coherent stores, waits for them, and counts itself on the counter of the head they
// belong to.  (Measured: with the attention workgroups of the earlier splits placed right behind the q product, so
// that they are resident from the start, the launch takes twice as long -- the k and v products and then the last
// split queue up behind them, and the last split's whole latency lands at the end.)
template <typename CT>
struct fa_args {
    CT *kc, *vc;
    float *part, *out;
    unsigned *done, *ready;
    const int32_t *pos;
    int32_t H, L, S, gemv_blocks;
    uint32_t target;
    int32_t spin_limit;  // polls of a bounded wait
    unsigned *status;    // the context's status word (pinned host memory): set when a wait runs out
    float freq_scale, theta_scale, scale;
    int64_t key_stride, head_stride;  // of the caches, in elements
};
constexpr int FA_WAVES = 8, FA_HEAD_DIM = 128;
constexpr int FA_R = 2;  // rows per wave of the products (measured: 4, which makes all products resident at once, 30.7 against 25.3 us)
static_assert(FA_HEAD_DIM % (FA_WAVES * FA_R) == 0, "a product workgroup's rows belong to one head");
constexpr int FA_MAX_SLOTS = 184;  // activation vectors of up to 11776 elements: 55,936 bytes of planes beside the attention's 8.9 KB

template <int PG, int NORM_MODE, typename CT>
__global__ __launch_bounds__(FA_WAVES * 64, 4) void qkv_attn_decode_fused(const gg_args a, const fa_args<CT> b) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    if ((int)blockIdx.x < b.gemv_blocks) {
        int item, item_block;
        gemv_group_wg<5, FA_R, FA_WAVES, PG, NORM_MODE, 4, false, true>(a, lds, item, item_block);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows are out
        __syncthreads();
        if (threadIdx.x == 0) atomicAdd(b.ready + item * b.H + item_block / (FA_HEAD_DIM / (FA_WAVES * FA_R)), 1u);
    } else {
        // split-major order: the last split, whose workgroups wait for all three products, comes last
        const int t = (int)blockIdx.x - b.gemv_blocks;
        attn_decode_wg<FA_HEAD_DIM / 4, CT, FA_WAVES * 64, true>(a.dst[0], a.dst[1], a.dst[2], b.kc, b.vc, b.part, b.done, b.out,
                                                                 b.H, b.L, b.pos, b.freq_scale, b.theta_scale, b.scale,
                                                                 t % b.H, t / b.H, b.S, b.ready, b.target, b.key_stride,
                                                                 b.head_stride, b.spin_limit, b.status);
    }
}

template <typename CT>
int32_t launch_qkv_attn(galois_hip_ctx *ctx, const galois_hip_gemv_item *items, CT *k_cache, CT *v_cache, float *out,
                        int32_t n_head, int32_t head_dim, int32_t n_past, const int32_t *pos, float freq_scale,
                        float theta_scale, float scale, int32_t head_major_n_ctx, const char *what) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, items && k_cache && v_cache && out && pos, GALOIS_HIP_E_NULL, what);
    GH_REQUIRE(ctx, head_dim == FA_HEAD_DIM, GALOIS_HIP_E_UNSUPPORTED, "qkv_attn_decode: head_dim 128");
    GH_REQUIRE(ctx, head_major_n_ctx == 0 || head_major_n_ctx > n_past, GALOIS_HIP_E_SHAPE,
               "qkv_attn_decode: head_major_n_ctx is 0 or the capacity of a [n_head][n_ctx][head_dim] cache, above n_past");
    GH_REQUIRE(ctx, n_head > 0 && n_head <= GH_ATTN_HEADS && n_past >= 0 && n_past < 0x7FFFFF00, GALOIS_HIP_E_SHAPE,
               "qkv_attn_decode: n_head in 1..65536, n_past >= 0");
    GH_REQUIRE(ctx, gh_aligned(k_cache, 16) && gh_aligned(v_cache, 16) && gh_aligned(out, 16) && gh_aligned(pos, 4),
               GALOIS_HIP_E_ALIGN, "qkv_attn_decode: 16-byte aligned caches and output");
    for (int i = 0; i < 3; i++) {
        const galois_hip_gemv_item &s = items[i];
        GH_REQUIRE(ctx, s.nrows == n_head * head_dim && s.ncols == items[0].ncols, GALOIS_HIP_E_SHAPE,
                   "qkv_attn_decode: three products of n_head * head_dim rows on vectors of one length");
        GH_REQUIRE(ctx, !s.vx_up && !s.residual && !s.dst_scaled && !s.sumsq_out, GALOIS_HIP_E_UNSUPPORTED,
                   "qkv_attn_decode: plain or normalising products (no pair, residual or second output)");
        GH_REQUIRE(ctx, gh_aligned(s.dst, 16), GALOIS_HIP_E_ALIGN, "qkv_attn_decode: 16-byte aligned q, k, v");
    }
    gg_args a;
    gg_plan plan;
    const int32_t st = prepare_group(ctx, items, 3, what, a, plan, FA_WAVES * FA_R);
    if (st != GALOIS_HIP_OK) return st;
    // the attention's own LDS (9 KB) shares the 64 KB of a workgroup with the products' activation planes
    GH_REQUIRE(ctx, plan.max_slots <= FA_MAX_SLOTS, GALOIS_HIP_E_SHAPE, "qkv_attn_decode: ncols at most 11776");
    const int L = n_past + 1;
    const int S = (L + AT_KEYS - 1) / AT_KEYS;
    GH_REQUIRE(ctx, S <= AT_MAX_SPLITS && (S == 1 || ((int64_t)n_head * S * (head_dim + 4) <= GH_PARTIAL_FLOATS)) &&
                        ctx->scratch != nullptr && ctx->attn_done != nullptr,
               GALOIS_HIP_E_UNSUPPORTED, "qkv_attn_decode: n_head * ceil((n_past + 1) / 128) * (head_dim + 4) floats of partial "
                                         "results must fit the context's 4 MB scratch block");
    GH_REQUIRE(ctx, plan.blocks + (int64_t)n_head * S < 0x7FFFFFFF, GALOIS_HIP_E_SHAPE, "qkv_attn_decode: too many workgroups");
    fa_args<CT> b;
    b.kc = k_cache, b.vc = v_cache, b.part = (float *)ctx->scratch, b.out = out;
    b.done = ctx->attn_done, b.ready = ctx->attn_done + GH_ATTN_HEADS, b.pos = pos;
    b.H = n_head, b.L = L, b.S = S, b.gemv_blocks = (int32_t)plan.blocks;
    b.target = FA_HEAD_DIM / (FA_WAVES * FA_R) + (uint32_t)ctx->wait_target_bias;  // product workgroups per head
    b.spin_limit = ctx->wait_spin_limit, b.status = ctx->dev_status_dev;
    GH_REQUIRE(ctx, b.status != nullptr, GALOIS_HIP_E_UNSUPPORTED, "qkv_attn_decode: the context has no status word");
    b.freq_scale = freq_scale, b.theta_scale = theta_scale, b.scale = scale;
    b.key_stride = head_major_n_ctx ? head_dim : (int64_t)n_head * head_dim;
    b.head_stride = head_major_n_ctx ? (int64_t)head_major_n_ctx * head_dim : head_dim;
    GH_BIND(ctx);
    const dim3 grid((unsigned)(plan.blocks + (int64_t)n_head * S)), block(FA_WAVES * 64);
    size_t lds = (size_t)plan.max_slots * slot_lds<5>::bytes_per_slot;
    constexpr int PGMAX = (kChunkSlots * 8 + FA_WAVES * 64 - 1) / (FA_WAVES * 64);
    const bool short_vec = plan.max_slots <= 64;
    if (plan.mode == 1 && short_vec) lds += (size_t)plan.max_slots * 64 * sizeof(float);  // staged, weighted activations
#define FA_LAUNCH(PG_, MODE_) \
    hipLaunchKernelGGL((qkv_attn_decode_fused<PG_, MODE_, CT>), grid, block, lds, ctx->stream, a, b)
    if (short_vec) {
        if (plan.mode == 0) FA_LAUNCH(1, 0);
        else if (plan.mode == 1) FA_LAUNCH(1, 1);
        else FA_LAUNCH(1, 2);
    } else {
        if (plan.mode == 0) FA_LAUNCH(PGMAX, 0);
        else if (plan.mode == 1) FA_LAUNCH(PGMAX, 1);
        else FA_LAUNCH(PGMAX, 2);
    }
#undef FA_LAUNCH
    GH_LAUNCH_CHECK(ctx, what);
}

}  // namespace

extern "C" int32_t galois_hip_dequantize_mul_mat_vec_q4_0(galois_hip_ctx *ctx, const void *vx, const float *y,
                                                          float *dst, int32_t ncols, int32_t nrows) {
    GH_REQUIRE_CTX(ctx);
    GH_REQUIRE(ctx, vx && y && dst, GALOIS_HIP_E_NULL, "dequantize_mul_mat_vec_q4_0");
    GH_REQUIRE(ctx, ncols > 0 && nrows > 0 && ncols % 32 == 0, GALOIS_HIP_E_SHAPE,
               "dequantize_mul_mat_vec_q4_0: ncols must be a positive multiple of 32, nrows positive");
    GH_REQUIRE(ctx, gh_aligned(vx, 2) && gh_aligned(y, 4) && gh_aligned(dst, 4), GALOIS_HIP_E_ALIGN,
               "dequantize_mul_mat_vec_q4_0");
    GH_BIND(ctx);
    // GALOIS_HIP_OPT_GEMV_F32_ARITHMETIC: the caller asked for the reference's f32 multiply-add, weight by weight
    const bool fast = (ncols % 64 == 0) && gh_aligned(vx, 4) && gh_aligned(y, 8) && !ctx->gemv_f32;
    if (fast) {
        const int nslots = ncols / 64;
        // Workgroup shape by rows per CU: few rows -> 16 waves x 1 row so every SIMD has work and the
        // activation preparation is spread over 1024 threads; more rows -> 8 waves x 2 rows, several
        // workgroups resident per CU so one's preparation overlaps another's streaming.
        const int64_t rows_per_cu = ((int64_t)nrows + ctx->n_cu - 1) / ctx->n_cu;
        if (rows_per_cu <= 16)
            launch_dot8<5, 1, 1, 16, 4>(ctx, vx, y, dst, nslots, nrows);  // 16 rows per workgroup, 16 waves
        else
            launch_dot8<5, 2, 1, 8, 4>(ctx, vx, y, dst, nslots, nrows);   // 16 rows per workgroup, 8 waves
    } else {
        hipLaunchKernelGGL(gemv_q4_0_generic, dim3((nrows + 3) / 4), dim3(256), 0, ctx->stream, (const uint16_t *)vx,
                           y, dst, ncols / 32, nrows);
    }
    GH_LAUNCH_CHECK(ctx, "dequantize_mul_mat_vec_q4_0 launch");
}

extern "C" int32_t galois_hip_dequantize_mul_mat_vec_q4_0_group(galois_hip_ctx *ctx, const galois_hip_gemv_item *items,
                                                                int32_t n_items) {
    GH_REQUIRE_CTX(ctx);
    return launch_group(ctx, items, n_items, "dequantize_mul_mat_vec_q4_0_group");
}

extern "C" int32_t galois_hip_qkv_attn_decode_f32(galois_hip_ctx *ctx, const galois_hip_gemv_item *qkv, float *k_cache,
                                                  float *v_cache, float *out, int32_t n_head, int32_t head_dim,
                                                  int32_t n_past, const int32_t *pos, float freq_scale, float theta_scale,
                                                  float scale, int32_t head_major_n_ctx) {
    return launch_qkv_attn<float>(ctx, qkv, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale, theta_scale,
                                  scale, head_major_n_ctx, "qkv_attn_decode_f32");
}

extern "C" int32_t galois_hip_qkv_attn_decode_f16kv(galois_hip_ctx *ctx, const galois_hip_gemv_item *qkv, void *k_cache,
                                                    void *v_cache, float *out, int32_t n_head, int32_t head_dim,
                                                    int32_t n_past, const int32_t *pos, float freq_scale,
                                                    float theta_scale, float scale, int32_t head_major_n_ctx) {
    return launch_qkv_attn<_Float16>(ctx, qkv, (_Float16 *)k_cache, (_Float16 *)v_cache, out, n_head, head_dim, n_past, pos,
                                     freq_scale, theta_scale, scale, head_major_n_ctx, "qkv_attn_decode_f16kv");
}
