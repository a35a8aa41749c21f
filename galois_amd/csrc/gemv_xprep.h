// Activation preparation for the Q4_0 decode GEMV: f32 -> signed 4-bit limb planes.
//
// The GEMV multiplies 4-bit weights with v_dot8_i32_i4 (eight int4 x int4 products per
// lane per instruction).  For that the f32 activations of one Q4_0 block (32 values) are
// turned into a block-scaled fixed-point integer X = rne(x * 2^(XBITS-1-e)), where
// 2^e <= max|x| < 2^(e+1), and X is written in balanced base 16: X = sum_l s_l * 16^l
// with every digit s_l in [-8, 7].  Digit l of eight activations is packed into one dword
// ("limb plane") in the nibble order of the weight dword they multiply, so that
//     sum_k (q_k - 8) * x_k  =  2^(e-XBITS+1) * sum_l 16^l * dot8(weights ^ 0x88888888, plane_l)
// holds exactly in integer arithmetic; the only rounding is that of x to XBITS-1 fractional
// bits below its block's leading power of two (2^-21 relative for 6 limbs).
//
// What the rounding drops is not lost.  The residual r = x - X * 2^(e-XBITS+1) is exact in f32 and at most half a
// grid step, 2^(e-XBITS).  That is 2^(1-XBITS) of a block's largest activation, but it can be all of a small one:
// a block in which one activation towers over the rest leaves the rest few bits, or none.  The decision is made on
// the sum of |x| over the block without its largest activation: if that sum is below 31 half steps times 2^13, the
// block gets a correction block -- the residuals of its activations below the top binade, in the same fixed-point
// form with their own scale and CORR_L limbs -- and the kernel adds dot(weights, correction planes) for it, which
// takes those activations to 2^-13 of their largest residual (at most 2^-31 of the block's largest activation).
// In every other block the activations other than the largest satisfy  sum |r_k| <= 2^-13 * sum |x_k|
// (the bound; rounding errors are spread over +-half a step, so the typical sum is half of that and signed).
// The threshold is a trade: a block of 32 N(0,1) values is never flagged, the product-shaped values of a SwiGLU
// (silu(g) * u) once in two thousand blocks; at 2^14 it was one block in fifty, enough for every workgroup of a
// down projection to run the correction code for a lane or two in every pass.
// A block too small for a grid of its own (largest activation below 2^-108) lives in its correction block alone.
//
// Plain C++ (no HIP builtins) so the same code is unit-tested on the CPU.
#pragma once
#include <stdint.h>
#include <string.h>

#ifdef __HIPCC__
#define GH_HD __host__ __device__ __forceinline__
#else
#define GH_HD inline
#endif

namespace xprep {

template <int L>
struct limb_cfg {
    static_assert(L >= 2 && L <= 6, "2..6 limbs");
    static constexpr int xbits = 4 * L - 2;                                  // |X| <= 2^xbits
    static constexpr uint32_t bias = (uint32_t)(0x88888888ull >> (4 * (8 - L)));  // 8 in each of L digits
};

GH_HD uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
GH_HD float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// Byte of the 16-byte qs array that nibble pair t (0..3) of weight-dword group g (0..7) holds:
// groups 0..3 are bytes 0-3, 4-7, 8-11, 12-15 of block A, groups 4..7 the same of block B.
// (A 36-byte slot is two blocks; block A's qs start 2 bytes into the slot, so the kernel
// assembles each of its four dwords from two neighbouring ones.)  A group's activations are
// then two runs of four consecutive floats, 16 apart: two aligned 16-byte pieces.
GH_HD int group_byte(int g, int t) { return 4 * (g & 3) + t; }

// Index (within the 64 activations of a slot) of nibble j (0..7) of group g:
// even nibbles are the low nibbles (weight b), odd nibbles the high nibbles (weight 16+b).
GH_HD int group_x_index(int g, int j) { return (g >= 4 ? 32 : 0) + group_byte(g, j >> 1) + ((j & 1) ? 16 : 0); }

// Scale pair for a block whose max|x| has f32 bits `amax_bits`: `mult` maps x to the integer
// grid, `scale` maps integer dot products back.  Both are powers of two (or 0 / NaN).
template <int L>
GH_HD void block_scales(uint32_t amax_bits, float *mult, float *scale) {
    const int eb = (int)((amax_bits >> 23) & 0xFF);
    constexpr int xb = limb_cfg<L>::xbits;
    if (eb == 255) {  // inf or nan in the block: poison the block's contribution
        *mult = 0.0f;
        *scale = bits_f32(0x7FC00000u);
    } else if (eb <= xb) {  // zero, subnormal or below 2^-100: contributes nothing representable
        *mult = 0.0f;
        *scale = 0.0f;
    } else {
        *mult = bits_f32((uint32_t)(253 + xb - eb) << 23);
        *scale = bits_f32((uint32_t)(eb - xb + 1) << 23);
    }
}

// x * mult rounded to nearest-even integer, offset by `bias`, digits made signed:
// returns the L balanced digits of X as packed 4-bit two's-complement nibbles.
template <int L>
GH_HD uint32_t signed_digits(float x, float mult) {
    const float f = __builtin_fmaf(x, mult, 12582912.0f);  // 1.5 * 2^23: integer lands in the mantissa
    const uint32_t y = f32_bits(f) - 0x4B400000u + limb_cfg<L>::bias;
    return y ^ limb_cfg<L>::bias;
}

// What signed_digits rounds away: x - X * scale with X = rne(x * mult) and scale = 1 / mult, exact in f32 (X * scale
// is a multiple of scale no further than scale / 2 from x, so the difference needs no more bits than x has).
// A block without a grid (mult = scale = 0: nothing above 2^-100) keeps all of x; a non-finite block gives NaN.
GH_HD float residual(float x, float mult, float scale) {
    const float X = __builtin_fmaf(x, mult, 12582912.0f) - 12582912.0f;
    return __builtin_fmaf(-X, scale, x);
}

constexpr int CORR_L = 4;                       // limbs of a correction block
constexpr float CORR_REST_FACTOR = 126976.0f;   // 31 * 2^12: 31 half grid steps times 2^13, in grid steps

// Whether |x| (as f32 bits with the sign cleared) lies below the top binade of a block whose largest |x| has the
// bits amax_bits: a correction block holds the residuals of such activations only (the others keep 2^(1-XBITS)).
GH_HD bool below_top_binade(uint32_t abs_bits, uint32_t amax_bits) { return abs_bits < (amax_bits & 0x7F800000u); }

// Whether a block gets a correction block: sum_abs_x is the block's sum of |x|, amax_bits its largest |x| and
// scale its grid step (block_scales).  False for a block with an inf or NaN in it: its scale already poisons the
// result.
GH_HD bool needs_correction(float sum_abs_x, uint32_t amax_bits, float scale) {
    const float rest = sum_abs_x - bits_f32(amax_bits);
    return rest < CORR_REST_FACTOR * scale || (scale == 0.0f && amax_bits != 0);
}

// 8x8 nibble transpose: in[j] nibble l  ->  out[l] nibble j.
GH_HD void transpose_nibbles(const uint32_t in[8], uint32_t out[8]) {
    uint32_t a[8], b[8];
    // 4x4 blocks of nibbles (16-bit halves) between rows j and j+4
    for (int j = 0; j < 4; j++) {
        a[j] = (in[j] & 0x0000FFFFu) | (in[j + 4] << 16);
        a[j + 4] = (in[j] >> 16) | (in[j + 4] & 0xFFFF0000u);
    }
    // 2x2 blocks (bytes) between rows j and j+2
    for (int h = 0; h < 8; h += 4)
        for (int j = h; j < h + 2; j++) {
            b[j] = (a[j] & 0x00FF00FFu) | ((a[j + 2] & 0x00FF00FFu) << 8);
            b[j + 2] = ((a[j] >> 8) & 0x00FF00FFu) | (a[j + 2] & 0xFF00FF00u);
        }
    // single nibbles between rows j and j+1
    for (int j = 0; j < 8; j += 2) {
        out[j] = (b[j] & 0x0F0F0F0Fu) | ((b[j + 1] & 0x0F0F0F0Fu) << 4);
        out[j + 1] = ((b[j] >> 4) & 0x0F0F0F0Fu) | (b[j + 1] & 0xF0F0F0F0u);
    }
}

// Eight activations (already in nibble order of their weight dword) -> L limb planes.
template <int L>
GH_HD void make_planes(const float x[8], float mult, uint32_t planes[L]) {
    uint32_t s[8], t[8];
    for (int j = 0; j < 8; j++) s[j] = signed_digits<L>(x[j], mult);
    transpose_nibbles(s, t);
    for (int l = 0; l < L; l++) planes[l] = t[l];
}

}  // namespace xprep
