// CPU shim over galois_amd/csrc/gemv_xprep.h so pytest can check the activation-limb
// preparation (the host-testable half of the decode GEMV) without a GPU.
#include "../galois_amd/csrc/gemv_xprep.h"

template <int L>
static void slot_planes(const float *x64, uint32_t *planes /* [L][8] */, float *scales /* [2] */) {
    for (int blk = 0; blk < 2; blk++) {
        uint32_t amax = 0;
        for (int k = 0; k < 32; k++) {
            uint32_t b = xprep::f32_bits(x64[32 * blk + k]) & 0x7FFFFFFFu;
            amax = b > amax ? b : amax;
        }
        float mult, scale;
        xprep::block_scales<L>(amax, &mult, &scale);
        scales[blk] = scale;
        for (int g = 4 * blk; g < 4 * blk + 4; g++) {
            float v[8];
            for (int j = 0; j < 8; j++) v[j] = x64[xprep::group_x_index(g, j)];
            uint32_t p[L];
            xprep::make_planes<L>(v, mult, p);
            for (int l = 0; l < L; l++) planes[l * 8 + g] = p[l];
        }
    }
}

// What the kernel's preparation leaves in LDS for one slot, corrections included: a thread holds the eight
// activations of one weight-dword group, the four threads of a block add up their |r| and |x| pairwise
// ((t0 + t1) + (t2 + t3), the order of the kernel's two quad exchanges).
template <int L>
static void slot_full(const float *x64, uint32_t *planes, float *scales, uint32_t *planes2 /* [CORR_L][8] */,
                      float *scales2 /* [2] */) {
    constexpr int CL = xprep::CORR_L;
    slot_planes<L>(x64, planes, scales);
    for (int blk = 0; blk < 2; blk++) {
        uint32_t amax = 0;
        for (int k = 0; k < 32; k++) {
            uint32_t b = xprep::f32_bits(x64[32 * blk + k]) & 0x7FFFFFFFu;
            amax = b > amax ? b : amax;
        }
        float mult, scale;
        xprep::block_scales<L>(amax, &mult, &scale);
        float r[4][8], sx[4];
        uint32_t rmax = 0;
        const bool no_grid = scale == 0.0f;
        for (int t = 0; t < 4; t++) {
            sx[t] = 0.0f;
            for (int j = 0; j < 8; j++) {
                const float x = x64[xprep::group_x_index(4 * blk + t, j)];
                const bool low = no_grid || xprep::below_top_binade(xprep::f32_bits(x) & 0x7FFFFFFFu, amax);
                r[t][j] = low ? xprep::residual(x, mult, scale) : 0.0f;
                const uint32_t b = xprep::f32_bits(r[t][j]) & 0x7FFFFFFFu;
                sx[t] += __builtin_fabsf(x);
                rmax = b > rmax ? b : rmax;
            }
        }
        const float sum_x = (sx[0] + sx[1]) + (sx[2] + sx[3]);
        scales2[blk] = 0.0f;
        for (int t = 0; t < 4; t++)
            for (int l = 0; l < CL; l++) planes2[l * 8 + 4 * blk + t] = 0;
        if (xprep::needs_correction(sum_x, amax, scale)) {
            float mult2;
            xprep::block_scales<CL>(rmax, &mult2, &scales2[blk]);
            for (int t = 0; t < 4; t++) {
                uint32_t p[CL];
                xprep::make_planes<CL>(r[t], mult2, p);
                for (int l = 0; l < CL; l++) planes2[l * 8 + 4 * blk + t] = p[l];
            }
        }
    }
}

extern "C" {
int xprep_corr_limbs() { return xprep::CORR_L; }
float xprep_residual(float x, float mult, float scale) { return xprep::residual(x, mult, scale); }
void xprep_slot_full(const float *x64, uint32_t *planes, float *scales, uint32_t *planes2, float *scales2) {
    slot_full<5>(x64, planes, scales, planes2, scales2);
}
void xprep_slot_planes(int L, const float *x64, uint32_t *planes, float *scales) {
    switch (L) {
        case 4: slot_planes<4>(x64, planes, scales); break;
        case 5: slot_planes<5>(x64, planes, scales); break;
        case 6: slot_planes<6>(x64, planes, scales); break;
    }
}
void xprep_transpose(const uint32_t *in, uint32_t *out) { xprep::transpose_nibbles(in, out); }
int xprep_group_x_index(int g, int j) { return xprep::group_x_index(g, j); }
}
