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

extern "C" {
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
