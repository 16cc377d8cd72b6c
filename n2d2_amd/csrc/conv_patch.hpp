// Interface between the convolution host code (conv_igemm.hip) and the 3x3 "patch" kernel (conv_patch.hip).
#pragma once

#include "common.h"

namespace n2d2hip {

// A 3x3, stride 1, undilated convolution over an NHWC byte tensor that carries its padding as a border of zeros (halo 1),
// input and output channel counts multiples of 64, integer rescale with the bias folded into its tables.
struct ConvPatchArgs {
    const signed char* in;      // B x Hp x Wp x C bytes, borders hold the storage form of 0
    const signed char* wfrag;   // weights in matrix-core fragment order (conv_patch_weight_layout)
    void* out;                  // NHWC bytes
    int C, O;
    int Hp, Wp;                 // input rows / columns per image, borders included
    int total;                  // B * Hp * Wp input positions
    int nchunk;                 // C / 64
    int out_cs, out_halo, OHp, OWp;   // output channel stride, its border, rows / columns per image with the border
    unsigned out_xor;           // 0x80808080 when the output is stored as value - 128
    int mtiles, ntiles_n, xcd_tiles, mlanes;
    unsigned img_mul, img_sh, row_mul, row_sh;    // division by Hp * Wp and by Wp
    // rescale tables of the output channels, bias folded in.  P16: c, d scaled up (result in the upper half); else a..e
    const int* ta; const int* tb; const int* tc; const int* td; const int* te;
    int lo, hi;                 // saturation range
    int preclamp;               // clamp the accumulator to [a, b] before the multiply (32-bit rescale only)
#ifdef N2D2HIP_PROFILE
    long long* prof;            // one 16-counter record per block
#endif
};

// Bytes of a convolution's weights in fragment order, and the reordering itself (host): `w` is [O][ky][kx][C] int8.
size_t conv_patch_weight_bytes(int C, int O);
void conv_patch_weight_layout(const signed char* w, int C, int O, signed char* frag);
// Can the kernel serve this shape (Wp = input columns with the border)?
bool conv_patch_eligible(int C, int O, int Wp);
// Launches the kernel; hi16 selects the scaled-up tables.  `blocks` is filled in (mtiles ... mlanes) here.
// tile_m: positions per block tile, 128 or 256, or 64 for four waves of 64 positions per block (a tile of 256 for layers of 64
// outputs per block); 0 lets the launch choose by the layer's channels and by how many blocks the tensor gives the chip.
int conv_patch_launch(ConvPatchArgs a, bool hi16, int num_cus, int tile_m, hipStream_t stream);

} // namespace n2d2hip
