// Arguments shared by the implicit-GEMM convolution kernels.
#pragma once

#include "common.h"

namespace n2d2hip {

struct ConvArgs {
    const signed char* in;
    int in_cs, B, H, W;
    int OH, OW, M;          // M = B*OH*OW output pixels
    const signed char* w;   // prepared weights
    int ktot;               // K bytes per weight row (multiple of 64)
    int niter;              // ktot / 64
    const int4* sub;        // sub-chunk table, ktot/16 entries
    const int* bias;        // [Opad], zero-point fold included
    void* out;
    int out_cs, out_dtype;
    int strideX, strideY, padL, padT, dilX, dilY;
    int kW, kH;
    int ntiles_n, nblocks;
    unsigned fill;          // padding byte replicated 4x (logical zero of the input)
    unsigned out_xor;       // 0x80808080 when the output is stored as value-128
    EpiArgs epi;
};

} // namespace n2d2hip
