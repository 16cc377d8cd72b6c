// Interface between the convolution host code (conv_igemm.hip) and the 3x3 depthwise kernel (depthwise.hip).
#pragma once

#include "common.h"

namespace n2d2hip {

// A 3x3 undilated depthwise convolution (groups == C == O), stride 1 or 2 in both directions, NHWC bytes in and out.
struct DepthwiseArgs {
    const signed char* in;   // B x H x W x cs bytes, signed storage (value or value - 128)
    void* out;               // B x OH x OW x cs bytes
    const int* wb;           // [3][cs] dwords (w[ky][0][c], w[ky][1][c], w[ky][2][c], 0), then [cs] biases, zero point folded in
    int cs;                  // channel stride of both tensors, a multiple of 4
    int B, H, W, OH, OW;
    int padL, padT;
    int rows;                // output rows each thread walks down
    int nstrips;             // ceil(OH / rows)
    unsigned cq;             // cs / 4
    unsigned nthreads;       // B * nstrips * OW * cq
    unsigned fill;           // the stored form of 0 in all four bytes
    unsigned out_xor;        // 0x80808080 when the output is stored as value - 128
    EpiArgs epi;
    // fast form of the integer rescale (no clamp before the multiply, saturation to [0, 255]): multiplier, rounding term
    // with the bias folded in, shift; by channel
    bool fast;
    const int* fc;
    const int* fd;
    const int* fe;
};

// Host side of the layout above: `w` is [C][3][3] int8, `bias` the biases with the zero point folded in.
void depthwise3x3_weight_layout(const signed char* w, const int* bias, int C, int cs, int* wb);
// Fills rows / nstrips / cq / nthreads and launches; stride is 1 or 2.
int depthwise3x3_launch(DepthwiseArgs a, int stride, int num_cus, hipStream_t stream);

} // namespace n2d2hip
