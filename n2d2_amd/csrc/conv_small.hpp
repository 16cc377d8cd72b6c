// Interface between the convolution host code (conv_igemm.hip) and the direct kernel for layers with a handful of
// channels (conv_small.hip).
#pragma once

#include "common.h"

namespace n2d2hip {

// A convolution with at most 16 input channels and at most 32 outputs (LeNet's layers; a matrix-core tile would be
// almost all padding): one thread per output pixel, 4-way byte dot products, any kernel size, stride, padding and dilation.
struct ConvSmallArgs {
    const signed char* in;      // NHWC bytes, channel stride in_cs (4 or 16), no halo
    int in_cs;
    int qn;                     // dwords of a pixel that hold channels: ceil(C / 4)
    int B, H, W;
    const signed char* w;       // [tap][rows][in_cs] (conv_small_weight_layout)
    int rows;                   // conv_small_rows of the layer
    const int* bias;            // per output, the input's zero point folded in
    void* out;                  // NHWC bytes, channel stride out_cs
    int out_cs, out_dtype;
    int O, OH, OW;
    int kW, kH, strideX, strideY, padL, padT, dilX, dilY;
    unsigned fill;              // four bytes of the input's stored 0 (taps outside the image)
    EpiArgs epi;
};

// Output rows the kernel is built for (8, 16 or 32) for a layer with O outputs, 0 if it does not serve the shape.
int conv_small_rows(int C, int O, int taps);
size_t conv_small_weight_bytes(int C, int O, int taps);
// `w` is [O][kH][kW][C] int8 (C channels, not padded); `img` receives [tap][rows][cs].
void conv_small_weight_layout(const signed char* w, int C, int O, int taps, signed char* img);
int conv_small_launch(const ConvSmallArgs& a, hipStream_t stream);

} // namespace n2d2hip
