// What a quantized ConvCell / FcCell handle holds (shared by the translation units that launch its kernels).
#pragma once

#include "common.h"

struct n2d2hip_conv_s {
    n2d2hip_conv_desc desc;
    n2d2hip_act_t act;
    int in_dtype;
    int in_cs;            // channel stride the weights were prepared for
    bool depthwise;
    bool pix4;
    int opad;             // weight rows (multiple of 128)
    int ktot;
    signed char* d_w;
    int4* d_sub;
    int* d_bias;
    signed char* d_fill;  // 16 bytes of the input's logical zero, source of padded taps in the direct-to-LDS kernel
    bool preclamp;        // some accumulator could overflow the rescale's 24x24 -> 32 bit product, or the cell has a Clip
    // residual sum folded into the epilogue (n2d2hip_conv_fuse_sum)
    n2d2hip_elemwise_t sum;
    int sum_other_dtype;  // storage type the tables below were made for
    // sum a,b,c,d,e then pre a,b,c,d,e, each [cpad], zero point of the other input folded in; then the sum's c, d, e as
    // 16-bit pairs, each [cpad / 2]
    int* d_res_tab;
    bool has_pre, pre_clamp, sum_clamp;
    bool sum16;           // the 16-bit pairs may be used: every intermediate behind the convolution's shift fits 16 bits
    bool pre_in_range;    // the folded ScalingCell maps every byte into its output range
    // integer rescale with the bias folded in, for the pipelined kernel: a - bias, b - bias, c, d + bias * c, e, each [cpad]
    // ... then, when hi16: c << (16 - e) and (d + bias * c) << (16 - e), which leave the rescaled value in the upper half
    // of the 32-bit result
    int* d_epi_tab;
    bool bias_folded;
    bool hi16;
    // first-layer kernel (<= 4 input channels, horizontal stride 2): weights as [channel][kH * 32]
    signed char* d_wstem;
    // first-layer kernel on space-to-depth inputs (<= 4 input channels, square kernel of 3 / 5 / 7, stride 2): weights per K step
    signed char* d_ws2d;
    // 3x3 stride-1 kernel over inputs that carry their padding: weights in matrix-core fragment order
    signed char* d_wfrag;
    // 1x1 expansion (C -> 4C, C = 64, 128 or 256) behind a 3x3 convolution in one launch: weights in fragment order
    signed char* d_wchain;
    // 3x3 depthwise kernel: per channel and kernel row the three weights in one dword, then the biases with the zero point folded in
    int* d_wdw;
    // 4-bit weights for the pipelined kernel: the ring's weight tiles as LDS wants them, two weights per byte
    signed char* d_w4img;
    // direct kernel for layers with a handful of channels: [tap][8 | 16 | 32 output rows][input channel stride]
    signed char* d_wsmall;
    bool is_fc;
    int fcH, fcW;
    // sub-sampling (desc.subX or subY > 1): the convolution proper is a handle of its own that stores raw sums without a
    // bias; one more launch adds them up per window, adds the bias and applies the cell's activation.  The other fields
    // above stay empty on such a handle.
    n2d2hip_conv_s* sub_inner;
    n2d2hip_act_t sub_raw_act;
    int* d_sub_bias;            // [O] or null
    int* d_sub_sums;            // raw sums of the last forward (grown on demand, kept until the handle goes)
    size_t sub_sums_bytes;
};

