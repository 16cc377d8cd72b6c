// Interface between the convolution host code (conv_igemm.hip) and the kernel that computes the second half of a residual
// bottleneck in one launch (conv_chain.hip): 3x3 convolution, 1x1 expansion to four times the channels, two-input sum.
#pragma once

#include "conv_pipe.hpp"

namespace n2d2hip {

struct ConvChainArgs {
    // The 3x3 convolution as the pipelined kernel takes it (no padding left: the input carries it as a border; scaled-up
    // rescale tables in c.epi.c / c.epi.d), with the block's output in c.out / c.out_cs / c.out_xor / out_halo /
    // out_pixels and the sum's other input, tables and ranges in the folded-sum fields (16-bit pairs).
    ConvPipeArgs p;
    const signed char* we;      // expansion weights in matrix-core fragment order (conv_chain_weight_layout)
    const int* etc;             // expansion's multiplier and addend, scaled up (result in the upper half)
    const int* etd;
    int e_lo, e_hi;             // saturation range of the expansion's own activation
    unsigned t2_xor;            // 0x80808080 when the expansion reads its input as value - 128
#ifdef N2D2HIP_PROFILE
    long long* prof;            // one 16-counter record per block
#endif
};

// Middle channel counts the kernel is built for; the expansion has four times as many outputs.
bool conv_chain_channels(int cmid);
// Bytes of the expansion's weights in fragment order, and the reordering (host): `w` is [O rows][row_bytes] int8, row o
// holding the C weights of output o.
size_t conv_chain_weight_bytes(int C, int O);
void conv_chain_weight_layout(const signed char* w, int row_bytes, int C, int O, signed char* frag);
// Launches the kernel for cmid = a.p.c.in_cs middle channels; fills in the tiling fields of a.p.
int conv_chain_launch(ConvChainArgs a, int num_cus, hipStream_t stream);

} // namespace n2d2hip
