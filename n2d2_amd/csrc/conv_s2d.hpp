// First-layer convolution (at most 4 input channels, stride 2, square kernel of 3, 5 or 7) on an input stored
// space-to-depth: a 2 x 2 block of input pixels with their (at most) 4 channel slots is one 16-byte pixel, so the
// stride-2 K x K convolution becomes a stride-1 convolution of ceil((K + f) / 2)^2 such pixels (f = 1 front zero tap
// when the padding is odd) whose every tap is one aligned 16-byte read and whose padding is a border of stored zeros.
#pragma once

#include "common.h"

namespace n2d2hip {

struct ConvS2dArgs {
    const signed char* in;       // [B][Hp][Wp] pixels of 16 bytes (dy, dx, channel slot), border included
    int Hp, Wp;
    int total;                   // B * Hp * Wp positions
    const signed char* wk;       // [64-channel rows][KS * 32]: K step (ky', half) = pixels kx' = 2 * half, 2 * half + 1 of row ky'
    int ty, tx;                  // window origin of output (0, 0) in the bordered image
    int OH, OW;
    unsigned wp_mul, wp_sh;      // division by Wp
    void* out;
    int out_cs;
    int out_bytes;               // size of the output buffer (plain convolution)
    unsigned out_xor;
    const int *ta, *tb, *tc, *td, *te;      // rescale tables (bias folded in); H16: tc, td scaled up
    int lo, hi, preclamp;
    // strips: a block takes strips nstrips apart; a strip is rows_per_strip consecutive rows (of pooled rows with POOL) of
    // one image, computed tile by tile (TR convolution rows each)
    int nstrips, strips_per_image, rows_per_strip;
    int TR, T, NT;               // rows, positions (TR * Wp) and 32-position wave tiles of a tile
    int PF;                      // positions loaded before a strip's first tile (multiple of 64)
    // POOL: 3x3 stride-2 max pooling behind the convolution
    int pool_pad, POH, POW, pool_halo, POHp, POWp;
#ifdef N2D2HIP_PROFILE
    long long* prof;
#endif
};

// Bytes of the weights in the kernel's order, and the reordering (host): `w` is the caller's OCHW array.
size_t conv_s2d_weight_bytes(int O, int k, int pad);
void conv_s2d_weight_layout(const signed char* w_ochw, int C, int O, int k, int padT, int padL, signed char* out);
// Border (in 16-byte pixels, every side; an even number) an H x W input is given for this kernel size and padding; -1: not
// served.
int conv_s2d_halo(int k, int padT, int padL, int padB, int padR, int H, int W);
// hi16: scaled-up tables; pool: with the max pooling; nblk: 32-channel blocks a work-group computes (1 or 2);
// channel_tiles: work-groups along the channels (blockIdx.y), each computing 32 * nblk of them for every strip.
int conv_s2d_launch(ConvS2dArgs a, int k, bool hi16, bool pool, int nblk, int blocks, int channel_tiles, hipStream_t stream);

} // namespace n2d2hip
