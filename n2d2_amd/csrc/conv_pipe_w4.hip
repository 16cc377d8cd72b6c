// The pipelined implicit-GEMM convolution for 4-bit weights: the instantiations of conv_pipe_kernel that keep the weights
// packed two per byte in memory and in LDS, and the host side of that layout.
#include "conv_pipe.hpp"

namespace n2d2hip {

size_t conv_pipe_w4_image_bytes(int rows, int ktot)
{
    return (size_t)rows * ktot / 2;
}

// `w` is [rows][ktot] int8 holding values in [-8, 7], rows a multiple of 32, ktot a multiple of 64.  The image is, per 32
// rows and per 64 of K, one 1 KB chunk: row r at byte 32 r, its four groups of 16 weights at 8-byte slots
// s ^ ((r >> 3) & 3) (so that the 32 rows one LDS read touches fall on different banks); in a slot, byte b of dword q
// holds weight 8q + b in its lower and weight 8q + 4 + b in its upper nibble.
void conv_pipe_w4_image(const signed char* w, int rows, int ktot, signed char* image)
{
    const int niter = ktot / 64;
    for (int g = 0; g < rows / 32; ++g)
        for (int it = 0; it < niter; ++it) {
            signed char* chunk = image + ((size_t)g * niter + it) * 1024;
            for (int r = 0; r < 32; ++r) {
                const signed char* src = w + (size_t)(g * 32 + r) * ktot + it * 64;
                for (int s = 0; s < 4; ++s)
                    for (int q = 0; q < 2; ++q)
                        for (int b = 0; b < 4; ++b) {
                            const int lo = src[s * 16 + 8 * q + b] & 15, hi = src[s * 16 + 8 * q + 4 + b] & 15;
                            chunk[r * 32 + ((s ^ ((r >> 3) & 3)) << 3) + 4 * q + b] = (signed char)(lo | (hi << 4));
                        }
            }
        }
}

namespace {

#ifndef W4_S128
#define W4_S128 3
#endif

// valid: 1 = 1x1 without padding, 2 = any kernel whose every tap reads inside the (physical) input, e.g. an input that
// carries its padding, 0 = per-tap validity bits
template <int BK, int S, int NI, int NJ, int WGM, int V>
void launch_valid(const ConvPipeArgs& a, bool hi16, int grid, hipStream_t stream)
{
    constexpr int NW = 4;
    if (a.res) {
        // residual sum in the epilogue; 16-bit pairs when the host has shown that they hold every intermediate
        if (a.sum16) N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, V, true, true, true), dim3(grid), dim3(NW * 64), 0, stream, a);
        else N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, V, true, false, true), dim3(grid), dim3(NW * 64), 0, stream, a);
    } else {
        if (hi16) N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, V, false, true, true), dim3(grid), dim3(NW * 64), 0, stream, a);
        else N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, V, false, false, true), dim3(grid), dim3(NW * 64), 0, stream, a);
    }
}

template <int BK, int S, int NI, int NJ, int WGM>
void launch_bk(ConvPipeArgs a, int valid, bool hi16, int grid, hipStream_t stream)
{
    a.c.niter = a.c.ktot / BK;
    a.cper = a.c.in_cs / BK;
    if (valid == 1) launch_valid<BK, S, NI, NJ, WGM, 1>(a, hi16, grid, stream);
    else if (valid == 2) launch_valid<BK, S, NI, NJ, WGM, 2>(a, hi16, grid, stream);
    else launch_valid<BK, S, NI, NJ, WGM, 0>(a, hi16, grid, stream);
}

// K advances by whole 128-byte lines of pixels (two weight chunks per channel block and stage) when the channel count
// allows, as with 8-bit weights; the packed weights leave room for a third ring stage.
template <int NI, int NJ, int WGM>
void launch(const ConvPipeArgs& a, int valid, bool hi16, int grid, hipStream_t stream)
{
    if (a.c.in_cs % 128 == 0) launch_bk<128, W4_S128, NI, NJ, WGM>(a, valid, hi16, grid, stream);
    else launch_bk<64, 4, NI, NJ, WGM>(a, valid, hi16, grid, stream);
}

} // namespace

int conv_pipe_w4_launch(ConvPipeArgs a, int tile, int valid, bool hi16, int grid, hipStream_t stream)
{
    N2D2HIP_REQUIRE(a.c.epi.kind == EPI_I24 && a.c.ktot % 64 == 0 && a.c.in_cs % 64 == 0, N2D2HIP_ERR_INVALID,
                    "conv_pipe_w4: integer rescale and a multiple of 64 channels expected");
    if (tile == 0) launch<2, 1, 4>(a, valid, hi16, grid, stream);
    else if (tile == 1) launch<2, 2, 2>(a, valid, hi16, grid, stream);
    else launch<2, 1, 2>(a, valid, hi16, grid, stream);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // namespace n2d2hip
