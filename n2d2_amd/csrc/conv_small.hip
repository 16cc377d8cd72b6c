// Direct convolution for layers with a handful of channels (at most 16 in, at most 32 out): LeNet's two convolutions.
// Such a layer is a few dozen multiply-adds per output; on the matrix cores its tile would be padding for the most part
// (1 input channel of 32 in a K step, 6 outputs of 64 in a tile), so each thread computes one output pixel with 4-way
// byte dot products instead.  ref: src/Cell/ConvCell_Frame_Kernels.cpp:26-174 (forward, forwardBias): a tap outside the
// image is skipped there and reads the stored form of 0 here, which adds nothing either.
#include "conv_small.hpp"
#include "epilogue.hpp"

#include <algorithm>

namespace n2d2hip {

// One thread per output pixel and group of 8 outputs (blockIdx.y).  The taps of a kernel row are loaded up front, from
// addresses clamped into the image, and replaced by the stored 0 where they lie outside only when they are used, so that
// the loads of a row are all in flight before the first dot product waits for one.
template <int CS>
__global__ __launch_bounds__(256) void conv_small_kernel(ConvSmallArgs p)
{
    extern __shared__ int lw[];         // this group's weights: [tap][CS / 4][8]
    constexpr int Q = CS / 4, ROWS = 8, KWMAX = 8;
    const int taps = p.kW * p.kH;
    const int group = blockIdx.y;
    for (int i = threadIdx.x; i < taps * ROWS * Q; i += 256) {       // lw: [tap][channel dword][8 outputs]
        const int t = i / (ROWS * Q), q = (i / ROWS) % Q, o = i % ROWS;
        lw[i] = ((const int*)p.w)[(t * p.rows + group * ROWS + o) * Q + q];
    }
    __syncthreads();
    const long long total = (long long)p.B * p.OH * p.OW;
    const long long pix = (long long)blockIdx.x * 256 + threadIdx.x;
    if (pix >= total)
        return;
    const int ox = (int)(pix % p.OW), oy = (int)((pix / p.OW) % p.OH);
    const long long b = pix / ((long long)p.OW * p.OH);
    const signed char* img = p.in + b * p.H * p.W * CS;
    const int iy0 = oy * p.strideY - p.padT, ix0 = ox * p.strideX - p.padL;
    int acc[ROWS];
#pragma unroll
    for (int o = 0; o < ROWS; ++o)
        acc[o] = 0;
    for (int ky = 0; ky < p.kH; ++ky) {
        const int iy = iy0 + ky * p.dilY;
        const bool row_in = (unsigned)iy < (unsigned)p.H;
        const signed char* row = img + (long long)min(max(iy, 0), p.H - 1) * p.W * CS;
        int x[KWMAX][Q];
#pragma unroll
        for (int kx = 0; kx < KWMAX; ++kx) {
            if (kx < p.kW) {
                const int* src = (const int*)(row + min(max(ix0 + kx * p.dilX, 0), p.W - 1) * CS);
#pragma unroll
                for (int q = 0; q < Q; ++q)
                    x[kx][q] = src[q];
            }
        }
#pragma unroll
        for (int kx = 0; kx < KWMAX; ++kx) {
            if (kx < p.kW) {
                const bool inside = row_in && (unsigned)(ix0 + kx * p.dilX) < (unsigned)p.W;
                const int* wt = lw + (ky * p.kW + kx) * ROWS * Q;      // the same address in every lane: an LDS broadcast
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    if (q < p.qn) {                                     // dwords past the last channel hold nothing
                        const int v = inside ? x[kx][q] : (int)p.fill;
#pragma unroll
                        for (int o = 0; o < ROWS; ++o)
                            acc[o] = __builtin_amdgcn_sdot4(v, wt[q * ROWS + o], acc[o], false);
                    }
                }
            }
        }
    }
    // bias, rescale, saturate; 4 channels per stored dword.  The last group also writes the stored form of 0 into the
    // channels between the last output and the channel stride.
    const unsigned out_xor = p.out_dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    unsigned* dst = (unsigned*)((signed char*)p.out + pix * p.out_cs) + 2 * group;
    unsigned v[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < ROWS; ++j) {
        const int o = group * ROWS + j;
        if (o < p.O)
            v[j / 4] |= ((unsigned)epi_apply_dyn(p.epi, acc[j] + p.bias[o], o) & 0xffu) << (8 * (j % 4));
    }
    dst[0] = v[0] ^ out_xor;
    if (8 * group + 4 < p.out_cs)
        dst[1] = v[1] ^ out_xor;
    if (group == (int)gridDim.y - 1)
        for (int g = 2 * group + 2; g < p.out_cs / 4; ++g)
            dst[g - 2 * group] = out_xor;
}

int conv_small_rows(int C, int O, int taps)
{
    if (C < 1 || C > 16 || O < 1 || O > 32 || taps < 1 || taps > 64)
        return 0;           // (the caller also checks the kernel's width: at most 8 taps per row)
    return O <= 8 ? 8 : (O <= 16 ? 16 : 32);
}

size_t conv_small_weight_bytes(int C, int O, int taps)
{
    return (size_t)taps * conv_small_rows(C, O, taps) * n2d2hip_nhwc_cs(C);
}

void conv_small_weight_layout(const signed char* w, int C, int O, int taps, signed char* img)
{
    const int rows = conv_small_rows(C, O, taps), cs = n2d2hip_nhwc_cs(C);
    memset(img, 0, conv_small_weight_bytes(C, O, taps));
    for (int o = 0; o < O; ++o)
        for (int t = 0; t < taps; ++t)
            for (int ch = 0; ch < C; ++ch)
                img[((size_t)t * rows + o) * cs + ch] = w[((size_t)o * taps + t) * C + ch];
}

int conv_small_launch(const ConvSmallArgs& a, hipStream_t stream)
{
    const int taps = a.kW * a.kH;
    const int C = a.in_cs == 4 ? 4 : 16;
    const int rows = conv_small_rows(C, a.O, taps);
    N2D2HIP_REQUIRE(rows != 0 && rows == a.rows && a.kW <= 8 && (a.in_cs == 4 || a.in_cs == 16) && a.out_cs % 4 == 0
                    && a.out_cs >= std::min(rows, 4) && is_byte_type(a.out_dtype), N2D2HIP_ERR_INVALID, "conv_small: shape not served");
    const long long total = (long long)a.B * a.OH * a.OW;
    N2D2HIP_REQUIRE(total > 0 && (total + 255) / 256 < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED, "conv_small: tensor too large");
    const dim3 grid((unsigned)((total + 255) / 256), (unsigned)((a.O + 7) / 8));
    const size_t lds = (size_t)taps * 8 * a.in_cs;
    if (a.in_cs == 4)
        N2D2HIP_LAUNCH_T(conv_small_kernel, (4), grid, dim3(256), lds, stream, a);
    else
        N2D2HIP_LAUNCH_T(conv_small_kernel, (16), grid, dim3(256), lds, stream, a);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // namespace n2d2hip
