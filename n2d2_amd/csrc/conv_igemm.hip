// Quantized ConvCell / FcCell forward as an implicit GEMM on the gfx950 int8
// matrix cores (v_mfma_i32_32x32x32_i8), with the cell's bias, rescale,
// saturation and ReLU fused into the accumulator epilogue.
//
// Data layout in HBM
//   activations  NHWC signed bytes, channel stride `cs` (multiple of 16, or 4 for
//                <=4-channel network inputs).  Unsigned values are stored minus
//                128 (N2D2HIP_U8B) so that the signed MFMA consumes them directly;
//                the constant 128*sum(w) is folded into the bias at creation.
//   weights      [Opad][ktot] signed bytes, K ordered as 16-byte "sub-chunks":
//                (ky, kx, 16 channels) for cs%16==0, (ky, 4 taps kx..kx+3, 4
//                channels) for cs==4.  int4 weights stay nibble-packed in HBM
//                ([Opad][ktot/2]) and are widened to int8 on their way into LDS.
//   sub-chunk table  one int4 {ky, kx, channel offset, valid} per sub-chunk.
//
// GEMM view: D[channel][pixel] += W[channel][k] * X[pixel][k].  The weights are
// the MFMA "A" operand and the pixels the "B" operand, so that every lane ends
// up with 4 consecutive output channels of one pixel: one packed dword.
#include <algorithm>
#include <cstdlib>
#include <limits>
#include <type_traits>

#include "common.h"
#include "epilogue.hpp"
#include "mfma_util.hpp"
#include "conv_args.hpp"
#include "conv_patch.hpp"
#include "depthwise.hpp"

namespace n2d2hip {


__device__ __forceinline__ int swz(int row, int q)
{
    // 16-byte slot of (row, sub-chunk q) in a [rows][64 B] tile; the XOR spreads
    // 16 consecutive rows of one sub-chunk over all 64 banks.
    return ((row << 2) + (q ^ ((row >> 2) & 3))) << 4;
}

// Widens 8 nibble-packed weights (one dword: byte b = {low: w[b], high: w[b+4]})
// to two dwords of int8.
__device__ __forceinline__ void unpack_w4(unsigned p, int& lo, int& hi)
{
    const unsigned l = p & 0x0F0F0F0Fu, h = (p >> 4) & 0x0F0F0F0Fu;
    // sign-extend each nibble inside its byte: ((n ^ 8) | 0x80) - 8, then clear the guard bit
    lo = (int)(((((l ^ 0x08080808u) | 0x80808080u) - 0x08080808u)) ^ 0x80808080u);
    hi = (int)(((((h ^ 0x08080808u) | 0x80808080u) - 0x08080808u)) ^ 0x80808080u);
}

template <int BM, int BN, int WGM, int EPI, bool PIX4, bool W4>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void conv_igemm_kernel(ConvArgs p)
{
    constexpr int WGN = 4 / WGM;
    constexpr int TM = BM / WGM;      // pixels per wave
    constexpr int TN = BN / WGN;      // channels per wave
    constexpr int NI = TN / 32;       // channel tiles per wave
    constexpr int NJ = TM / 32;       // pixel tiles per wave
    constexpr int P_LOADS = BM / 64;  // 16 B loads per thread and K step, pixels
    constexpr int W_LOADS = BN / 64;  // same, weights
    constexpr int TILE_BYTES = (BM + BN) * 64;
    constexpr int STAGE_STRIDE = BN + 16;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(2 * TILE_BYTES >= BM * STAGE_STRIDE, "output staging must fit the operand buffers");

    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * TILE_BYTES];

    // XCD-aware block order: consecutive logical tiles run on the same XCD (they
    // share the pixel tile in that XCD's L2); the grid is padded to a multiple of 8.
    const int nbp = gridDim.x;
    const int logical = (blockIdx.x & 7) * (nbp >> 3) + (blockIdx.x >> 3);
    if (logical >= p.nblocks)
        return;
    const int tile_n = logical % p.ntiles_n;
    const int tile_m = logical / p.ntiles_n;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WGM;
    const int wn = wave / WGM;
    const int lq = tid & 3;       // sub-chunk this thread loads
    const int lr = tid >> 2;      // first tile row this thread loads

    // ---- per-thread pixel rows
    const signed char* rowptr[P_LOADS];
    int base_y[P_LOADS], base_x[P_LOADS];
    bool compact[P_LOADS];        // the reference's hand-unrolled 3x3 window: first 3x3 taps at undilated offsets
    const bool dilated = p.dilX != 1 || p.dilY != 1;
    const int dil_kw = p.kW + (p.dilX - 1) * (p.kW - 1), dil_kh = p.kH + (p.dilY - 1) * (p.kH - 1);
    const int ohw = p.OH * p.OW;
#pragma unroll
    for (int i = 0; i < P_LOADS; ++i) {
        const int m = m0 + lr + 64 * i;
        if (m < p.M) {
            const int b = m / ohw;
            const int rem = m - b * ohw;
            const int oy = rem / p.OW;
            const int ox = rem - oy * p.OW;
            base_y[i] = oy * p.strideY - p.padT;
            base_x[i] = ox * p.strideX - p.padL;
            rowptr[i] = p.in + (((long long)b * p.H + base_y[i]) * p.W + base_x[i]) * (long long)p.in_cs;
            // The reference recognises "a 3x3 window fully inside" by its tap bounds alone and unrolls it without the
            // dilation (ref: src/Cell/ConvCell_Frame_Kernels.cpp:95-117); a dilated kernel can meet those bounds.
            compact[i] = dilated && base_x[i] >= 0 && base_y[i] >= 0 && min(max(p.W - base_x[i], 0), dil_kw) == 3
                && min(max(p.H - base_y[i], 0), dil_kh) == 3;
        } else {
            compact[i] = false;
            base_y[i] = -(1 << 28);     // every tap test fails: the row is all padding
            base_x[i] = -(1 << 28);
            rowptr[i] = p.in;
        }
    }
    const signed char* wptr[W_LOADS];
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i)
        wptr[i] = p.w + (long long)(n0 + lr + 64 * i) * (W4 ? (p.ktot >> 1) : p.ktot) + (W4 ? lq * 8 : lq * 16);

    v4i preg[P_LOADS];
    v4i wreg[W_LOADS];

    auto load_global = [&](int it) {
        const int4 s = p.sub[it * 4 + lq];     // {ky, kx, channel offset, valid}
        const int dy = s.x * p.dilY;
#pragma unroll
        for (int i = 0; i < P_LOADS; ++i) {
            // Tap validity exactly as the reference computes its window
            // (ref: src/Cell/ConvCell_Frame_Kernels.cpp:72-83): tap index >= max(pad - o*stride, 0)
            // and dilated offset inside the input.
            const bool cmp = compact[i];
            const int dyy = cmp ? s.x : dy;
            const bool yok = s.w && (cmp ? s.x < 3 : (s.x >= -base_y[i] && base_y[i] + dy < p.H));
            if (PIX4) {
                const int* src = (const int*)(rowptr[i] + ((long long)dyy * p.W + s.y) * 4);
                v4i v;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int kx = s.y + t;
                    const bool ok = yok && (cmp ? kx < 3 : (kx >= -base_x[i] && base_x[i] + kx < p.W));
                    v[t] = ok ? src[t] : (int)p.fill;
                }
                preg[i] = v;
            } else {
                const int dx = cmp ? s.y : s.y * p.dilX;
                const bool ok = yok && (cmp ? s.y < 3 : (s.y >= -base_x[i] && base_x[i] + dx < p.W));
                if (ok) {
                    preg[i] = *(const v4i*)(rowptr[i] + ((long long)dyy * p.W + dx) * p.in_cs + s.z);
                } else {
                    const int f = (int)p.fill;
                    preg[i] = v4i{f, f, f, f};
                }
            }
        }
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            if (W4) {
                // nibble-packed: 8 bytes carry this thread's 16 weights; widened in store_lds
                const uint2 pk = *(const uint2*)(wptr[i] + (long long)it * 32);
                wreg[i] = v4i{(int)pk.x, (int)pk.y, 0, 0};
            } else {
                wreg[i] = *(const v4i*)(wptr[i] + (long long)it * 64);
            }
        }
    };
    auto store_lds = [&](int buf) {
        unsigned char* tp = smem + buf * TILE_BYTES;
        unsigned char* tw = tp + BM * 64;
#pragma unroll
        for (int i = 0; i < P_LOADS; ++i)
            *(v4i*)(tp + swz(lr + 64 * i, lq)) = preg[i];
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            if (W4) {
                v4i v;
                int a, b;
                unpack_w4((unsigned)wreg[i][0], a, b); v[0] = a; v[1] = b;
                unpack_w4((unsigned)wreg[i][1], a, b); v[2] = a; v[3] = b;
                *(v4i*)(tw + swz(lr + 64 * i, lq)) = v;
            } else {
                *(v4i*)(tw + swz(lr + 64 * i, lq)) = wreg[i];
            }
        }
    };

    v16i acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;

    load_global(0);
    store_lds(0);
    __syncthreads();

    const int l32 = lane & 31;
    const int lh = lane >> 5;
    for (int it = 0; it < p.niter; ++it) {
        const int buf = it & 1;
        if (it + 1 < p.niter)
            load_global(it + 1);          // in flight while the matrix cores work
        const unsigned char* tp = smem + buf * TILE_BYTES;
        const unsigned char* tw = tp + BM * 64;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v4i wf[NI], pf[NJ];
#pragma unroll
            for (int i = 0; i < NI; ++i)
                wf[i] = *(const v4i*)(tw + swz(wn * TN + i * 32 + l32, 2 * ks + lh));
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                pf[j] = *(const v4i*)(tp + swz(wm * TM + j * 32 + l32, 2 * ks + lh));
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], pf[j], acc[i][j], 0, 0, 0);
        }
        if (it + 1 < p.niter)
            store_lds(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: bias, rescale, saturate, ReLU, pack, coalesced store.
    // Accumulator layout of the 32x32 tile: lane holds column (pixel) lane%32 and rows
    // (channels) 8*(r/4) + 4*(lane/32) + r%4 for r = 0..15.
    const bool out_bytes = p.out_dtype != N2D2HIP_I32;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int ch_local = wn * TN + i * 32 + 8 * g + 4 * lh;
            const int ch = n0 + ch_local;
            const int4 bias4 = *(const int4*)(p.bias + ch);
            int4 ta = {0, 0, 0, 0}, tb = ta, tc = ta, td = ta, te = ta;
            if (EPI != EPI_RAW) {
                ta = *(const int4*)(p.epi.a + ch);
                tb = *(const int4*)(p.epi.b + ch);
                tc = *(const int4*)(p.epi.c + ch);
                if (EPI == EPI_I24)
                    td = *(const int4*)(p.epi.d + ch);
                if (EPI != EPI_F32)
                    te = *(const int4*)(p.epi.e + ch);
            }
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int pix_local = wm * TM + j * 32 + l32;
                const int r0 = epi_apply<EPI>(acc[i][j][4 * g + 0] + bias4.x, ta.x, tb.x, tc.x, td.x, te.x, p.epi.lo, p.epi.hi, p.epi.relu);
                const int r1 = epi_apply<EPI>(acc[i][j][4 * g + 1] + bias4.y, ta.y, tb.y, tc.y, td.y, te.y, p.epi.lo, p.epi.hi, p.epi.relu);
                const int r2 = epi_apply<EPI>(acc[i][j][4 * g + 2] + bias4.z, ta.z, tb.z, tc.z, td.z, te.z, p.epi.lo, p.epi.hi, p.epi.relu);
                const int r3 = epi_apply<EPI>(acc[i][j][4 * g + 3] + bias4.w, ta.w, tb.w, tc.w, td.w, te.w, p.epi.lo, p.epi.hi, p.epi.relu);
                if (out_bytes) {
                    const unsigned packed = ((unsigned)r0 & 255u) | (((unsigned)r1 & 255u) << 8)
                                          | (((unsigned)r2 & 255u) << 16) | ((unsigned)r3 << 24);
                    *(unsigned*)(smem + pix_local * STAGE_STRIDE + ch_local) = packed ^ p.out_xor;
                } else {
                    const int m = m0 + pix_local;
                    if (m < p.M && ch < p.out_cs)
                        *(int4*)((int*)p.out + (long long)m * p.out_cs + ch) = int4{r0, r1, r2, r3};
                }
            }
        }
    }
    if (out_bytes && p.out_cs == 4) {
        // at most 4 outputs: a pixel is one dword
        __syncthreads();
        for (int row = tid; row < BM; row += 256)
            if (n0 == 0 && m0 + row < p.M)
                *(unsigned*)((signed char*)p.out + (long long)(m0 + row) * 4) = *(const unsigned*)(smem + row * STAGE_STRIDE);
    } else if (out_bytes) {
        __syncthreads();
        constexpr int CHUNKS = BN / 16;
        for (int id = tid; id < BM * CHUNKS; id += 256) {
            const int row = id / CHUNKS;
            const int cq = id - row * CHUNKS;
            const int m = m0 + row;
            const int ch = n0 + cq * 16;
            if (m < p.M && ch < p.out_cs)
                *(v4i*)((signed char*)p.out + (long long)m * p.out_cs + ch) = *(const v4i*)(smem + row * STAGE_STRIDE + cq * 16);
        }
    }
}

} // namespace n2d2hip
#include "conv_pipe.hpp"
#include "conv_stem.hpp"
#include "conv_small.hpp"
namespace n2d2hip {

// ------------------------------------------------------------ depthwise
// groups == C == O: one output channel per input channel, no reduction over
// channels, hence no matrix core: a bandwidth kernel.  Each thread produces 4
// consecutive channels of one output pixel; weights are prepared as [tap][cs]
// so that consecutive lanes read consecutive bytes of both operands.
__global__ __launch_bounds__(256) void depthwise_kernel(const signed char* __restrict__ in, int cs, int B, int H, int W,
                                                        int OH, int OW, const signed char* __restrict__ w, int kH, int kW,
                                                        const int* __restrict__ bias, void* __restrict__ out, int out_dtype,
                                                        int strideX, int strideY, int padL, int padT, int dilX, int dilY,
                                                        int in_zp, unsigned out_xor, EpiArgs epi)
{
    const int cq = cs >> 2;
    const long long total = (long long)B * OH * OW * cq;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
        const int c4 = (int)(idx % cq) * 4;
        long long r = idx / cq;
        const int ox = (int)(r % OW); r /= OW;
        const int oy = (int)(r % OH);
        const int b = (int)(r / OH);
        const int by = oy * strideY - padT, bx = ox * strideX - padL;
        int a0 = 0, a1 = 0, a2 = 0, a3 = 0;
        // the reference's hand-unrolled 3x3 window ignores the dilation (ref: src/Cell/ConvCell_Frame_Kernels.cpp:95-117)
        const bool cmp = (dilX != 1 || dilY != 1) && bx >= 0 && by >= 0
            && min(max(W - bx, 0), kW + (dilX - 1) * (kW - 1)) == 3 && min(max(H - by, 0), kH + (dilY - 1) * (kH - 1)) == 3;
        for (int ky = 0; ky < kH; ++ky) {
            const int iy = by + (cmp ? ky : ky * dilY);
            if (cmp ? ky >= 3 : (ky < -by || iy >= H)) continue;
            for (int kx = 0; kx < kW; ++kx) {
                const int ix = bx + (cmp ? kx : kx * dilX);
                if (cmp ? kx >= 3 : (kx < -bx || ix >= W)) continue;
                const int xv = *(const int*)(in + (((long long)b * H + iy) * W + ix) * cs + c4);
                const int wv = *(const int*)(w + (long long)(ky * kW + kx) * cs + c4);
                a0 += ((int)(signed char)(xv) + in_zp) * (int)(signed char)(wv);
                a1 += ((int)(signed char)(xv >> 8) + in_zp) * (int)(signed char)(wv >> 8);
                a2 += ((int)(signed char)(xv >> 16) + in_zp) * (int)(signed char)(wv >> 16);
                a3 += ((xv >> 24) + in_zp) * (wv >> 24);
            }
        }
        const int4 b4 = *(const int4*)(bias + c4);
        const int r0 = epi_apply_dyn(epi, a0 + b4.x, c4 + 0);
        const int r1 = epi_apply_dyn(epi, a1 + b4.y, c4 + 1);
        const int r2 = epi_apply_dyn(epi, a2 + b4.z, c4 + 2);
        const int r3 = epi_apply_dyn(epi, a3 + b4.w, c4 + 3);
        if (out_dtype == N2D2HIP_I32) {
            *(int4*)((int*)out + idx * 4) = int4{r0, r1, r2, r3};
        } else {
            const unsigned packed = ((unsigned)r0 & 255u) | (((unsigned)r1 & 255u) << 8) | (((unsigned)r2 & 255u) << 16) | ((unsigned)r3 << 24);
            *(unsigned*)((signed char*)out + idx * 4) = packed ^ out_xor;
        }
    }
}

} // namespace n2d2hip

using namespace n2d2hip;

#include "conv_handle.hpp"
#include "conv_s2d.hpp"
#include "conv_chain.hpp"

namespace {

int conv_out_dim(int in, int k, int stride, int pad0, int pad1, int dil)
{
    // ref: src/Cell/ConvCell_Frame_Kernels.cpp:37-45
    return (int)((in + pad0 + pad1 - dil * (k - 1) - 1 + stride) / (double)stride);
}

template <int BM, int BN, int WGM, bool PIX4, bool W4>
void launch_cfg(const ConvArgs& a, hipStream_t stream)
{
    const int grid = round_up(a.nblocks, 8);
    switch (a.epi.kind) {
    case EPI_RAW: N2D2HIP_LAUNCH_T(conv_igemm_kernel, (BM, BN, WGM, EPI_RAW, PIX4, W4), dim3(grid), dim3(256), 0, stream, a); break;
    case EPI_I24: N2D2HIP_LAUNCH_T(conv_igemm_kernel, (BM, BN, WGM, EPI_I24, PIX4, W4), dim3(grid), dim3(256), 0, stream, a); break;
    case EPI_I64: N2D2HIP_LAUNCH_T(conv_igemm_kernel, (BM, BN, WGM, EPI_I64, PIX4, W4), dim3(grid), dim3(256), 0, stream, a); break;
    default: N2D2HIP_LAUNCH_T(conv_igemm_kernel, (BM, BN, WGM, EPI_F32, PIX4, W4), dim3(grid), dim3(256), 0, stream, a); break;
    }
}

template <int NW, int BK, int NI, int NJ, int WGM, int S>
void launch_pipe(ConvPipeArgs a, int valid, bool hi16, int grid, hipStream_t stream)
{
    a.c.niter = a.c.ktot / BK;
    a.cper = a.c.in_cs / BK;
#define N2D2HIP_PIPE(EPI) \
    do { if (valid == 1) N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI, S, 1), dim3(grid), dim3(NW * 64), 0, stream, a); \
         else if (valid == 2) N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI, S, 2), dim3(grid), dim3(NW * 64), 0, stream, a); \
         else N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI, S, 0), dim3(grid), dim3(NW * 64), 0, stream, a); } while (0)
    switch (a.c.epi.kind) {
    case EPI_RAW: N2D2HIP_PIPE(EPI_RAW); break;
    case EPI_I24:
        if (!hi16) {
            N2D2HIP_PIPE(EPI_I24);
        } else if (valid == 1) {
            N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, 1, false, true), dim3(grid), dim3(NW * 64), 0, stream, a);
        } else if (valid == 2) {
            N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, 2, false, true), dim3(grid), dim3(NW * 64), 0, stream, a);
        } else {
            N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, 0, false, true), dim3(grid), dim3(NW * 64), 0, stream, a);
        }
        break;
    case EPI_I64: N2D2HIP_PIPE(EPI_I64); break;     // (multipliers of 24 bits and more: N2D2's 32-bit fixed point)
    default: N2D2HIP_PIPE(EPI_F32); break;
    }
#undef N2D2HIP_PIPE
}

// narrow: at most 32 output channels and the integer rescale: one 32-channel block per work-group
template <int KH>
void launch_stem(const ConvStemArgs& a, bool hi16, bool narrow, int grid, hipStream_t stream)
{
    switch (a.c.epi.kind) {
    case EPI_RAW: N2D2HIP_LAUNCH_T(conv_stem_kernel, (KH, EPI_RAW), dim3(grid), dim3(256), 0, stream, a); break;
    case EPI_I24:
        if (narrow) {
            if (hi16) N2D2HIP_LAUNCH_T(conv_stem_kernel, (KH, EPI_I24, true, false, 1), dim3(grid), dim3(256), 0, stream, a);
            else N2D2HIP_LAUNCH_T(conv_stem_kernel, (KH, EPI_I24, false, false, 1), dim3(grid), dim3(256), 0, stream, a);
        } else if (hi16) {
            N2D2HIP_LAUNCH_T(conv_stem_kernel, (KH, EPI_I24, true), dim3(grid), dim3(256), 0, stream, a);
        } else {
            N2D2HIP_LAUNCH_T(conv_stem_kernel, (KH, EPI_I24), dim3(grid), dim3(256), 0, stream, a);
        }
        break;
    default: N2D2HIP_LAUNCH_T(conv_stem_kernel, (KH, EPI_F32), dim3(grid), dim3(256), 0, stream, a); break;
    }
}

template <int NW, int BK, int NI, int NJ, int WGM, int S>
void launch_pipe_res(ConvPipeArgs a, int grid, hipStream_t stream)
{
    a.c.niter = a.c.ktot / BK;
    a.cper = a.c.in_cs / BK;
    if (a.sum16)
        N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, 1, true, true), dim3(grid), dim3(NW * 64), 0, stream, a);
    else
        N2D2HIP_LAUNCH_T(conv_pipe_kernel, (NW, BK, NI, NJ, WGM, EPI_I24, S, 1, true, false), dim3(grid), dim3(NW * 64), 0, stream, a);
}

// (multiplier, shift) with n / d == umulhi(n, multiplier) >> shift for 0 <= n < 2^31; multiplier 0 stands for d == 1
void magic_div(unsigned d, unsigned* mul, unsigned* sh)
{
    if (d <= 1) { *mul = 0; *sh = 0; return; }
    unsigned s = 0;
    while ((1ull << s) < d) ++s;
    *mul = (unsigned)((1ull << (31 + s)) / d + 1);
    *sh = s - 1;
}

int num_cus()
{
    static int n = 0;
    if (n == 0) {
        hipDeviceProp_t prop;
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            n = prop.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

int sext4(int n) { return (n & 8) ? (n | ~15) : (n & 15); }

// Reads weight element `idx` of the caller's OCHW array (int8 or nibble-packed).
int read_weight(const void* w, long long idx, int bits)
{
    if (bits == 8)
        return ((const signed char*)w)[idx];
    const unsigned char byte = ((const unsigned char*)w)[idx >> 1];
    return sext4((idx & 1) ? (byte >> 4) : (byte & 15));
}

} // namespace

extern "C" {

int n2d2hip_conv_out_dims(const n2d2hip_conv_desc* d, int H, int W, int* outH, int* outW)
{
    N2D2HIP_REQUIRE(d && outH && outW, N2D2HIP_ERR_INVALID, "conv_out_dims: null argument");
    N2D2HIP_REQUIRE(d->strideX > 0 && d->strideY > 0 && d->kW > 0 && d->kH > 0 && d->dilX > 0 && d->dilY > 0,
                    N2D2HIP_ERR_INVALID, "conv_out_dims: non-positive kernel / stride / dilation");
    *outW = conv_out_dim(W, d->kW, d->strideX, d->padL, d->padR, d->dilX);
    *outH = conv_out_dim(H, d->kH, d->strideY, d->padT, d->padB, d->dilY);
    N2D2HIP_REQUIRE(*outW > 0 && *outH > 0, N2D2HIP_ERR_INVALID, "conv_out_dims: empty output %dx%d", *outW, *outH);
    N2D2HIP_REQUIRE(d->subX >= 0 && d->subY >= 0, N2D2HIP_ERR_INVALID, "conv_out_dims: negative sub-sampling");
    // ceil(positions / subSample): the last window may hold fewer positions
    *outW = (*outW + std::max(d->subX, 1) - 1) / std::max(d->subX, 1);
    *outH = (*outH + std::max(d->subY, 1) - 1) / std::max(d->subY, 1);
    return N2D2HIP_OK;
}

// Sub-sampling: out(b, oy, ox, ch) = act(sum of the raw sums at positions (oy subY + j, ox subX + i) inside the tensor + bias)
// (ref: src/Cell/ConvCell_Frame_Kernels.cpp:135-140, then forwardBias `:151-174` and the activation).  One thread per output.
__global__ __launch_bounds__(256) void conv_subsample_kernel(const int* __restrict__ sums, int H, int W, int cs, int B, int OH, int OW, int O,
                                                             int subX, int subY, const int* __restrict__ bias, const EpiArgs epi, void* out,
                                                             int out_cs, int out_dtype)
{
    const long long total = (long long)B * OH * OW * O;
    for (long long i = blockIdx.x * 256ll + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const int ch = (int)(i % O);
        long long p = i / O;
        const int ox = (int)(p % OW);
        p /= OW;
        const int oy = (int)(p % OH);
        const int b = (int)(p / OH);
        int v = bias ? bias[ch] : 0;
        for (int y = oy * subY; y < min((oy + 1) * subY, H); ++y)
            for (int x = ox * subX; x < min((ox + 1) * subX, W); ++x)
                v += sums[(((size_t)b * H + y) * W + x) * cs + ch];
        store_value(out, (((size_t)b * OH + oy) * OW + ox) * out_cs + ch, out_dtype, epi_apply_dyn(epi, v, ch));
    }
}

static bool sub_sampled(const n2d2hip_conv_s* c) { return c && c->sub_inner != nullptr; }

static int conv_subsample_create(const n2d2hip_conv_desc* d, const void* weights, const int32_t* bias, n2d2hip_act_t act, int in_dtype,
                                 n2d2hip_conv_t* conv)
{
    n2d2hip_conv_s* c = new n2d2hip_conv_s();
    c->desc = *d;
    c->act = act;
    c->in_dtype = in_dtype;
    c->in_cs = n2d2hip_nhwc_cs(d->C);
    c->sum_other_dtype = -1;
    n2d2hip_activation raw = {};
    raw.kind = N2D2HIP_ACT_LINEAR;
    raw.scaling_mode = N2D2HIP_SCALING_NONE;
    int rc = n2d2hip_act_create(&raw, d->O, &c->sub_raw_act);
    n2d2hip_conv_desc inner = *d;
    inner.subX = inner.subY = 1;
    if (rc == N2D2HIP_OK)
        rc = n2d2hip_conv_create(&inner, weights, nullptr, c->sub_raw_act, in_dtype, &c->sub_inner);
    if (rc == N2D2HIP_OK && bias) {
        hipError_t e = hipMalloc((void**)&c->d_sub_bias, (size_t)d->O * sizeof(int));
        if (e == hipSuccess) e = hipMemcpy(c->d_sub_bias, bias, (size_t)d->O * sizeof(int), hipMemcpyHostToDevice);
        if (e != hipSuccess) rc = fail(N2D2HIP_ERR_HIP, "conv_create: copying the bias failed: %s", hipGetErrorString(e));
    }
    if (rc != N2D2HIP_OK) {
        n2d2hip_conv_destroy(c);
        return rc;
    }
    *conv = c;
    return N2D2HIP_OK;
}

static int conv_subsample_forward(n2d2hip_conv_t c, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc, H, W, OH, OW;
    if ((rc = check_tensor(in, "conv input", true)) || (rc = check_tensor(out, "conv output")))
        return rc;
    const n2d2hip_conv_desc& d = c->desc;
    if ((rc = n2d2hip_conv_out_dims(&c->sub_inner->desc, in->H, in->W, &H, &W)) || (rc = n2d2hip_conv_out_dims(&d, in->H, in->W, &OH, &OW)))
        return rc;
    N2D2HIP_REQUIRE(out->layout == N2D2HIP_NHWC && out->B == in->B && out->C == d.O && out->H == OH && out->W == OW && out->halo == 0,
                    N2D2HIP_ERR_INVALID, "conv_forward: sub-sampled output is %dx%dx%dx%d, expected %dx%dx%dx%d without a halo", out->B, out->C,
                    out->H, out->W, in->B, d.O, OH, OW);
    const n2d2hip_act_s* act = c->act;
    if (act->args.kind == EPI_RAW) {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_INVALID, "conv_forward: without a rescale the cell outputs raw sums; the output dtype must be I32");
    } else if (is_byte_type(out->dtype)) {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(act->min_out >= lo && act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "conv_forward: activation range [%d,%d] does not fit output dtype %d", act->min_out, act->max_out, out->dtype);
    } else {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: F32 outputs are produced with n2d2hip_convert");
    }
    n2d2hip_tensor sums = {};
    sums.dtype = N2D2HIP_I32; sums.layout = N2D2HIP_NHWC; sums.B = in->B; sums.C = d.O; sums.H = H; sums.W = W;
    sums.cs = n2d2hip_nhwc_cs(d.O); sums.halo = 0;
    const size_t need = n2d2hip_tensor_bytes(&sums);
    if (need > c->sub_sums_bytes) {
        // (the first forward, or a larger input than before: not a call for a caller that cannot allocate)
        N2D2HIP_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
        if (c->d_sub_sums) (void)hipFree(c->d_sub_sums);
        c->d_sub_sums = nullptr; c->sub_sums_bytes = 0;
        N2D2HIP_HIP_CHECK(hipMalloc((void**)&c->d_sub_sums, need));
        c->sub_sums_bytes = need;
    }
    sums.data = c->d_sub_sums;
    if ((rc = n2d2hip_conv_forward(c->sub_inner, in, &sums, stream)))
        return rc;
    const long long total = (long long)in->B * OH * OW * d.O;
    const unsigned grid = (unsigned)std::max<long long>(1, std::min<long long>((total + 255) / 256, 256 * 32));
    N2D2HIP_LAUNCH(conv_subsample_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const int*)c->d_sub_sums, H, W, sums.cs, in->B, OH, OW,
                   d.O, std::max(d.subX, 1), std::max(d.subY, 1), (const int*)c->d_sub_bias, act->args, out->data, out->cs, out->dtype);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_conv_create(const n2d2hip_conv_desc* d, const void* weights, const int32_t* bias, n2d2hip_act_t act,
                        int in_dtype, n2d2hip_conv_t* conv)
{
    N2D2HIP_REQUIRE(d && weights && act && conv, N2D2HIP_ERR_INVALID, "conv_create: null argument");
    N2D2HIP_REQUIRE(d->C > 0 && d->O > 0 && d->kW > 0 && d->kH > 0 && d->strideX > 0 && d->strideY > 0
                    && d->dilX > 0 && d->dilY > 0 && d->padL >= 0 && d->padT >= 0 && d->padR >= 0 && d->padB >= 0,
                    N2D2HIP_ERR_INVALID, "conv_create: bad descriptor");
    N2D2HIP_REQUIRE(d->weight_bits == 8 || d->weight_bits == 4, N2D2HIP_ERR_INVALID, "conv_create: weight_bits %d (8 or 4)", d->weight_bits);
    N2D2HIP_REQUIRE(is_byte_type(in_dtype), N2D2HIP_ERR_INVALID, "conv_create: input dtype must be U8, I8 or U8B");
    N2D2HIP_REQUIRE(in_dtype != N2D2HIP_U8, N2D2HIP_ERR_UNSUPPORTED,
                    "conv_create: plain U8 inputs cannot feed the signed matrix cores; convert to U8B first");
    N2D2HIP_REQUIRE(act->nb_channels == d->O, N2D2HIP_ERR_INVALID, "conv_create: activation built for %d channels, conv has %d outputs",
                    act->nb_channels, d->O);
    N2D2HIP_REQUIRE(d->groups >= 1, N2D2HIP_ERR_UNSUPPORTED, "conv_create: irregular mapping (nbGroups = %d)", d->groups);
    N2D2HIP_REQUIRE(d->subX >= 0 && d->subY >= 0, N2D2HIP_ERR_INVALID, "conv_create: negative sub-sampling");
    if (d->subX > 1 || d->subY > 1)
        return conv_subsample_create(d, weights, bias, act, in_dtype, conv);
    const bool depthwise = d->groups > 1 && d->groups == d->C && d->C == d->O;
    if (d->groups > 1 && !depthwise) {
        // G equal groups, output o of group o / (O/G) connected to channels [g C/G, (g+1) C/G) with its weights indexed by
        // the position among them (ConvCell_Frame_Kernels.cpp:89-96,132): the same sums as a full connection whose
        // weights outside the group are 0, which is how the matrix-core kernels run it (G times the multiplications, no
        // change to the bytes moved; the depthwise case above has its own kernel).
        N2D2HIP_REQUIRE(d->C % d->groups == 0 && d->O % d->groups == 0, N2D2HIP_ERR_INVALID,
                        "conv_create: %d groups do not divide %d channels and %d outputs", d->groups, d->C, d->O);
        const int Cg = d->C / d->groups, Og = d->O / d->groups;
        const long long taps = (long long)d->kH * d->kW, n = (long long)d->O * d->C * taps;
        std::vector<unsigned char> dense((size_t)(d->weight_bits == 8 ? n : (n + 1) / 2), 0);
        for (int o = 0; o < d->O; ++o)
            for (int cg = 0; cg < Cg; ++cg)
                for (long long t = 0; t < taps; ++t) {
                    const int v = read_weight(weights, ((long long)o * Cg + cg) * taps + t, d->weight_bits);
                    const long long at = ((long long)o * d->C + (long long)(o / Og) * Cg + cg) * taps + t;
                    if (d->weight_bits == 8) dense[(size_t)at] = (unsigned char)(signed char)v;
                    else dense[(size_t)(at >> 1)] |= (unsigned char)((v & 15) << ((at & 1) ? 4 : 0));
                }
        n2d2hip_conv_desc full = *d;
        full.groups = 1;
        return n2d2hip_conv_create(&full, dense.data(), bias, act, in_dtype, conv);
    }

    n2d2hip_conv_s* c = new n2d2hip_conv_s();
    c->desc = *d;
    c->act = act;
    c->in_dtype = in_dtype;
    c->in_cs = n2d2hip_nhwc_cs(d->C);
    c->depthwise = depthwise;
    c->pix4 = (!depthwise && c->in_cs == 4);
    c->d_w = nullptr; c->d_sub = nullptr; c->d_bias = nullptr; c->d_fill = nullptr;
    c->d_epi_tab = nullptr; c->bias_folded = false; c->hi16 = false; c->d_wstem = nullptr; c->d_ws2d = nullptr; c->d_wfrag = nullptr; c->d_wchain = nullptr; c->d_wdw = nullptr; c->d_w4img = nullptr; c->d_wsmall = nullptr;
    c->sum = nullptr; c->d_res_tab = nullptr; c->sum_other_dtype = -1; c->has_pre = c->pre_clamp = c->sum_clamp = c->sum16 = false;
    c->is_fc = false; c->fcH = c->fcW = 0;
    if (c->pix4 && d->dilX != 1) {
        delete c;
        return fail(N2D2HIP_ERR_UNSUPPORTED, "conv_create: <=4 input channels with dilationX = %d", d->dilX);
    }
    if (depthwise && d->weight_bits != 8) {
        delete c;
        return fail(N2D2HIP_ERR_UNSUPPORTED, "conv_create: depthwise with 4-bit weights");
    }
    const int zp = zero_point(in_dtype);
    const int Cg = d->C / d->groups;
    const int cs = c->in_cs;
    std::vector<signed char> hw;
    std::vector<int4> hsub;
    std::vector<int> hwdw;
    std::vector<signed char> hw4img;
    c->opad = round_up(d->O, 128);
    std::vector<int> hbias((size_t)std::max(c->opad, act->cpad), 0);
    const long long wstrideO = (long long)Cg * d->kH * d->kW;
    for (int o = 0; o < d->O; ++o) {
        long long s = 0;
        for (long long i = 0; i < wstrideO; ++i)
            s += read_weight(weights, o * wstrideO + i, d->weight_bits);
        const long long b = (bias ? (long long)bias[o] : 0) + (long long)zp * s;
        if (b < std::numeric_limits<int>::min() || b > std::numeric_limits<int>::max()) {
            delete c;
            return fail(N2D2HIP_ERR_UNSUPPORTED, "conv_create: folded bias of output %d overflows int32", o);
        }
        hbias[o] = (int)b;
    }
    // Can the rescale multiply raw accumulators?  |sum| <= 128 * sum|w| + |folded bias| for byte inputs.
    c->preclamp = act->clipped;
    std::vector<long long> acc_bound((size_t)act->cpad, 0);
    if (act->args.kind == EPI_I24 && !c->preclamp) {
        const int cp = act->cpad;
        for (int o = 0; o < d->O && !c->preclamp; ++o) {
            long long s = 0;
            for (long long i = 0; i < wstrideO; ++i)
                s += std::abs(read_weight(weights, o * wstrideO + i, d->weight_bits));
            const long long bound = 128 * s + std::llabs((long long)hbias[o]);
            acc_bound[o] = bound;
            const long long mult = act->htab[2 * (size_t)cp + o], half = act->htab[3 * (size_t)cp + o];
            if (bound >= (1ll << 23) || bound * std::llabs(mult) + std::llabs(half) > std::numeric_limits<int>::max())
                c->preclamp = true;
        }
    } else if (act->args.kind != EPI_F32) {
        c->preclamp = true;
    }
    // The pipelined kernel starts its accumulators from zero and finds the bias inside the integer rescale:
    // ((v + bias) * c + d) >> e == (v * c + (d + bias * c)) >> e in wrapping 32-bit arithmetic, the pre-clamp bounds move
    // by the bias and must stay 24-bit for the multiplier.
    std::vector<int> hepi;
    if (act->args.kind == EPI_I24) {
        const int cp = act->cpad;
        hepi.assign(7 * (size_t)cp, 0);
        c->bias_folded = true;
        c->hi16 = !c->preclamp;
        for (int ch = 0; ch < cp; ++ch) {
            const long long b = hbias[ch];
            const long long lo = (long long)act->htab[ch] - b, hi = (long long)act->htab[cp + ch] - b;
            const long long m = act->htab[2 * (size_t)cp + ch];
            if (c->preclamp && (lo <= -(1ll << 23) || hi >= (1ll << 23)))
                c->bias_folded = false;
            hepi[ch] = (int)std::max<long long>(std::min<long long>(lo, std::numeric_limits<int>::max()), std::numeric_limits<int>::min());
            hepi[cp + ch] = (int)std::max<long long>(std::min<long long>(hi, std::numeric_limits<int>::max()), std::numeric_limits<int>::min());
            hepi[2 * (size_t)cp + ch] = (int)m;
            hepi[3 * (size_t)cp + ch] = (int)(unsigned)(unsigned long long)((long long)act->htab[3 * (size_t)cp + ch] + b * m);
            hepi[4 * (size_t)cp + ch] = act->htab[4 * (size_t)cp + ch];
            // the same rescale scaled up by 2^(16 - e), if that still fits: |v| * m + half bounds the unscaled value
            const long long e16 = act->htab[4 * (size_t)cp + ch], half = act->htab[3 * (size_t)cp + ch];
            const long long up = (e16 >= 0 && e16 <= 16) ? (1ll << (16 - e16)) : 0;
            if (up == 0 || std::llabs(m) * up >= (1ll << 23)
                || (acc_bound[ch] * std::llabs(m) + std::llabs(half)) * up > std::numeric_limits<int>::max()) {
                c->hi16 = false;
            } else {
                hepi[5 * (size_t)cp + ch] = (int)(m * up);
                hepi[6 * (size_t)cp + ch] = (int)(unsigned)(unsigned long long)((half + b * m) * up);
            }
        }
    }

    if (depthwise) {
        // [tap][cs]
        hw.assign((size_t)d->kH * d->kW * cs, 0);
        for (int ch = 0; ch < d->C; ++ch)
            for (int ky = 0; ky < d->kH; ++ky)
                for (int kx = 0; kx < d->kW; ++kx)
                    hw[(size_t)(ky * d->kW + kx) * cs + ch] = (signed char)read_weight(weights, ((long long)ch * d->kH + ky) * d->kW + kx, 8);
        if (d->kH == 3 && d->kW == 3 && d->dilX == 1 && d->dilY == 1 && !(d->kernel_choice & N2D2HIP_KERNEL_NO_PIPE)) {
            std::vector<signed char> w9((size_t)d->C * 9);
            for (size_t i = 0; i < w9.size(); ++i)
                w9[i] = (signed char)read_weight(weights, (long long)i, 8);
            hwdw.resize(4 * (size_t)cs);
            depthwise3x3_weight_layout(w9.data(), hbias.data(), d->C, cs, hwdw.data());
        }
        // the general kernel adds the zero point to every loaded input, so the fold is not wanted there
        for (int o = 0; o < d->O; ++o)
            hbias[o] = bias ? bias[o] : 0;
        c->ktot = 0;
    } else {
        // sub-chunk table
        if (c->pix4) {
            for (int ky = 0; ky < d->kH; ++ky)
                for (int kx0 = 0; kx0 < d->kW; kx0 += 4)
                    hsub.push_back(int4{ky, kx0, 0, 1});
        } else {
            for (int ky = 0; ky < d->kH; ++ky)
                for (int kx = 0; kx < d->kW; ++kx)
                    for (int c0 = 0; c0 < cs; c0 += 16)
                        hsub.push_back(int4{ky, kx, c0, 1});
        }
        while (hsub.size() % 4 != 0)
            hsub.push_back(int4{0, 0, 0, 0});
        c->ktot = (int)hsub.size() * 16;
        std::vector<signed char> full((size_t)c->opad * c->ktot, 0);
        for (int o = 0; o < d->O; ++o) {
            signed char* row = full.data() + (size_t)o * c->ktot;
            for (size_t j = 0; j < hsub.size(); ++j) {
                if (!hsub[j].w) continue;
                for (int e = 0; e < 16; ++e) {
                    int ky = hsub[j].x, kx, ch;
                    if (c->pix4) { kx = hsub[j].y + e / 4; ch = e % 4; }
                    else { kx = hsub[j].y; ch = hsub[j].z + e; }
                    if (kx >= d->kW || ch >= d->C) continue;
                    row[j * 16 + e] = (signed char)read_weight(weights, (((long long)o * d->C + ch) * d->kH + ky) * d->kW + kx, d->weight_bits);
                }
            }
        }
        if (d->weight_bits == 4 && !c->pix4 && c->in_cs == d->C && d->C % 64 == 0 && c->ktot == d->kH * d->kW * d->C
            && !(d->kernel_choice & N2D2HIP_KERNEL_NO_PIPE)) {
            hw4img.resize(conv_pipe_w4_image_bytes(c->opad, c->ktot));
            conv_pipe_w4_image(full.data(), c->opad, c->ktot, hw4img.data());
        }
        if (d->weight_bits == 4) {
            // nibble-pack per 16-weight sub-chunk: byte b of dword q holds weight 8q+b (low) and 8q+4+b (high)
            hw.assign(full.size() / 2, 0);
            for (size_t s16 = 0; s16 < full.size() / 16; ++s16)
                for (int q = 0; q < 2; ++q)
                    for (int b = 0; b < 4; ++b) {
                        const int lo = full[s16 * 16 + 8 * q + b] & 15, hi = full[s16 * 16 + 8 * q + 4 + b] & 15;
                        hw[s16 * 8 + 4 * q + b] = (signed char)(lo | (hi << 4));
                    }
        } else {
            hw.swap(full);
        }
    }
    std::vector<signed char> hfrag;
    if (!depthwise && !c->pix4 && d->weight_bits == 8 && d->kW == 3 && d->kH == 3 && d->strideX == 1 && d->strideY == 1 && d->dilX == 1
        && d->dilY == 1 && d->padL == 1 && d->padT == 1 && d->padR == 1 && d->padB == 1 && c->in_cs == d->C && d->C % 64 == 0
        && d->O % 64 == 0 && c->ktot == 9 * d->C && !(d->kernel_choice & N2D2HIP_KERNEL_NO_PATCH)) {
        hfrag.resize(conv_patch_weight_bytes(d->C, d->O));
        conv_patch_weight_layout(hw.data(), d->C, d->O, hfrag.data());
    }

    hipError_t e = hipMalloc((void**)&c->d_w, hw.size());
    if (e == hipSuccess) e = hipMemcpy(c->d_w, hw.data(), hw.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void**)&c->d_bias, hbias.size() * sizeof(int));
    if (e == hipSuccess) e = hipMemcpy(c->d_bias, hbias.data(), hbias.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e == hipSuccess && c->pix4 && d->weight_bits == 8 && d->strideX == 2 && d->dilX == 1 && d->dilY == 1 && d->kW <= 8
        && (d->kH == 3 || d->kH == 5 || d->kH == 7)) {
        // [channel][kernel row][8 tap slots][4 channel slots], zero where the kernel has nothing
        const int orows = round_up(d->O, 64);
        std::vector<signed char> ws((size_t)orows * d->kH * 32, 0);
        for (int o = 0; o < d->O; ++o)
            for (int ky = 0; ky < d->kH; ++ky)
                for (int kx = 0; kx < d->kW; ++kx)
                    for (int ch = 0; ch < d->C; ++ch)
                        ws[((size_t)o * d->kH + ky) * 32 + kx * 4 + ch] =
                            (signed char)read_weight(weights, (((long long)o * d->C + ch) * d->kH + ky) * d->kW + kx, 8);
        e = hipMalloc((void**)&c->d_wstem, ws.size());
        if (e == hipSuccess) e = hipMemcpy(c->d_wstem, ws.data(), ws.size(), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && c->pix4 && d->weight_bits == 8 && d->strideX == 2 && d->strideY == 2 && d->dilX == 1 && d->dilY == 1 && d->kW == d->kH
        && (d->kH == 3 || d->kH == 5 || d->kH == 7) && d->O <= 64 && !(d->kernel_choice & N2D2HIP_KERNEL_NO_STEM)) {
        std::vector<signed char> ochw((size_t)d->O * d->C * d->kH * d->kW), ws(conv_s2d_weight_bytes(d->O, d->kH, d->padT));
        for (size_t i = 0; i < ochw.size(); ++i)
            ochw[i] = (signed char)read_weight(weights, (long long)i, 8);
        conv_s2d_weight_layout(ochw.data(), d->C, d->O, d->kH, d->padT, d->padL, ws.data());
        e = hipMalloc((void**)&c->d_ws2d, ws.size());
        if (e == hipSuccess) e = hipMemcpy(c->d_ws2d, ws.data(), ws.size(), hipMemcpyHostToDevice);
    }
    // (a dilated kernel with padding keeps the kernel that follows the reference's window arithmetic tap by tap: what the
    // reference skips at the borders is then not what zero padding would skip)
    if (e == hipSuccess && !depthwise && d->weight_bits == 8 && d->kW <= 8 && conv_small_rows(d->C, d->O, d->kW * d->kH)
        && ((d->dilX == 1 && d->dilY == 1) || (d->padL == 0 && d->padT == 0 && d->padR == 0 && d->padB == 0))
        && !(d->kernel_choice & N2D2HIP_KERNEL_NO_DIRECT)) {
        const int taps = d->kW * d->kH;
        std::vector<signed char> ohwc((size_t)d->O * taps * d->C), img(conv_small_weight_bytes(d->C, d->O, taps));
        for (int o = 0; o < d->O; ++o)
            for (int ch = 0; ch < d->C; ++ch)
                for (int t = 0; t < taps; ++t)
                    ohwc[((size_t)o * taps + t) * d->C + ch] = (signed char)read_weight(weights, ((long long)o * d->C + ch) * taps + t, 8);
        conv_small_weight_layout(ohwc.data(), d->C, d->O, taps, img.data());
        e = hipMalloc((void**)&c->d_wsmall, img.size());
        if (e == hipSuccess) e = hipMemcpy(c->d_wsmall, img.data(), img.size(), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !hfrag.empty()) {
        e = hipMalloc((void**)&c->d_wfrag, hfrag.size());
        if (e == hipSuccess) e = hipMemcpy(c->d_wfrag, hfrag.data(), hfrag.size(), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !depthwise && !c->pix4 && d->weight_bits == 8 && d->kW == 1 && d->kH == 1 && conv_chain_channels(d->C)
        && c->in_cs == d->C && d->O == 4 * d->C && c->ktot == d->C) {
        std::vector<signed char> img(conv_chain_weight_bytes(d->C, d->O));
        conv_chain_weight_layout(hw.data(), c->ktot, d->C, d->O, img.data());
        e = hipMalloc((void**)&c->d_wchain, img.size());
        if (e == hipSuccess) e = hipMemcpy(c->d_wchain, img.data(), img.size(), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !hw4img.empty()) {
        e = hipMalloc((void**)&c->d_w4img, hw4img.size());
        if (e == hipSuccess) e = hipMemcpy(c->d_w4img, hw4img.data(), hw4img.size(), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !hwdw.empty()) {
        e = hipMalloc((void**)&c->d_wdw, hwdw.size() * sizeof(int));
        if (e == hipSuccess) e = hipMemcpy(c->d_wdw, hwdw.data(), hwdw.size() * sizeof(int), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !hepi.empty()) {
        e = hipMalloc((void**)&c->d_epi_tab, hepi.size() * sizeof(int));
        if (e == hipSuccess) e = hipMemcpy(c->d_epi_tab, hepi.data(), hepi.size() * sizeof(int), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !hsub.empty()) {
        e = hipMalloc((void**)&c->d_sub, hsub.size() * sizeof(int4));
        if (e == hipSuccess) e = hipMemcpy(c->d_sub, hsub.data(), hsub.size() * sizeof(int4), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess) {
        signed char fill[16];
        memset(fill, zp ? 0x80 : 0x00, sizeof(fill));
        e = hipMalloc((void**)&c->d_fill, sizeof(fill));
        if (e == hipSuccess) e = hipMemcpy(c->d_fill, fill, sizeof(fill), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
        n2d2hip_conv_destroy(c);
        return fail(N2D2HIP_ERR_HIP, "conv_create: device upload failed: %s", hipGetErrorString(e));
    }
    *conv = c;
    return N2D2HIP_OK;
}

int n2d2hip_conv_destroy(n2d2hip_conv_t c)
{
    if (!c) return N2D2HIP_OK;
    if (c->sub_inner) n2d2hip_conv_destroy(c->sub_inner);
    if (c->sub_raw_act) n2d2hip_act_destroy(c->sub_raw_act);
    if (c->d_sub_bias) (void)hipFree(c->d_sub_bias);
    if (c->d_sub_sums) (void)hipFree(c->d_sub_sums);
    if (c->d_w) (void)hipFree(c->d_w);
    if (c->d_sub) (void)hipFree(c->d_sub);
    if (c->d_bias) (void)hipFree(c->d_bias);
    if (c->d_fill) (void)hipFree(c->d_fill);
    if (c->d_res_tab) (void)hipFree(c->d_res_tab);
    if (c->d_epi_tab) (void)hipFree(c->d_epi_tab);
    if (c->d_wstem) (void)hipFree(c->d_wstem);
    if (c->d_ws2d) (void)hipFree(c->d_ws2d);
    if (c->d_wsmall) (void)hipFree(c->d_wsmall);
    if (c->d_wfrag) (void)hipFree(c->d_wfrag);
    if (c->d_wchain) (void)hipFree(c->d_wchain);
    if (c->d_wdw) (void)hipFree(c->d_wdw);
    if (c->d_w4img) (void)hipFree(c->d_w4img);
    delete c;
    return N2D2HIP_OK;
}

// Can this convolution run on the pipelined kernel, and with which channel tile?
// What the pipelined kernel asks of a convolution's shape (its rescale is the cell's business, below)
static bool pipe_shape(const n2d2hip_conv_desc& d)
{
    const bool depthwise = d.groups > 1 && d.groups == d.C && d.C == d.O;       // (other groups run as a full connection)
    return d.O > 4              // (a pixel of at most 4 outputs is one dword: the general kernel stores those)
        && !depthwise && (d.weight_bits == 4 || d.weight_bits == 8) && d.C % 64 == 0 && d.kW * d.kH <= 31;
}

static bool pipe_eligible(const n2d2hip_conv_s* c, bool* bn128)
{
    const n2d2hip_conv_desc& d = c->desc;
    const int opad_n = round_up(d.O, 64);
    *bn128 = opad_n % 128 == 0 || opad_n > 256;
    const int k = c->act->args.kind;
    if (!pipe_shape(d) || c->sub_inner)     // (a sub-sampled cell's own handle launches nothing but the window sums)
        return false;
    if (d.weight_bits == 4)     // packed weights: integer rescale only
        return c->d_w4img != nullptr && k == EPI_I24 && c->bias_folded;
    return !c->depthwise && !c->pix4 && c->in_cs == d.C && (k == EPI_RAW || (k == EPI_I24 && c->bias_folded) || k == EPI_F32 || k == EPI_I64);
}

// Is this convolution served by the space-to-depth first-layer kernel on an H x W input?  Returns the border it needs, or -1.
static int s2d_halo(const n2d2hip_conv_s* c, int H, int W)
{
    const n2d2hip_conv_desc& d = c->desc;
    if (!c->d_ws2d || c->act->args.kind != EPI_I24 || !c->bias_folded || c->act->min_out < -128 || c->act->max_out > 255)
        return -1;
    const int halo = conv_s2d_halo(d.kH, d.padT, d.padL, d.padB, d.padR, H, W);
    // a tile is at least one row of the bordered image and at most 256 positions
    if (halo < 0 || halo > 16 || (W + 1) / 2 + 2 * halo > 128)
        return -1;
    return halo;
}

// The first-layer kernel on a space-to-depth input; `pd` non-null: with the 3x3 stride-2 max pooling behind it (`out` is the
// pooled tensor).  Shapes of `out` have been checked by the caller.
static int conv_s2d_forward(n2d2hip_conv_t c, const n2d2hip_tensor* in, const n2d2hip_tensor* out, const n2d2hip_pool_desc* pd,
                            int OH, int OW, int POH, int POW, hipStream_t stream)
{
    const n2d2hip_conv_desc& d = c->desc;
    const int need = s2d_halo(c, in->H, in->W);
    N2D2HIP_REQUIRE(need >= 0, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: this convolution does not read space-to-depth inputs (n2d2hip_conv_s2d_halo)");
    N2D2HIP_REQUIRE(in->halo >= need, N2D2HIP_ERR_INVALID, "conv_forward: the space-to-depth input has a border of %d, the convolution needs %d",
                    in->halo, need);
    N2D2HIP_REQUIRE(in->dtype == c->in_dtype && in->C == d.C, N2D2HIP_ERR_INVALID, "conv_forward: input has %d channels of type %d, conv expects %d of type %d",
                    in->C, in->dtype, d.C, c->in_dtype);
    ConvS2dArgs a = {};
    a.in = (const signed char*)in->data;
    a.Hp = (in->H + 1) / 2 + 2 * in->halo;
    a.Wp = (in->W + 1) / 2 + 2 * in->halo;
    N2D2HIP_REQUIRE(a.Wp <= 128 && (long long)in->B * a.Hp * a.Wp * 16 < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED,
                    "conv_forward: space-to-depth input too wide or too large");
    a.total = in->B * a.Hp * a.Wp;
    a.wk = c->d_ws2d;
    a.ty = in->halo - (d.padT + 1) / 2;
    a.tx = in->halo - (d.padL + 1) / 2;
    a.OH = OH; a.OW = OW;
    magic_div((unsigned)a.Wp, &a.wp_mul, &a.wp_sh);
    a.out = out->data; a.out_cs = out->cs;
    N2D2HIP_REQUIRE(n2d2hip_tensor_bytes(out) < (1ull << 31), N2D2HIP_ERR_UNSUPPORTED, "conv_forward: output too large for the first-layer kernel");
    a.out_bytes = (int)n2d2hip_tensor_bytes(out);
    a.out_xor = out->dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    const int cp = c->act->cpad;
    const bool hi16 = c->hi16 && !(d.kernel_choice & N2D2HIP_KERNEL_NO_HI16);
    a.ta = c->d_epi_tab; a.tb = c->d_epi_tab + cp; a.tc = c->d_epi_tab + (hi16 ? 5 : 2) * cp;
    a.td = c->d_epi_tab + (hi16 ? 6 : 3) * cp; a.te = c->d_epi_tab + 4 * cp;
    a.lo = c->act->args.lo; a.hi = c->act->args.hi; a.preclamp = c->preclamp ? 1 : 0;
    const int ny = (d.kH + 1) / 2, nxh = (ny + 1) / 2;
    const int slots = 2 * num_cus();
    if (pd) {
        N2D2HIP_REQUIRE(hi16 && POW <= 62 && round_up(d.O, 16) == 64, N2D2HIP_ERR_UNSUPPORTED,
                        "conv_forward_maxpool: the pooled first-layer kernel needs scaled-up tables, 49 to 64 outputs and at most 62 pooled columns");
        a.TR = 2;
        a.pool_pad = pd->padX; a.POH = POH; a.POW = POW;
        a.pool_halo = out->halo; a.POHp = POH + 2 * out->halo; a.POWp = POW + 2 * out->halo;
        // strips of pooled rows: one per block slot if the batch has that many rows, never shorter than 4 rows (each
        // strip computes one or two convolution rows more than it needs)
        int rows = std::max(1, (int)(((long long)in->B * POH + slots - 1) / slots));
        rows = std::min(std::max(rows, std::min(POH, 4)), POH);
        a.rows_per_strip = rows;
        a.strips_per_image = (POH + rows - 1) / rows;
    } else {
        a.TR = std::max(1, std::min(256 / a.Wp, OH));
        int rows = std::max(a.TR, (int)(((long long)in->B * OH + slots - 1) / slots));
        rows = std::min(round_up(rows, a.TR), round_up(OH, a.TR));
        a.rows_per_strip = rows;
        a.strips_per_image = (OH + rows - 1) / rows;
    }
    a.T = a.TR * a.Wp;
    a.NT = (a.T + 31) / 32;
    // positions a tile's window reaches past its first one (the last 32-position tile in full, the last window row and
    // pixel pair, the upper lane half's + 1), and one more tile: what must be in the ring before a strip's first tile
    const int window = a.NT * 32 + (ny - 1) * a.Wp + 2 * nxh + 1;
    a.PF = round_up(window + a.T, 64);
    N2D2HIP_REQUIRE(a.T <= 256 && a.PF + a.T + 64 < 2048, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: space-to-depth rows too long");
    a.nstrips = in->B * a.strips_per_image;
    const int blocks = std::max(1, std::min(a.nstrips, slots));
    const int o16 = round_up(d.O, 16);
    return conv_s2d_launch(a, d.kH, hi16, pd != nullptr, o16 <= 32 ? 1 : 2, blocks, 1, stream);
}

static int conv_forward_impl(n2d2hip_conv_t c, const n2d2hip_tensor* in, const n2d2hip_tensor* other, const n2d2hip_tensor* out,
                             n2d2hip_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    int rc;
    N2D2HIP_REQUIRE(c != nullptr, N2D2HIP_ERR_INVALID, "conv_forward: null conv");
    if ((rc = check_tensor(in, "conv input", true, true)) || (rc = check_tensor(out, "conv output", true)))
        return rc;
    const n2d2hip_conv_desc& d = c->desc;
    if (in->layout == N2D2HIP_S2D) {
        int OH, OW;
        if ((rc = n2d2hip_conv_out_dims(&d, in->H, in->W, &OH, &OW)))
            return rc;
        N2D2HIP_REQUIRE(!other && out->halo == 0 && out->layout == N2D2HIP_NHWC && is_byte_type(out->dtype) && out->cs % 16 == 0,
                        N2D2HIP_ERR_UNSUPPORTED, "conv_forward: a space-to-depth input goes to a plain NHWC byte output");
        N2D2HIP_REQUIRE(out->B == in->B && out->C == d.O && out->H == OH && out->W == OW, N2D2HIP_ERR_INVALID,
                        "conv_forward: output is %dx%dx%dx%d, expected %dx%dx%dx%d", out->B, out->C, out->H, out->W, in->B, d.O, OH, OW);
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(c->act->min_out >= lo && c->act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "conv_forward: activation range [%d,%d] does not fit output dtype %d", c->act->min_out, c->act->max_out, out->dtype);
        return conv_s2d_forward(c, in, out, nullptr, OH, OW, 0, 0, (hipStream_t)stream_);
    }
    bool bn128_unused;
    N2D2HIP_REQUIRE((in->halo == 0 && out->halo == 0)
                        || (pipe_eligible(c, &bn128_unused) && !(d.kernel_choice & N2D2HIP_KERNEL_NO_PIPE) && d.dilX == 1 && d.dilY == 1),
                    N2D2HIP_ERR_UNSUPPORTED, "conv_forward: this convolution does not take tensors with a halo (n2d2hip_conv_accepts_halo)");
    N2D2HIP_REQUIRE(in->layout == N2D2HIP_NHWC && out->layout == N2D2HIP_NHWC, N2D2HIP_ERR_UNSUPPORTED,
                    "conv_forward: tensors must be NHWC (use n2d2hip_convert at graph edges)");
    N2D2HIP_REQUIRE(in->dtype == c->in_dtype, N2D2HIP_ERR_INVALID, "conv_forward: input dtype %d, conv created for %d", in->dtype, c->in_dtype);
    N2D2HIP_REQUIRE(in->C == d.C && in->cs == c->in_cs, N2D2HIP_ERR_INVALID,
                    "conv_forward: input has %d channels (stride %d), conv expects %d (stride %d)", in->C, in->cs, d.C, c->in_cs);
    int OH, OW;
    if ((rc = n2d2hip_conv_out_dims(&d, in->H, in->W, &OH, &OW)))
        return rc;
    N2D2HIP_REQUIRE(out->B == in->B && out->C == d.O && out->H == OH && out->W == OW, N2D2HIP_ERR_INVALID,
                    "conv_forward: output is %dx%dx%dx%d, expected %dx%dx%dx%d", out->B, out->C, out->H, out->W, in->B, d.O, OH, OW);
    N2D2HIP_REQUIRE(out->cs % 16 == 0 || out->cs == 4, N2D2HIP_ERR_INVALID,
                    "conv_forward: output channel stride %d must be a multiple of 16 (or 4 for at most 4 outputs)", out->cs);
    // with a folded sum the stored values are the sum cell's
    const n2d2hip_act_s* act = other ? c->sum->act : c->act;
    if (other) {
        if ((rc = check_tensor(other, "sum input", true)))
            return rc;
        N2D2HIP_REQUIRE(other->layout == N2D2HIP_NHWC && other->dtype == c->sum_other_dtype && other->B == out->B && other->C == out->C
                        && other->H == out->H && other->W == out->W && other->cs % 16 == 0 && other->cs >= round_up(d.O, 16),
                        N2D2HIP_ERR_INVALID, "conv_forward_sum: the other input must be an NHWC tensor of the output's shape and of the "
                        "storage type given to n2d2hip_conv_fuse_sum");
    }
    if (act->args.kind == EPI_RAW) {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_INVALID,
                        "conv_forward: without a rescale the cell outputs raw sums; the output dtype must be I32");
    } else if (is_byte_type(out->dtype)) {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(act->min_out >= lo && act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "conv_forward: activation range [%d,%d] does not fit output dtype %d", act->min_out, act->max_out, out->dtype);
    } else {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: F32 outputs are produced with n2d2hip_convert");
    }
    const long long Mll = (long long)in->B * OH * OW;
    // An input with a halo is a larger input with less padding: the kernels see its physical size
    const int Hp = in->H + 2 * in->halo, Wp = in->W + 2 * in->halo;
    const int padL = d.padL - in->halo, padT = d.padT - in->halo, padR = d.padR - in->halo, padB = d.padB - in->halo;
    const long long out_pixels = (long long)in->B * (OH + 2 * out->halo) * (OW + 2 * out->halo);
    N2D2HIP_REQUIRE(Mll < (1ll << 31) && out_pixels < (1ll << 31) && (long long)in->B * Hp * Wp * in->cs < (1ll << 40),
                    N2D2HIP_ERR_UNSUPPORTED, "conv_forward: tensor too large");
    const unsigned out_xor = out->dtype == N2D2HIP_U8B ? 0x80808080u : 0u;

    if (c->depthwise) {
        N2D2HIP_REQUIRE(out->cs == in->cs, N2D2HIP_ERR_INVALID, "conv_forward: depthwise needs equal channel strides");
        N2D2HIP_REQUIRE(in->halo == 0 && out->halo == 0, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: depthwise tensors carry no border");
        if (c->d_wdw && in->cs % 16 == 0 && d.strideX == d.strideY && (d.strideX == 1 || d.strideX == 2) && is_byte_type(out->dtype)
            && c->act->cpad >= in->cs) {
            DepthwiseArgs q;
            q.in = (const signed char*)in->data; q.out = out->data; q.wb = c->d_wdw;
            q.cs = in->cs; q.B = in->B; q.H = in->H; q.W = in->W; q.OH = OH; q.OW = OW; q.padL = d.padL; q.padT = d.padT;
            q.fill = zero_point(in->dtype) ? 0x80808080u : 0u;
            q.out_xor = out_xor;
            q.epi = c->act->args;
            // rescale with the bias folded in, when no clamp has to come before the multiply and the result saturates to
            // [0, 255]: the kernel then starts from zero and saturates while it packs
            q.fast = c->bias_folded && c->d_epi_tab && !c->preclamp && q.epi.kind == EPI_I24 && q.epi.lo == 0 && q.epi.hi == 255;
            q.fc = q.fast ? c->d_epi_tab + 2 * c->act->cpad : nullptr;
            q.fd = q.fast ? c->d_epi_tab + 3 * c->act->cpad : nullptr;
            q.fe = q.fast ? c->d_epi_tab + 4 * c->act->cpad : nullptr;
            return depthwise3x3_launch(q, d.strideX, num_cus(), stream);
        }
        const long long total = Mll * (in->cs / 4);
        const unsigned grid = (unsigned)std::min<long long>((total + 255) / 256, 256 * 64);
        N2D2HIP_LAUNCH(depthwise_kernel, dim3(grid), dim3(256), 0, stream, (const signed char*)in->data, in->cs, in->B, in->H,
                           in->W, OH, OW, c->d_w, d.kH, d.kW, c->d_bias, out->data, out->dtype, d.strideX, d.strideY, d.padL,
                           d.padT, d.dilX, d.dilY, zero_point(in->dtype), out_xor, c->act->args);
        N2D2HIP_HIP_CHECK(hipGetLastError());
        return N2D2HIP_OK;
    }

    ConvArgs a;
    a.in = (const signed char*)in->data;
    a.in_cs = in->cs; a.B = in->B; a.H = Hp; a.W = Wp;
    a.OH = OH; a.OW = OW; a.M = (int)Mll;
    a.w = c->d_w; a.ktot = c->ktot; a.niter = c->ktot / 64; a.sub = c->d_sub; a.bias = c->d_bias;
    a.out = out->data; a.out_cs = out->cs; a.out_dtype = out->dtype;
    a.strideX = d.strideX; a.strideY = d.strideY; a.padL = padL; a.padT = padT; a.dilX = d.dilX; a.dilY = d.dilY;
    a.kW = d.kW; a.kH = d.kH;
    a.fill = zero_point(in->dtype) ? 0x80808080u : 0u;
    a.out_xor = out_xor;
    a.epi = c->act->args;

    // Tile choice: 128 channels per block when the layer has them, and 64-pixel
    // tiles when 128-pixel tiles would leave most of the 256 CUs idle.
    const bool w4 = d.weight_bits == 4;
    const int opad_n = round_up(d.O, 64);
    const bool bn128 = opad_n % 128 == 0 || opad_n > 256;
    const int BN = bn128 ? 128 : 64;
    a.ntiles_n = (round_up(d.O, 16) + BN - 1) / BN;
    const long long blocks128 = ((Mll + 127) / 128) * a.ntiles_n;
    const bool bm64 = bn128 && !c->pix4 && blocks128 < 512;
    const int BM = bm64 ? 64 : 128;
    a.nblocks = (int)(((Mll + BM - 1) / BM) * a.ntiles_n);
    const bool fits32 = (long long)in->B * Hp * Wp * in->cs < (1ll << 31) && (long long)c->opad * c->ktot < (1ll << 31);
    const bool pipe = pipe_eligible(c, &bn128_unused) && fits32;
    N2D2HIP_REQUIRE(!other || (pipe && out_pixels * out->cs < (1ll << 31)), N2D2HIP_ERR_UNSUPPORTED,
                    "conv_forward_sum: tensor too large for the fused kernel");
    N2D2HIP_REQUIRE((in->halo == 0 && out->halo == 0) || pipe, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: tensor with a halo too large");
    if (pipe && !other && c->d_wfrag && in->halo == 1 && c->act->args.kind == EPI_I24 && c->bias_folded && is_byte_type(out->dtype)
        && conv_patch_eligible(d.C, d.O, Wp) && out_pixels * out->cs < (1ll << 31) && !(d.kernel_choice & N2D2HIP_KERNEL_NO_PIPE)
        // where it is the faster of the two (measured): images large enough that the border positions it computes and drops
        // stay under a third of the work
        // ... and enough tiles (of 128 positions, the kernel's smaller form) to give every CU a block
        && ((d.kernel_choice & N2D2HIP_KERNEL_PATCH)
            || ((long long)Hp * Wp * 100 <= (long long)in->H * in->W * 135
                && (((long long)in->B * Hp * Wp + 127) / 128) * (d.O / (d.O % 128 == 0 ? 128 : 64)) >= num_cus()))) {
        // 3x3, stride 1, on an input that carries its padding: nine shifted reads of one patch of pixels
        ConvPatchArgs q = {};
        q.in = a.in; q.wfrag = c->d_wfrag; q.out = out->data;
        q.C = d.C; q.O = d.O; q.Hp = Hp; q.Wp = Wp; q.total = in->B * Hp * Wp;
        q.out_cs = out->cs; q.out_halo = out->halo; q.OHp = OH + 2 * out->halo; q.OWp = OW + 2 * out->halo;
        q.out_xor = out_xor;
        magic_div((unsigned)(Hp * Wp), &q.img_mul, &q.img_sh);
        magic_div((unsigned)Wp, &q.row_mul, &q.row_sh);
        const int cp = c->act->cpad;
        const bool hi16 = c->hi16 && !(d.kernel_choice & N2D2HIP_KERNEL_NO_HI16);
        q.ta = c->d_epi_tab; q.tb = c->d_epi_tab + cp; q.tc = c->d_epi_tab + (hi16 ? 5 : 2) * cp;
        q.td = c->d_epi_tab + (hi16 ? 6 : 3) * cp; q.te = c->d_epi_tab + 4 * cp;
        q.lo = c->act->args.lo; q.hi = c->act->args.hi; q.preclamp = c->preclamp ? 1 : 0;
        const int tile_m = (d.kernel_choice & N2D2HIP_KERNEL_TILE_M256) ? 256 : ((d.kernel_choice & N2D2HIP_KERNEL_TILE_M128) ? 128
            : ((d.kernel_choice & N2D2HIP_KERNEL_TILE_M64) ? 64 : 0));
        return conv_patch_launch(q, hi16, num_cus(), tile_m, stream);
    }
    if (pipe && (other || !(d.kernel_choice & N2D2HIP_KERNEL_NO_PIPE))) {
        // persistent pipelined kernel: 2 blocks per CU, each walking pixel tiles of one channel tile
        ConvPipeArgs q;
        q.c = a;
        q.fill16 = c->d_fill;
        q.cper = d.C / 64;
        q.kW = d.kW; q.kH = d.kH;
        q.preclamp = c->preclamp ? 1 : 0;
        if (c->act->args.kind == EPI_I24) {
            const int cp = c->act->cpad;
            q.c.epi.a = c->d_epi_tab; q.c.epi.b = c->d_epi_tab + cp; q.c.epi.c = c->d_epi_tab + 2 * cp;
            q.c.epi.d = c->d_epi_tab + 3 * cp; q.c.epi.e = c->d_epi_tab + 4 * cp;
        }
#ifdef N2D2HIP_PROFILE
        q.prof = nullptr;      // probe builds: launch_kernel() points it at this launch's records
#endif
        magic_div((unsigned)(OH * OW), &q.ohw_mul, &q.ohw_sh);
        magic_div((unsigned)OW, &q.ow_mul, &q.ow_sh);
        // no padding: every tap of every window reads inside the input (also a dilated kernel's, whose hand-unrolled
        // special case in the reference needs a window cut to 3 taps by the input's edge, which cannot happen then)
        const int all_valid = (padL <= 0 && padT <= 0 && padR <= 0 && padB <= 0) ? (d.kW * d.kH > 1 ? 2 : 1) : 0;
        q.out_halo = out->halo;
        q.out_pixels = (int)out_pixels;
        // Two independent 4-wave blocks per CU, 128 pixels x 128 (or 64) channels each: one block's epilogue and
        // barrier waits overlap the other's MFMAs.  K advances by whole 128-byte lines when the channel count allows.
        // Layers with few pixels (deep stages) take 64-pixel tiles so that every CU still gets its two blocks.
        const long long tiles128 = ((Mll + 127) / 128) * a.ntiles_n;
        const bool small_m = bn128 && (w4 || d.C % 128 == 0)
            && ((d.kernel_choice & (N2D2HIP_KERNEL_TILE_M64 | N2D2HIP_KERNEL_TILE_M128)) ? (d.kernel_choice & N2D2HIP_KERNEL_TILE_M64) != 0
                                                                                            : tiles128 < (3 * num_cus()) / 2);
        // 64-channel layers whose K advances in 64-byte steps take 256-pixel tiles: twice the MFMAs per ring stage
        const bool wide64 = !w4 && !bn128 && !other && d.C % 128 != 0 && Mll >= 256ll * 4 * num_cus();
        // A handful of tiles (the classifier's FC): 64 x 64 tiles, four times as many blocks share the long K
        const bool tiny = !w4 && small_m && !other && ((Mll + 63) / 64) * a.ntiles_n * 8 < num_cus();
        if (tiny) a.ntiles_n = (round_up(d.O, 16) + 63) / 64;
        const int BMp = small_m ? 64 : wide64 ? 256 : 128;
        q.mtiles = (int)((Mll + BMp - 1) / BMp);
        const int per_xcd = std::max(1, std::min((q.mtiles + 7) / 8, 2 * num_cus() / (8 * a.ntiles_n)));
        q.mlanes = per_xcd;
        q.xcd_tiles = (q.mtiles + 7) / 8;
        const int grid = 8 * a.ntiles_n * per_xcd;
        q.res = nullptr; q.res_cs = 0; q.res_halo = 0; q.res_flip = 0; q.has_pre = q.pre_clamp = q.sum_clamp = 0;
        q.sum16 = nullptr; q.sum16_stride = 0; q.pre_in_range = 0;
        q.sum = EpiArgs(); q.pre = EpiArgs();
        // Byte outputs of an integer rescale whose scaled-up tables fit: the rescaled value is read from the upper half of
        // the multiply-add's result
        const bool hi16 = !other && c->hi16 && c->act->args.kind == EPI_I24 && is_byte_type(out->dtype) && !(d.kernel_choice & N2D2HIP_KERNEL_NO_HI16);
        if (hi16) { q.c.epi.c = c->d_epi_tab + 5 * c->act->cpad; q.c.epi.d = c->d_epi_tab + 6 * c->act->cpad; }
        if (w4 && !other) {
            // 4-bit weights, packed in memory and in LDS
            q.c.w = c->d_w4img;
            return conv_pipe_w4_launch(q, small_m ? 2 : bn128 ? 1 : 0, all_valid, hi16, grid, stream);
        }
        if (other) {
            const int cp = c->sum->act->cpad;
            q.res = (const signed char*)other->data;
            q.res_cs = other->cs;
            q.res_halo = other->halo;
            q.res_flip = other->dtype == N2D2HIP_U8 ? 0u : 0x80808080u;
            q.sum16 = c->sum16 ? c->d_res_tab + 10 * cp : nullptr;
            q.sum16_stride = cp / 2;
            q.pre_in_range = c->pre_in_range ? 1 : 0;
            q.sum = c->sum->act->args;
            q.sum.a = c->d_res_tab; q.sum.b = c->d_res_tab + cp; q.sum.c = c->d_res_tab + 2 * cp;
            q.sum.d = c->d_res_tab + 3 * cp; q.sum.e = c->d_res_tab + 4 * cp;
            q.has_pre = c->has_pre; q.pre_clamp = c->pre_clamp; q.sum_clamp = c->sum_clamp;
            if (c->has_pre) {
                q.pre = c->sum->pre_act->args;
                q.pre.a = c->d_res_tab + 5 * cp; q.pre.b = c->d_res_tab + 6 * cp; q.pre.c = c->d_res_tab + 7 * cp;
                q.pre.d = c->d_res_tab + 8 * cp; q.pre.e = c->d_res_tab + 9 * cp;
                if (c->sum16) { q.pre.c = c->d_res_tab + 12 * cp; q.pre.d = c->d_res_tab + 13 * cp; }
            }
            if (c->sum16) { q.c.epi.c = c->d_epi_tab + 5 * c->act->cpad; q.c.epi.d = c->d_epi_tab + 6 * c->act->cpad; }
            if (w4) {
                q.c.w = c->d_w4img;
                return conv_pipe_w4_launch(q, small_m ? 2 : bn128 ? 1 : 0, all_valid, false, grid, stream);
            }
            if (small_m) {
                launch_pipe_res<4, 128, 2, 1, 2, 3>(q, grid, stream);
            } else if (d.C % 128 == 0) {
                if (bn128) launch_pipe_res<4, 128, 2, 2, 2, 2>(q, grid, stream);
                else launch_pipe_res<4, 128, 2, 1, 4, 3>(q, grid, stream);
            } else {
                if (bn128) launch_pipe_res<4, 64, 2, 2, 2, 4>(q, grid, stream);
                else launch_pipe_res<4, 64, 2, 1, 4, 4>(q, grid, stream);
            }
        } else if (wide64) {
            launch_pipe<4, 64, 2, 2, 4, 3>(q, all_valid, hi16, grid, stream);
        } else if (tiny) {
            q.c.ntiles_n = a.ntiles_n;
            launch_pipe<4, 128, 1, 1, 2, 3>(q, all_valid, hi16, grid, stream);
        } else if (small_m) {
            launch_pipe<4, 128, 2, 1, 2, 3>(q, all_valid, hi16, grid, stream);
        } else if (d.C % 128 == 0) {
            if (bn128) launch_pipe<4, 128, 2, 2, 2, 2>(q, all_valid, hi16, grid, stream);
            else launch_pipe<4, 128, 2, 1, 4, 3>(q, all_valid, hi16, grid, stream);
        } else {
            if (bn128) launch_pipe<4, 64, 2, 2, 2, 4>(q, all_valid, hi16, grid, stream);
            else launch_pipe<4, 64, 2, 1, 4, 4>(q, all_valid, hi16, grid, stream);
        }
        N2D2HIP_HIP_CHECK(hipGetLastError());
        return N2D2HIP_OK;
    }
    {
        const int k = c->act->args.kind;
        if (c->d_wstem && out->cs % 16 == 0 && !other && (k == EPI_RAW || (k == EPI_I24 && c->bias_folded) || k == EPI_F32) && fits32
            && !(d.kernel_choice & N2D2HIP_KERNEL_NO_STEM)) {
            ConvStemArgs q;
            q.c = a;
            if (k == EPI_I24) {
                const int cp = c->act->cpad;
                q.c.epi.a = c->d_epi_tab; q.c.epi.b = c->d_epi_tab + cp; q.c.epi.c = c->d_epi_tab + 2 * cp;
                q.c.epi.d = c->d_epi_tab + 3 * cp; q.c.epi.e = c->d_epi_tab + 4 * cp;
            }
            q.wk = c->d_wstem;
            q.fill16 = c->d_fill;
            q.preclamp = c->preclamp ? 1 : 0;
            q.tiles_per_row = (OW + 127) / 128;
            q.ntiles = in->B * OH * q.tiles_per_row;
            const bool narrow = k == EPI_I24 && round_up(d.O, 16) <= 32;
            q.c.ntiles_n = narrow ? 1 : (round_up(d.O, 16) + 63) / 64;
            q.nlanes = std::max(1, std::min((q.ntiles + 7) / 8, (3 * num_cus()) / (8 * q.c.ntiles_n)));
            q.xcd_tiles = (q.ntiles + 7) / 8;
            magic_div((unsigned)OH, &q.oh_mul, &q.oh_sh);
            magic_div((unsigned)q.tiles_per_row, &q.tpr_mul, &q.tpr_sh);
            const int grid = 8 * q.nlanes * q.c.ntiles_n;
            const bool hi16 = k == EPI_I24 && c->hi16 && is_byte_type(out->dtype) && !(d.kernel_choice & N2D2HIP_KERNEL_NO_HI16);
            if (hi16) { q.c.epi.c = c->d_epi_tab + 5 * c->act->cpad; q.c.epi.d = c->d_epi_tab + 6 * c->act->cpad; }
            if (d.kH == 3) launch_stem<3>(q, hi16, narrow, grid, stream);
            else if (d.kH == 5) launch_stem<5>(q, hi16, narrow, grid, stream);
            else launch_stem<7>(q, hi16, narrow, grid, stream);
            N2D2HIP_HIP_CHECK(hipGetLastError());
            return N2D2HIP_OK;
        }
    }
    if (c->d_wsmall && !other && !c->is_fc && in->halo == 0 && out->halo == 0 && is_byte_type(out->dtype)
        && c->act->args.kind != EPI_RAW && (c->pix4 || (d.kernel_choice & N2D2HIP_KERNEL_DIRECT))) {
        // A handful of channels: one thread per output pixel.  Taken by itself for at most 4 input channels, where the
        // matrix-core kernel spends its K steps on padding (LeNet's first layer: 29 -> 21 us); with more channels the two
        // are on a par or the matrix cores ahead (LeNet's second layer: 16 against 20 us).
        ConvSmallArgs q;
        q.in = (const signed char*)in->data; q.in_cs = in->cs; q.qn = (d.C + 3) / 4;
        q.B = in->B; q.H = in->H; q.W = in->W;
        q.w = c->d_wsmall; q.rows = conv_small_rows(d.C, d.O, d.kW * d.kH); q.bias = c->d_bias;
        q.out = out->data; q.out_cs = out->cs; q.out_dtype = out->dtype;
        q.O = d.O; q.OH = OH; q.OW = OW;
        q.kW = d.kW; q.kH = d.kH; q.strideX = d.strideX; q.strideY = d.strideY; q.padL = d.padL; q.padT = d.padT;
        q.dilX = d.dilX; q.dilY = d.dilY;
        q.fill = a.fill;
        q.epi = c->act->args;
        return conv_small_launch(q, stream);
    }
    if (c->pix4) {
        if (bn128) { if (w4) launch_cfg<128, 128, 2, true, true>(a, stream); else launch_cfg<128, 128, 2, true, false>(a, stream); }
        else { if (w4) launch_cfg<128, 64, 2, true, true>(a, stream); else launch_cfg<128, 64, 2, true, false>(a, stream); }
    } else if (!bn128) {
        if (w4) launch_cfg<128, 64, 2, false, true>(a, stream); else launch_cfg<128, 64, 2, false, false>(a, stream);
    } else if (bm64) {
        if (w4) launch_cfg<64, 128, 1, false, true>(a, stream); else launch_cfg<64, 128, 1, false, false>(a, stream);
    } else {
        if (w4) launch_cfg<128, 128, 2, false, true>(a, stream); else launch_cfg<128, 128, 2, false, false>(a, stream);
    }
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_conv_forward(n2d2hip_conv_t c, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    if (sub_sampled(c)) {
        N2D2HIP_REQUIRE(in && in->halo == 0, N2D2HIP_ERR_UNSUPPORTED, "conv_forward: a sub-sampled convolution takes its input without a halo");
        return conv_subsample_forward(c, in, out, stream);
    }
    return conv_forward_impl(c, in, nullptr, out, stream);
}

// The first-layer kernel can compute the max pooling behind it: 3x3 windows, stride 2, padding 0 or 1, on rows of at most
// 128 convolution outputs with at most 64 channels, byte outputs of an integer rescale whose scaled-up tables fit.
static bool stem_pool_eligible(const n2d2hip_conv_s* c, const n2d2hip_pool_desc* pd, int H, int W, int* OHo, int* OWo, int* POHo, int* POWo)
{
    const n2d2hip_conv_desc& d = c->desc;
    int OH, OW, POH, POW;
    if (!c->d_wstem || (d.kernel_choice & (N2D2HIP_KERNEL_NO_STEM | N2D2HIP_KERNEL_NO_HI16)) || c->act->args.kind != EPI_I24 || !c->bias_folded
        || !c->hi16 || c->act->min_out < -128 || c->act->max_out > 255 || d.O > 64 || d.O <= 48 || (d.kH != 3 && d.kH != 5 && d.kH != 7))
        return false;
    if (n2d2hip_conv_out_dims(&d, H, W, &OH, &OW) != N2D2HIP_OK || OW > 128)
        return false;
    if (pd->pooling != N2D2HIP_POOL_MAX || pd->poolW != 3 || pd->poolH != 3 || pd->strideX != 2 || pd->strideY != 2 || pd->padX != pd->padY
        || (pd->padX != 0 && pd->padX != 1) || n2d2hip_pool_out_dims(pd, OH, OW, &POH, &POW) != N2D2HIP_OK || POW > 64)
        return false;
    // every window holds at least one convolution output
    if ((POW - 1) * 2 - pd->padX >= OW || (POH - 1) * 2 - pd->padY >= OH)
        return false;
    *OHo = OH; *OWo = OW; *POHo = POH; *POWo = POW;
    return true;
}

int n2d2hip_conv_accepts_maxpool(n2d2hip_conv_t c, const n2d2hip_pool_desc* pool, int H, int W)
{
    int a, b, e, f;
    return c && pool && stem_pool_eligible(c, pool, H, W, &a, &b, &e, &f) ? 1 : 0;
}

int n2d2hip_conv_s2d_halo(n2d2hip_conv_t c, const n2d2hip_pool_desc* pool, int H, int W)
{
    if (!c || H <= 0 || W <= 0)
        return -1;
    const int halo = s2d_halo(c, H, W);
    if (halo < 0 || !pool)
        return halo;
    int OH, OW, POH, POW;
    const bool hi16 = c->hi16 && !(c->desc.kernel_choice & N2D2HIP_KERNEL_NO_HI16);
    if (!stem_pool_eligible(c, pool, H, W, &OH, &OW, &POH, &POW) || !hi16 || POW > 62)
        return -1;
    return halo;
}

int n2d2hip_conv_forward_maxpool(n2d2hip_conv_t c, const n2d2hip_pool_desc* pool, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                                 n2d2hip_stream_t stream_)
{
    int rc, OH, OW, POH, POW;
    N2D2HIP_REQUIRE(c && pool, N2D2HIP_ERR_INVALID, "conv_forward_maxpool: null argument");
    if ((rc = check_tensor(in, "conv input", false, true)) || (rc = check_tensor(out, "pooled output", true)))
        return rc;
    const n2d2hip_conv_desc& d = c->desc;
    const bool s2d = in->layout == N2D2HIP_S2D;
    N2D2HIP_REQUIRE((in->layout == N2D2HIP_NHWC || s2d) && out->layout == N2D2HIP_NHWC, N2D2HIP_ERR_UNSUPPORTED,
                    "conv_forward_maxpool: the input must be NHWC or space-to-depth, the output NHWC");
    N2D2HIP_REQUIRE(in->dtype == c->in_dtype && in->C == d.C && (s2d || in->cs == c->in_cs), N2D2HIP_ERR_INVALID,
                    "conv_forward_maxpool: input has %d channels (stride %d) of type %d, conv expects %d (stride %d) of type %d", in->C, in->cs,
                    in->dtype, d.C, c->in_cs, c->in_dtype);
    N2D2HIP_REQUIRE(stem_pool_eligible(c, pool, in->H, in->W, &OH, &OW, &POH, &POW), N2D2HIP_ERR_UNSUPPORTED,
                    "conv_forward_maxpool: needs a convolution the first-layer kernel runs with scaled-up integer tables (at most 4 input and "
                    "64 output channels, rows of at most 128 outputs) and a 3x3 stride-2 max pooling with padding 0 or 1 "
                    "(n2d2hip_conv_accepts_maxpool)");
    N2D2HIP_REQUIRE(out->B == in->B && out->C == d.O && out->H == POH && out->W == POW && out->cs == 64
                        && (out->dtype == N2D2HIP_U8B || out->dtype == N2D2HIP_I8),
                    N2D2HIP_ERR_INVALID, "conv_forward_maxpool: output must be %dx%dx%dx%d bytes (U8B or I8) with a channel stride of 64", in->B,
                    d.O, POH, POW);
    {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(c->act->min_out >= lo && c->act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "conv_forward_maxpool: activation range [%d,%d] does not fit output dtype %d", c->act->min_out, c->act->max_out, out->dtype);
    }
    N2D2HIP_REQUIRE((long long)in->B * in->H * in->W * in->cs < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED, "conv_forward_maxpool: tensor too large");
    if (s2d) {
        N2D2HIP_REQUIRE(n2d2hip_conv_s2d_halo(c, pool, in->H, in->W) >= 0, N2D2HIP_ERR_UNSUPPORTED,
                        "conv_forward_maxpool: this pair does not read space-to-depth inputs (n2d2hip_conv_s2d_halo)");
        return conv_s2d_forward(c, in, out, pool, OH, OW, POH, POW, (hipStream_t)stream_);
    }
    ConvArgs a;
    a.in = (const signed char*)in->data;
    a.in_cs = in->cs; a.B = in->B; a.H = in->H; a.W = in->W;
    a.OH = OH; a.OW = OW; a.M = in->B * OH * OW;
    a.w = c->d_w; a.ktot = c->ktot; a.niter = c->ktot / 64; a.sub = c->d_sub; a.bias = c->d_bias;
    a.out = out->data; a.out_cs = out->cs; a.out_dtype = out->dtype;
    a.strideX = d.strideX; a.strideY = d.strideY; a.padL = d.padL; a.padT = d.padT; a.dilX = d.dilX; a.dilY = d.dilY;
    a.kW = d.kW; a.kH = d.kH;
    a.ntiles_n = 1; a.nblocks = 0;
    a.fill = zero_point(in->dtype) ? 0x80808080u : 0u;
    a.out_xor = out->dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    a.epi = c->act->args;
    ConvStemArgs q = {};
    q.c = a;
    const int cp = c->act->cpad;
    q.c.epi.a = c->d_epi_tab; q.c.epi.b = c->d_epi_tab + cp; q.c.epi.c = c->d_epi_tab + 5 * cp;
    q.c.epi.d = c->d_epi_tab + 6 * cp; q.c.epi.e = c->d_epi_tab + 4 * cp;
    q.wk = c->d_wstem;
    q.fill16 = c->d_fill;
    q.preclamp = c->preclamp ? 1 : 0;
    q.tiles_per_row = 1;
    // strips: about two per block slot, so that the one convolution row two neighbouring strips both compute stays a small
    // share of the work; a strip's rows are consecutive, so its input rows come out of the cache
    const int slots = 2 * num_cus();
    int rows = std::max(1, (int)(((long long)in->B * POH + 2 * slots - 1) / (2 * slots)));
    rows = std::min(std::max(rows, std::min(POH, 4)), POH);
    q.pool_rows = rows;
    q.strips_per_image = (POH + rows - 1) / rows;
    q.pool_pad = pool->padX;
    q.POH = POH; q.POW = POW;
    q.pool_halo = out->halo; q.POHp = POH + 2 * out->halo; q.POWp = POW + 2 * out->halo;
    q.ntiles = in->B * q.strips_per_image;
    // two blocks per compute unit (64 KB of LDS each)
    q.nlanes = std::max(1, std::min((q.ntiles + 7) / 8, (2 * num_cus()) / 8));
    q.xcd_tiles = (q.ntiles + 7) / 8;
    const int grid = 8 * q.nlanes;
    hipStream_t stream = (hipStream_t)stream_;
    if (d.kH == 3) N2D2HIP_LAUNCH_T(conv_stem_kernel, (3, EPI_I24, true, true), dim3(grid), dim3(256), 0, stream, q);
    else if (d.kH == 5) N2D2HIP_LAUNCH_T(conv_stem_kernel, (5, EPI_I24, true, true), dim3(grid), dim3(256), 0, stream, q);
    else N2D2HIP_LAUNCH_T(conv_stem_kernel, (7, EPI_I24, true, true), dim3(grid), dim3(256), 0, stream, q);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_conv_accepts_halo(n2d2hip_conv_t c)
{
    bool bn128;
    return c && pipe_eligible(c, &bn128) && c->desc.dilX == 1 && c->desc.dilY == 1 && !(c->desc.kernel_choice & N2D2HIP_KERNEL_NO_PIPE) ? 1 : 0;
}

int n2d2hip_conv_desc_reads_halo(const n2d2hip_conv_desc* d)
{
    return d && pipe_shape(*d) && d->dilX == 1 && d->dilY == 1 && d->subX <= 1 && d->subY <= 1 && !(d->kernel_choice & N2D2HIP_KERNEL_NO_PIPE) ? 1 : 0;
}

int n2d2hip_conv_fuse_sum(n2d2hip_conv_t c, n2d2hip_elemwise_t sum, int conv_input_index, int other_dtype)
{
    N2D2HIP_REQUIRE(c != nullptr, N2D2HIP_ERR_INVALID, "conv_fuse_sum: null conv");
    if (c->d_res_tab) { (void)hipFree(c->d_res_tab); c->d_res_tab = nullptr; }
    c->sum = nullptr;
    if (!sum)
        return N2D2HIP_OK;
    N2D2HIP_REQUIRE(conv_input_index == 0 || conv_input_index == 1, N2D2HIP_ERR_INVALID, "conv_fuse_sum: input index %d", conv_input_index);
    N2D2HIP_REQUIRE(is_byte_type(other_dtype), N2D2HIP_ERR_INVALID, "conv_fuse_sum: the other input must be U8, I8 or U8B");
    const n2d2hip_conv_desc& d = c->desc;
    N2D2HIP_REQUIRE(sum->nb_channels == d.O, N2D2HIP_ERR_INVALID, "conv_fuse_sum: the sum has %d channels, the conv %d outputs", sum->nb_channels, d.O);
    bool bn128;
    const bool one_by_one = d.kW == 1 && d.kH == 1 && d.padL == 0 && d.padT == 0 && d.padR == 0 && d.padB == 0;
    const n2d2hip_act_s* ca = c->act;
    const n2d2hip_act_s* sa = sum->act;
    const n2d2hip_act_s* pa = sum->pre_input >= 0 ? sum->pre_act : nullptr;
    const bool ok = pipe_eligible(c, &bn128) && (d.weight_bits == 4 || one_by_one) && d.dilX == 1 && d.dilY == 1 && round_up(d.O, 16) % (bn128 ? 128 : 64) == 0
        && ca->args.kind == EPI_I24 && ca->min_out >= -128 && ca->max_out <= 255
        && sum->nb_inputs == 2 && sum->unit_coeff && sa->args.kind == EPI_I24 && sa->min_out >= -128 && sa->max_out <= 255
        && (sum->pre_input < 0 || sum->pre_input == 1 - conv_input_index);
    N2D2HIP_REQUIRE(ok, N2D2HIP_ERR_UNSUPPORTED,
                    "conv_fuse_sum: needs a 1x1 unpadded 8-bit convolution (or any undilated one with 4-bit weights) with a multiple of 64 "
                    "input and output channels and integer rescales on the convolution and on a two-input unit-coefficient sum");
    // Tables of the sum (and of the ScalingCell folded onto the other input) with the other input's zero point
    // folded in: the kernel turns the stored byte into an unsigned one (U8B and I8 bytes with their top bit flipped,
    // which is the value itself for U8B and the value + 128 for I8) and adds that.
    const int cp = sa->cpad;
    const long long zp = other_dtype == N2D2HIP_I8 ? -128 : 0;
    const long long IMIN = std::numeric_limits<int>::min(), IMAX = std::numeric_limits<int>::max();
    std::vector<int> t(14 * (size_t)cp, 0);
    // The sum stage in 16-bit pairs needs: no clamp before a multiply anywhere, (conv + other) * c + d inside 16 bits, and
    // the two rescales in front of it in the form that leaves their result in the upper half of a 32-bit register
    bool sum16 = !c->preclamp && c->hi16 && cp % 2 == 0 && !(d.kernel_choice & N2D2HIP_KERNEL_NO_SUM16);
    short* t16 = (short*)(t.data() + 10 * (size_t)cp);
    bool pre_clamp = pa ? pa->clipped : false, sum_clamp = sa->clipped;
    bool pre_in_range = pa != nullptr;
    const long long other_lo = pa ? pa->min_out : (other_dtype == N2D2HIP_I8 ? -128 : 0);
    const long long other_hi = pa ? pa->max_out : (other_dtype == N2D2HIP_I8 ? 127 : 255);
    for (int ch = 0; ch < cp; ++ch) {
        // sum: s = conv + other (+ zp when there is no ScalingCell in between)
        const long long szp = pa ? 0 : zp;
        const long long a = sa->htab[ch], b = sa->htab[cp + ch], m = sa->htab[2 * (size_t)cp + ch], dd = sa->htab[3 * (size_t)cp + ch];
        t[ch] = (int)std::min(IMAX, std::max(IMIN, a - szp));
        t[cp + ch] = (int)std::min(IMAX, std::max(IMIN, b - szp));
        t[2 * (size_t)cp + ch] = (int)m;
        const long long d2 = dd + szp * m;
        t[4 * (size_t)cp + ch] = sa->htab[4 * (size_t)cp + ch];
        const long long smax = std::max(std::llabs(ca->min_out + other_lo - szp), std::llabs(ca->max_out + other_hi - szp)) + 1;
        if (d2 < IMIN || d2 > IMAX)
            return fail(N2D2HIP_ERR_UNSUPPORTED, "conv_fuse_sum: the sum's rescale of channel %d leaves 32 bits once folded", ch);
        if (smax * m + std::llabs(d2) > IMAX)
            sum_clamp = true;
        t[3 * (size_t)cp + ch] = (int)d2;
        const long long e2 = sa->htab[4 * (size_t)cp + ch];
        if (m < 0 || e2 < 0 || e2 > 15 || smax * m + std::llabs(d2) > 32767)
            sum16 = false;
        t16[ch] = (short)m;
        t16[cp + ch] = (short)d2;
        t16[2 * (size_t)cp + ch] = (short)e2;
        if (pa) {
            const long long xa = pa->htab[ch], xb = pa->htab[cp + ch], xm = pa->htab[2 * (size_t)cp + ch], xd = pa->htab[3 * (size_t)cp + ch];
            const long long xd2 = xd + zp * xm;
            if (xd2 < IMIN || xd2 > IMAX || 256 * xm + std::llabs(xd2) > IMAX)
                pre_clamp = true;
            if (xd2 < IMIN || xd2 > IMAX)
                return fail(N2D2HIP_ERR_UNSUPPORTED, "conv_fuse_sum: the folded ScalingCell of channel %d leaves 32 bits", ch);
            // 16-bit pairs: the stored byte (0..255) times a 24-bit unsigned multiplier scaled up by 2^(16 - e), inside 32
            // bits with the addend
            const long long xe = pa->htab[4 * (size_t)cp + ch];
            // a non-negative multiplier makes the rescale monotonic: its extremes are at the bytes 0 and 255
            if (xm < 0 || xe < 0 || xe > 31 || (xd2 >> xe) < pa->min_out || ((255 * xm + xd2) >> xe) > pa->max_out)
                pre_in_range = false;
            const long long up = (xe >= 0 && xe <= 16) ? (1ll << (16 - xe)) : 0;
            if (up == 0 || xm < 0 || xm * up >= (1 << 24) || (255 * xm + std::llabs(xd2)) * up > IMAX) {
                sum16 = false;
            } else {
                t[12 * (size_t)cp + ch] = (int)(xm * up);
                t[13 * (size_t)cp + ch] = (int)(xd2 * up);
            }
            t[5 * (size_t)cp + ch] = (int)std::min(IMAX, std::max(IMIN, xa - zp));
            t[6 * (size_t)cp + ch] = (int)std::min(IMAX, std::max(IMIN, xb - zp));
            t[7 * (size_t)cp + ch] = (int)xm;
            t[8 * (size_t)cp + ch] = (int)xd2;
            t[9 * (size_t)cp + ch] = pa->htab[4 * (size_t)cp + ch];
        }
    }
    hipError_t e = hipMalloc((void**)&c->d_res_tab, t.size() * sizeof(int));
    if (e == hipSuccess) e = hipMemcpy(c->d_res_tab, t.data(), t.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        if (c->d_res_tab) { (void)hipFree(c->d_res_tab); c->d_res_tab = nullptr; }
        return fail(N2D2HIP_ERR_HIP, "conv_fuse_sum: device upload failed: %s", hipGetErrorString(e));
    }
    c->sum = sum;
    c->sum_other_dtype = other_dtype;
    c->has_pre = pa != nullptr;
    c->pre_clamp = pre_clamp;
    c->sum_clamp = sum_clamp;
    c->sum16 = sum16 && !pre_clamp && !sum_clamp;
    c->pre_in_range = pre_in_range;
    return N2D2HIP_OK;
}

int n2d2hip_conv_forward_sum(n2d2hip_conv_t c, const n2d2hip_tensor* in, const n2d2hip_tensor* other, const n2d2hip_tensor* out,
                             n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(c != nullptr && other != nullptr, N2D2HIP_ERR_INVALID, "conv_forward_sum: null argument");
    N2D2HIP_REQUIRE(c->sum != nullptr, N2D2HIP_ERR_INVALID, "conv_forward_sum: no sum has been folded into this convolution");
    return conv_forward_impl(c, in, other, out, stream);
}

// Can the pair (3x3 convolution, 1x1 expansion with a folded sum) run as one launch?
static bool chain_ok(const n2d2hip_conv_s* c3, const n2d2hip_conv_s* ce)
{
    if (!c3 || !ce)
        return false;
    const n2d2hip_conv_desc& d = c3->desc;
    const n2d2hip_conv_desc& x = ce->desc;
    if (c3->depthwise || c3->pix4 || d.weight_bits != 8 || d.groups != 1 || d.kW != 3 || d.kH != 3 || d.dilX != 1 || d.dilY != 1
        || d.strideX != d.strideY || (d.strideX != 1 && d.strideX != 2) || d.padL != 1 || d.padT != 1 || d.padR != 1 || d.padB != 1
        || d.C != d.O || !conv_chain_channels(d.C) || c3->in_cs != d.C || c3->ktot != 9 * d.C || c3->act->args.kind != EPI_I24
        || !c3->bias_folded || !c3->hi16 || (d.kernel_choice & (N2D2HIP_KERNEL_NO_PIPE | N2D2HIP_KERNEL_NO_HI16)))
        return false;
    if (!ce->d_wchain || x.C != d.O || x.O != 4 * d.O || x.strideX != 1 || x.strideY != 1 || x.padL != 0 || x.padT != 0 || x.padR != 0
        || x.padB != 0 || !ce->sum || !ce->sum16 || !ce->hi16 || ce->act->args.kind != EPI_I24
        || (x.kernel_choice & (N2D2HIP_KERNEL_NO_PIPE | N2D2HIP_KERNEL_NO_HI16 | N2D2HIP_KERNEL_NO_SUM16)))
        return false;
    // the middle tensor is stored as the expansion reads its input
    const int lo = ce->in_dtype == N2D2HIP_I8 ? -128 : 0, hi = ce->in_dtype == N2D2HIP_I8 ? 127 : 255;
    return c3->act->min_out >= lo && c3->act->max_out <= hi;
}

int n2d2hip_conv_chain_supported(n2d2hip_conv_t conv3x3, n2d2hip_conv_t expand)
{
    return chain_ok(conv3x3, expand) ? 1 : 0;
}

int n2d2hip_conv_chain_forward(n2d2hip_conv_t c3, n2d2hip_conv_t ce, const n2d2hip_tensor* in, const n2d2hip_tensor* other,
                               const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc;
    N2D2HIP_REQUIRE(c3 && ce && other, N2D2HIP_ERR_INVALID, "conv_chain_forward: null argument");
    N2D2HIP_REQUIRE(chain_ok(c3, ce), N2D2HIP_ERR_UNSUPPORTED,
                    "conv_chain_forward: needs a 3x3 convolution (stride 1 or 2, padding 1, 64, 128 or 256 channels in and out) and a 1x1 "
                    "expansion to four times the channels with a folded sum on 16-bit pairs, both 8-bit with scaled-up integer "
                    "rescales (n2d2hip_conv_chain_supported)");
    if ((rc = check_tensor(in, "conv input", true)) || (rc = check_tensor(other, "sum input", true)) || (rc = check_tensor(out, "sum output", true)))
        return rc;
    const n2d2hip_conv_desc& d = c3->desc;
    const int OC = ce->desc.O;
    N2D2HIP_REQUIRE(in->layout == N2D2HIP_NHWC && other->layout == N2D2HIP_NHWC && out->layout == N2D2HIP_NHWC, N2D2HIP_ERR_UNSUPPORTED,
                    "conv_chain_forward: tensors must be NHWC");
    N2D2HIP_REQUIRE(in->dtype == c3->in_dtype && in->C == d.C && in->cs == c3->in_cs && in->halo >= 1, N2D2HIP_ERR_INVALID,
                    "conv_chain_forward: the input must have %d channels of type %d and carry its padding as a border (halo >= 1)", d.C,
                    c3->in_dtype);
    int OH, OW;
    if ((rc = n2d2hip_conv_out_dims(&d, in->H, in->W, &OH, &OW)))
        return rc;
    N2D2HIP_REQUIRE(out->B == in->B && out->C == OC && out->H == OH && out->W == OW && is_byte_type(out->dtype) && out->cs % 16 == 0
                        && out->cs >= OC,
                    N2D2HIP_ERR_INVALID, "conv_chain_forward: output must be %dx%dx%dx%d bytes", in->B, OC, OH, OW);
    N2D2HIP_REQUIRE(other->dtype == ce->sum_other_dtype && other->B == out->B && other->C == OC && other->H == OH && other->W == OW
                        && other->cs % 16 == 0 && other->cs >= OC,
                    N2D2HIP_ERR_INVALID, "conv_chain_forward: the other input must be an NHWC tensor of the output's shape and of the "
                    "storage type given to n2d2hip_conv_fuse_sum");
    const n2d2hip_act_s* sact = ce->sum->act;
    {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(sact->min_out >= lo && sact->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "conv_chain_forward: activation range [%d,%d] does not fit output dtype %d", sact->min_out, sact->max_out, out->dtype);
    }
    const int Hp = in->H + 2 * in->halo, Wp = in->W + 2 * in->halo;
    const long long Mll = (long long)in->B * OH * OW;
    const long long out_pixels = (long long)in->B * (OH + 2 * out->halo) * (OW + 2 * out->halo);
    const long long other_pixels = (long long)in->B * (OH + 2 * other->halo) * (OW + 2 * other->halo);
    N2D2HIP_REQUIRE(Mll < (1ll << 31) && (long long)in->B * Hp * Wp * in->cs < (1ll << 31) && out_pixels * out->cs < (1ll << 31)
                        && other_pixels * other->cs < (1ll << 31),
                    N2D2HIP_ERR_UNSUPPORTED, "conv_chain_forward: tensor too large");
    ConvChainArgs a = {};
    ConvArgs& ca = a.p.c;
    ca.in = (const signed char*)in->data;
    ca.in_cs = in->cs; ca.B = in->B; ca.H = Hp; ca.W = Wp;
    ca.OH = OH; ca.OW = OW; ca.M = (int)Mll;
    ca.w = c3->d_w; ca.ktot = c3->ktot; ca.niter = 0; ca.sub = nullptr; ca.bias = nullptr;
    ca.out = out->data; ca.out_cs = out->cs; ca.out_dtype = out->dtype;
    ca.strideX = d.strideX; ca.strideY = d.strideY; ca.padL = d.padL - in->halo; ca.padT = d.padT - in->halo; ca.dilX = 1; ca.dilY = 1;
    ca.kW = 3; ca.kH = 3;
    ca.ntiles_n = 1; ca.nblocks = 0;
    ca.fill = 0;
    ca.out_xor = out->dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    ca.epi = c3->act->args;
    ca.epi.c = c3->d_epi_tab + 5 * c3->act->cpad;
    ca.epi.d = c3->d_epi_tab + 6 * c3->act->cpad;
    a.p.fill16 = c3->d_fill;
    a.p.kW = 3; a.p.kH = 3;
    a.p.preclamp = 0;
    magic_div((unsigned)(OH * OW), &a.p.ohw_mul, &a.p.ohw_sh);
    magic_div((unsigned)OW, &a.p.ow_mul, &a.p.ow_sh);
    a.p.out_halo = out->halo;
    a.p.out_pixels = (int)out_pixels;
    const int cps = sact->cpad;
    a.p.res = (const signed char*)other->data;
    a.p.res_cs = other->cs;
    a.p.res_halo = other->halo;
    a.p.res_flip = other->dtype == N2D2HIP_U8 ? 0u : 0x80808080u;
    a.p.sum = sact->args;
    a.p.sum16 = ce->d_res_tab + 10 * cps;
    a.p.sum16_stride = cps / 2;
    a.p.has_pre = ce->has_pre ? 1 : 0;
    a.p.pre_clamp = 0; a.p.sum_clamp = 0;
    a.p.pre_in_range = ce->pre_in_range ? 1 : 0;
    a.p.pre = EpiArgs();
    if (ce->has_pre) {
        a.p.pre = ce->sum->pre_act->args;
        a.p.pre.c = ce->d_res_tab + 12 * cps;
        a.p.pre.d = ce->d_res_tab + 13 * cps;
    }
    a.we = ce->d_wchain;
    a.etc = ce->d_epi_tab + 5 * ce->act->cpad;
    a.etd = ce->d_epi_tab + 6 * ce->act->cpad;
    a.e_lo = ce->act->args.lo; a.e_hi = ce->act->args.hi;
    a.t2_xor = ce->in_dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    return conv_chain_launch(a, num_cus(), (hipStream_t)stream);
}

// ------------------------------------------------------------------- fc
int n2d2hip_fc_create(int C, int H, int W, int O, int weight_bits, const void* weights, const int32_t* bias,
                      n2d2hip_act_t act, int in_dtype, n2d2hip_fc_t* fc)
{
    N2D2HIP_REQUIRE(C > 0 && H > 0 && W > 0 && O > 0, N2D2HIP_ERR_INVALID, "fc_create: bad shape");
    // [O][C*H*W] in CHW order is exactly an OCHW kernel of size H x W.
    n2d2hip_conv_desc d = {};
    d.C = C; d.O = O; d.kW = W; d.kH = H;
    d.strideX = d.strideY = 1; d.dilX = d.dilY = 1; d.groups = 1; d.weight_bits = weight_bits;
    int rc = n2d2hip_conv_create(&d, weights, bias, act, in_dtype, fc);
    if (rc == N2D2HIP_OK) { (*fc)->is_fc = true; (*fc)->fcH = H; (*fc)->fcW = W; }
    return rc;
}

int n2d2hip_fc_destroy(n2d2hip_fc_t fc) { return n2d2hip_conv_destroy(fc); }

int n2d2hip_fc_forward(n2d2hip_fc_t fc, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(fc != nullptr && in != nullptr, N2D2HIP_ERR_INVALID, "fc_forward: null argument");
    N2D2HIP_REQUIRE(fc->is_fc, N2D2HIP_ERR_INVALID, "fc_forward: handle was not created by n2d2hip_fc_create");
    N2D2HIP_REQUIRE(in->H == fc->fcH && in->W == fc->fcW, N2D2HIP_ERR_INVALID, "fc_forward: input is %dx%d, cell built for %dx%d",
                    in->H, in->W, fc->fcH, fc->fcW);
    return n2d2hip_conv_forward(fc, in, out, stream);
}

} // extern "C"
