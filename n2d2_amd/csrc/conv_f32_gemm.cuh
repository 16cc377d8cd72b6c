// Float32 convolution (forward, backward-data, backward-filter) as an implicit GEMM on the fp32 matrix cores
// (v_mfma_f32_32x32x2f32), for ungrouped convolutions without dilation on N2D2's NCHW / OCHW tensors.
//
// One kernel, three addressings.  The product is out[q][p] = sum_k Qop[q][k] * Pop[k][p], where p runs along the
// dimension that is contiguous in the output tensor (so that the 32 lanes holding one accumulator row write 128
// consecutive bytes) and q along the other one:
//   forward          p = output pixel (b,oy,ox)   q = output channel   k = (c,ty,tx)      Pop = x gathered, Qop = w
//   backward data    p = input pixel (b,iy,ix)    q = input channel    k = (o,ty,tx)      Pop = dy gathered, Qop = w
//   backward filter  p = weight (c,ty,tx)         q = output channel   k = pixel (b,oy,ox) Pop = x gathered, Qop = dy
// Taps that fall outside the tensor contribute zero, which is what the reference's clipped window computes.
//
// A block of 256 threads (4 waves as 2 x 2) owns a 128 (q) x 128 (p) tile; each wave 64 x 64 as 2 x 2 MFMA tiles.
// K advances in steps of 16 through two LDS tiles [k][p] and [k][q] (row stride 129 floats); the next step's
// elements are fetched into registers while the matrix cores work on the current one.  Backward-filter, whose K is
// the whole batch of pixels and whose output is small, splits K over blockIdx.z into partial results that a second
// kernel adds up in a fixed order.
#pragma once

#include "common.h"

namespace n2d2hip {

typedef float v16f __attribute__((ext_vector_type(16)));

enum { GEMM_FWD = 0, GEMM_BWD_DATA = 1, GEMM_BWD_FILTER = 2 };

struct GemmF32 {
    int B, C, H, W, O, oH, oW, kW, kH;
    int sx, sy, pl, pt;
    int P, Q, K;          // GEMM extents
    int kchunk;           // K range of one blockIdx.z (a multiple of 16)
};

constexpr int GT = 128;       // tile edge (both p and q)
constexpr int GK = 16;        // K step
constexpr int GLD = GT + 1;   // LDS row stride in floats

template <int MODE>
__global__ __launch_bounds__(256) void conv_f32_gemm_kernel(GemmF32 g, const float* __restrict__ srcP, const float* __restrict__ srcQ,
                                                            const float* __restrict__ bias, float beta, float* __restrict__ out)
{
    __shared__ float Ps[GK * GLD];
    __shared__ float Qs[GK * GLD];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wq = wave >> 1, wp = wave & 1;
    const int ptile = blockIdx.x * GT, qtile = blockIdx.y * GT;
    const int kbeg = blockIdx.z * g.kchunk, kend = min(kbeg + g.kchunk, g.K);
    const int kHW = g.kH * g.kW;

    // ---- per-thread loader state.  FWD / BWD_DATA: thread owns one p (and one q) and 8 consecutive k of each step.
    // BWD_FILTER: thread owns one k of each step and 8 p (and 8 q) spaced by 16.
    const int lp = (MODE == GEMM_BWD_FILTER) ? (t >> 4) : (t & 127);     // first local p (and q for BWD_DATA / BWD_FILTER)
    const int lk = (MODE == GEMM_BWD_FILTER) ? (t & 15) : ((t >> 7) * 8); // first local k
    // FWD Q operand (weights, contiguous along k): q = t / 2, k = (t % 2) * 8 + i
    const int lq_w = t >> 1, lk_w = (t & 1) * 8;

    int pb = 0, py = 0, px = 0;             // decoded p (FWD: b,oy,ox; BWD_DATA: b,iy,ix)
    bool pvalid = false;
    int pc[8], pty[8], ptx[8];              // BWD_FILTER: decoded p_i = (c,ty,tx)
    if (MODE == GEMM_BWD_FILTER) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int p = ptile + lp + 16 * i;
            const int pp = min(p, g.P - 1);
            pc[i] = (p < g.P) ? pp / kHW : -1;
            pty[i] = (pp % kHW) / g.kW;
            ptx[i] = pp % g.kW;
        }
    } else {
        const int p = ptile + lp;
        pvalid = p < g.P;
        const int plane = (MODE == GEMM_FWD) ? g.oH * g.oW : g.H * g.W;
        const int row = (MODE == GEMM_FWD) ? g.oW : g.W;
        const int pp = pvalid ? p : 0;
        pb = pp / plane;
        py = (pp % plane) / row;
        px = pp % row;
    }

    float rp[8], rq[8];
    auto fetch = [&](int k0) {
        if (MODE == GEMM_BWD_FILTER) {
            const int k = k0 + lk;
            const bool kv = k < kend;
            const int kk = kv ? k : 0;
            const int plane = g.oH * g.oW;
            const int b = kk / plane, oy = (kk % plane) / g.oW, ox = kk % g.oW;
            const int iy0 = oy * g.sy - g.pt, ix0 = ox * g.sx - g.pl;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int iy = iy0 + pty[i], ix = ix0 + ptx[i];
                const bool v = kv && pc[i] >= 0 && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                rp[i] = v ? srcP[(((size_t)b * g.C + pc[i]) * g.H + iy) * g.W + ix] : 0.0f;
                const int q = qtile + lp + 16 * i;
                rq[i] = (kv && q < g.Q) ? srcQ[((size_t)b * g.O + q) * plane + kk % plane] : 0.0f;
            }
        } else {
            // P operand: k = k0 + lk + i -> (channel-like, ty, tx), advanced with carries
            int k = k0 + lk;
            int ch = k / kHW, ty = (k % kHW) / g.kW, tx = k % g.kW;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float v = 0.0f;
                if (pvalid && k + i < kend) {
                    if (MODE == GEMM_FWD) {
                        const int iy = py * g.sy - g.pt + ty, ix = px * g.sx - g.pl + tx;
                        if (iy >= 0 && iy < g.H && ix >= 0 && ix < g.W)
                            v = srcP[(((size_t)pb * g.C + ch) * g.H + iy) * g.W + ix];
                    } else {
                        const int ny = py + g.pt - ty, nx = px + g.pl - tx;
                        if (ny >= 0 && nx >= 0 && ny % g.sy == 0 && nx % g.sx == 0) {
                            const int oy = ny / g.sy, ox = nx / g.sx;
                            if (oy < g.oH && ox < g.oW)
                                v = srcP[(((size_t)pb * g.O + ch) * g.oH + oy) * g.oW + ox];
                        }
                    }
                }
                rp[i] = v;
                if (++tx == g.kW) { tx = 0; if (++ty == g.kH) { ty = 0; ++ch; } }
            }
            if (MODE == GEMM_FWD) {
                const int q = qtile + lq_w;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int kq = k0 + lk_w + i;
                    rq[i] = (q < g.Q && kq < kend) ? srcQ[(size_t)q * g.K + kq] : 0.0f;
                }
            } else {
                const int q = qtile + lp;           // input channel c; w[(o*C + c)*kHW + tap], k = o*kHW + tap
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int kq = k + i;
                    rq[i] = (q < g.Q && kq < kend) ? srcQ[((size_t)(kq / kHW) * g.C + q) * kHW + kq % kHW] : 0.0f;
                }
            }
        }
    };
    auto stage = [&]() {
        if (MODE == GEMM_BWD_FILTER) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                Ps[lk * GLD + lp + 16 * i] = rp[i];
                Qs[lk * GLD + lp + 16 * i] = rq[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                Ps[(lk + i) * GLD + lp] = rp[i];
                if (MODE == GEMM_FWD) Qs[(lk_w + i) * GLD + lq_w] = rq[i];
                else Qs[(lk + i) * GLD + lp] = rq[i];
            }
        }
    };

    v16f acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    if (kbeg < kend) {
        fetch(kbeg);
        for (int k0 = kbeg; k0 < kend; k0 += GK) {
            __syncthreads();            // the previous step's reads of the LDS tiles are done
            stage();
            __syncthreads();
            if (k0 + GK < kend)
                fetch(k0 + GK);         // in flight while the matrix cores run
            const int kr = lane >> 5, col = lane & 31;
#pragma unroll
            for (int kk = 0; kk < GK / 2; ++kk) {
                const float* qrow = Qs + (kk * 2 + kr) * GLD + wq * 64 + col;
                const float* prow = Ps + (kk * 2 + kr) * GLD + wp * 64 + col;
                const float a0 = qrow[0], a1 = qrow[32], b0 = prow[0], b1 = prow[32];
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
                acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
                acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: lane holds column p = .. + lane % 32 and rows q = .. + 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int pi = 0; pi < 2; ++pi) {
        const int p = ptile + wp * 64 + pi * 32 + (lane & 31);
        if (p >= g.P) continue;
        size_t base, qstride;
        if (MODE == GEMM_FWD) {
            const int plane = g.oH * g.oW;
            base = (size_t)(p / plane) * g.O * plane + p % plane;
            qstride = plane;
        } else if (MODE == GEMM_BWD_DATA) {
            const int plane = g.H * g.W;
            base = (size_t)(p / plane) * g.C * plane + p % plane;
            qstride = plane;
        } else {
            base = (size_t)blockIdx.z * g.Q * g.P + p;      // partial result of this K range
            qstride = g.P;
        }
#pragma unroll
        for (int qi = 0; qi < 2; ++qi) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int q = qtile + wq * 64 + qi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (q >= g.Q) continue;
                const size_t idx = base + (size_t)q * qstride;
                float v = acc[qi][pi][r];
                if (MODE != GEMM_BWD_FILTER) {
                    if (beta != 0.0f) v += beta * out[idx];
                    if (MODE == GEMM_FWD && bias) v = bias[q] + v;
                }
                out[idx] = v;
            }
        }
    }
}

// dw[i] = sum over the K ranges, in their order, + beta * dw[i]
__global__ __launch_bounds__(256) void conv_f32_reduce_partials_kernel(const float* __restrict__ partial, int splits, size_t n, float beta,
                                                                       float* __restrict__ dw)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        double s = 0.0;
        for (int z = 0; z < splits; ++z) s += (double)partial[(size_t)z * n + i];
        dw[i] = (float)s + (beta != 0.0f ? beta * dw[i] : 0.0f);
    }
}

} // namespace n2d2hip
