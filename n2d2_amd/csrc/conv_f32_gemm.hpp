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
// A block of 256 threads (4 waves as 2 x 2) owns a 128 (q) x 128 (p) tile; each wave 64 x 64 as 2 x 2 MFMA tiles.  With at
// most 64 rows of q (QT = 64) the four waves sit side by side along p instead, each 64 x 32.
// K advances in steps of 16 through two LDS tiles [k][p] and [k][q] (row stride 129 floats); the next step's
// elements are fetched into registers while the matrix cores work on the current one and are written to the other pair
// of tiles, so one barrier per step suffices.  Backward-filter, whose K is
// the whole batch of pixels and whose output is small, splits K over blockIdx.z into partial results that a second
// kernel adds up in a fixed order; forward and backward-data do the same when their tiles alone would not fill the chip.
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
    unsigned bytesP, bytesQ;   // sizes of the two operand tensors (each at most 2 GiB)
};

constexpr int GT = 128;       // tile edge (both p and q)
constexpr int GK = 16;        // K step
constexpr int GLD = GT + 1;   // LDS row stride in floats

template <int MODE, int QT>
__global__ __launch_bounds__(256) void conv_f32_gemm_kernel(GemmF32 g, const float* __restrict__ srcP, const float* __restrict__ srcQ,
                                                            const float* __restrict__ bias, float beta, float* __restrict__ out)
{
    __shared__ float Pbuf[2][GK * GLD];
    __shared__ float Qbuf[2][GK * GLD];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    constexpr int NP = QT / 64;                 // 32-column MFMA tiles of p per wave
    constexpr int NQL = QT / 16;                // q elements a thread fetches per step
    const int wq = (QT == 128) ? (wave >> 1) : 0;
    const int pw = (QT == 128) ? (wave & 1) * 64 : wave * 32;     // the wave's first p inside the tile
    const int ptile = blockIdx.x * GT, qtile = blockIdx.y * QT;
    const int kbeg = blockIdx.z * g.kchunk, kend = min(kbeg + g.kchunk, g.K);
    const int kHW = g.kH * g.kW;

    // ---- per-thread loader state.  FWD / BWD_DATA: thread owns one p (and one q) and 8 consecutive k of each step.
    // BWD_FILTER: thread owns one k of each step and 8 p (and 8 q) spaced by 16.
    const int lp = (MODE == GEMM_BWD_FILTER) ? (t >> 4) : (t & 127);     // first local p (and q for BWD_DATA / BWD_FILTER)
    const int lk = (MODE == GEMM_BWD_FILTER) ? (t & 15) : ((t >> 7) * 8); // first local k
    // Q operand of FWD (weights, contiguous along k): q = t / (16 / NQL), k = (t % (16 / NQL)) * NQL + i;
    // of BWD_DATA: q = t % QT, k = (t / QT) * NQL + i
    const int lq_w = (MODE == GEMM_FWD) ? t / (16 / NQL) : t % QT;
    const int lk_w = (MODE == GEMM_FWD) ? (t % (16 / NQL)) * NQL : (t / QT) * NQL;

    // Operands are read through buffer descriptors: an element that does not exist (padding, past the tile or the K
    // range) is requested at an offset past the end and comes back as zero, so the loads need no branches.  All
    // offsets fit 32 bits (checked by the host).
    const __amdgpu_buffer_rsrc_t rsrcP = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(srcP), 0, g.bytesP, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcQ = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(srcQ), 0, g.bytesQ, 0x00020000);
    auto ldP = [&](int off, bool valid) -> float {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrcP, valid ? (unsigned)off * 4u : 0x80000000u, 0, 0));
    };
    auto ldQ = [&](int off, bool valid) -> float {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrcQ, valid ? (unsigned)off * 4u : 0x80000000u, 0, 0));
    };
    int pb = 0, py = 0, px = 0;             // decoded p (FWD: b,oy,ox; BWD_DATA: b,iy,ix)
    bool pvalid = false;
    int pbase = 0;                          // FWD: offset of tap (0,0) of channel 0 for this pixel; BWD_DATA: of (b, o = 0)
    unsigned long long tapmask = 0;         // FWD: bit ty*kW+tx set if that tap lies inside the input (kH*kW <= 64)
    int poff[8], pty[8], ptx[8];            // BWD_FILTER: p_i = (c,ty,tx): offset c*H*W + ty*W + tx (-1: no such p), ty, tx
    if (MODE == GEMM_BWD_FILTER) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int p = ptile + lp + 16 * i;
            const int pp = min(p, g.P - 1);
            pty[i] = (pp % kHW) / g.kW;
            ptx[i] = pp % g.kW;
            poff[i] = (p < g.P) ? (pp / kHW) * g.H * g.W + pty[i] * g.W + ptx[i] : -1;
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
        if (MODE == GEMM_FWD) {
            const int iy0 = py * g.sy - g.pt, ix0 = px * g.sx - g.pl;
            pbase = (pb * g.C * g.H + iy0) * g.W + ix0;
            if (pvalid)
                for (int ty = 0; ty < g.kH; ++ty)
                    for (int tx = 0; tx < g.kW; ++tx)
                        if (iy0 + ty >= 0 && iy0 + ty < g.H && ix0 + tx >= 0 && ix0 + tx < g.W)
                            tapmask |= 1ull << (ty * g.kW + tx);
        } else {
            pbase = pb * g.O * g.oH * g.oW;
        }
    }

    float rp[8], rq[8];
    auto fetch = [&](int k0) {
        if (MODE == GEMM_BWD_FILTER) {
            const int k = k0 + lk;
            const bool kv = k < kend;
            const int kk = kv ? k : 0;
            const int plane = g.oH * g.oW;
            const int b = kk / plane, rem = kk % plane, oy = rem / g.oW, ox = rem % g.oW;
            const int iy0 = oy * g.sy - g.pt, ix0 = ox * g.sx - g.pl;
            const int xbase = (b * g.C * g.H + iy0) * g.W + ix0;
            const int ybase = b * g.O * plane + rem;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int iy = iy0 + pty[i], ix = ix0 + ptx[i];
                const bool v = kv && poff[i] >= 0 && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                rp[i] = ldP(xbase + poff[i], v);
                if (i < NQL) {
                    const int q = qtile + lp + 16 * i;
                    rq[i] = ldQ(ybase + q * plane, kv && q < g.Q);
                }
            }
        } else {
            // P operand: k = k0 + lk + i -> (channel-like, ty, tx), advanced with carries
            const int k = k0 + lk;
            int ch = k / kHW, tap = k % kHW, ty = tap / g.kW, tx = tap % g.kW;
            if (MODE == GEMM_FWD) {
                int off = pbase + ch * g.H * g.W + ty * g.W + tx;       // walks (c,ty,tx) with carries
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const bool v = ((tapmask >> tap) & 1) && k + i < kend;
                    rp[i] = ldP(off, v);
                    ++off; ++tap;
                    if (++tx == g.kW) {
                        tx = 0; off += g.W - g.kW;
                        if (tap == kHW) { tap = 0; off += (g.H - g.kH) * g.W; }
                    }
                }
            } else {
                const bool unit = g.sx == 1 && g.sy == 1;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int ny = py + g.pt - ty, nx = px + g.pl - tx;
                    int oy = ny, ox = nx;
                    bool v = pvalid && k + i < kend && ny >= 0 && nx >= 0;
                    if (!unit) {
                        oy = ny / g.sy; ox = nx / g.sx;
                        v = v && oy * g.sy == ny && ox * g.sx == nx;
                    }
                    v = v && oy < g.oH && ox < g.oW;
                    rp[i] = ldP(pbase + (ch * g.oH + oy) * g.oW + ox, v);
                    if (++tx == g.kW) { tx = 0; if (++ty == g.kH) { ty = 0; ++ch; } }
                }
            }
            if (MODE == GEMM_FWD) {
                const int q = qtile + lq_w;
#pragma unroll
                for (int i = 0; i < NQL; ++i) {
                    const int kq = k0 + lk_w + i;
                    rq[i] = ldQ(q * g.K + kq, q < g.Q && kq < kend);
                }
            } else {
                const int q = qtile + lq_w;         // input channel c; w[(o*C + c)*kHW + tap], k = o*kHW + tap
#pragma unroll
                for (int i = 0; i < NQL; ++i) {
                    const int kq = k0 + lk_w + i;
                    rq[i] = ldQ(((kq / kHW) * g.C + q) * kHW + kq % kHW, q < g.Q && kq < kend);
                }
            }
        }
    };
    auto stage = [&](int buf) {
        float* Ps = Pbuf[buf];
        float* Qs = Qbuf[buf];
        if (MODE == GEMM_BWD_FILTER) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                Ps[lk * GLD + lp + 16 * i] = rp[i];
                if (i < NQL) Qs[lk * GLD + lp + 16 * i] = rq[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                Ps[(lk + i) * GLD + lp] = rp[i];
                if (i < NQL) Qs[(lk_w + i) * GLD + lq_w] = rq[i];
            }
        }
    };

    v16f acc[2][NP];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < NP; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    if (kbeg < kend) {
        fetch(kbeg);
        stage(0);
        __syncthreads();
        int buf = 0;
        for (int k0 = kbeg; k0 < kend; k0 += GK, buf ^= 1) {
            const bool more = k0 + GK < kend;
            if (more)
                fetch(k0 + GK);         // in flight while the matrix cores run
            const float* Ps = Pbuf[buf];
            const float* Qs = Qbuf[buf];
            const int kr = lane >> 5, col = lane & 31;
#pragma unroll
            for (int kk = 0; kk < GK / 2; ++kk) {
                const float* qrow = Qs + (kk * 2 + kr) * GLD + wq * 64 + col;
                const float* prow = Ps + (kk * 2 + kr) * GLD + pw + col;
                const float a0 = qrow[0], a1 = qrow[32];
#pragma unroll
                for (int pi = 0; pi < NP; ++pi) {
                    const float b = prow[32 * pi];
                    acc[0][pi] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b, acc[0][pi], 0, 0, 0);
                    acc[1][pi] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b, acc[1][pi], 0, 0, 0);
                }
            }
            if (more)
                stage(buf ^ 1);         // the other tile: its readers passed the barrier of the previous step
            __syncthreads();
        }
    }

    // ---- epilogue: lane holds column p = .. + lane % 32 and rows q = .. + 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int pi = 0; pi < NP; ++pi) {
        const int p = ptile + pw + pi * 32 + (lane & 31);
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
            base = p;
            qstride = g.P;
        }
        const bool partial = MODE == GEMM_BWD_FILTER || gridDim.z > 1;     // `out` is then the buffer of partial results
        if (partial)
            base += (size_t)blockIdx.z * g.Q * g.P;
#pragma unroll
        for (int qi = 0; qi < 2; ++qi) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int q = qtile + wq * 64 + qi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (q >= g.Q) continue;
                const size_t idx = base + (size_t)q * qstride;
                float v = acc[qi][pi][r];
                if (!partial) {
                    if (beta != 0.0f) v += beta * out[idx];
                    if (MODE == GEMM_FWD && bias) v = bias[q] + v;
                }
                out[idx] = v;
            }
        }
    }
}

// out[i] = sum over the K ranges, in their order, + beta * out[i] (+ bias of element i's channel, NCHW with `plane`
// pixels per channel and O channels)
__global__ __launch_bounds__(256) void conv_f32_reduce_partials_kernel(const float* __restrict__ partial, int splits, size_t n, float beta,
                                                                       float* __restrict__ out, const float* __restrict__ bias, int plane, int O)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        double s = 0.0;
        for (int z = 0; z < splits; ++z) s += (double)partial[(size_t)z * n + i];
        float v = (float)s + (beta != 0.0f ? beta * out[i] : 0.0f);
        if (bias) v = bias[(i / plane) % O] + v;
        out[i] = v;
    }
}

} // namespace n2d2hip
