// Bandwidth-bound cells on NHWC byte tensors: PoolCell (max / truncated
// average) and ElemWiseCell Sum with its activation.  One thread moves 4
// consecutive channels (one dword) per tensor, so that a wavefront touches 256
// contiguous bytes of every operand.
#include <algorithm>

#include "common.h"
#include "epilogue.hpp"

namespace n2d2hip {

__device__ __forceinline__ void unpack4(int x, int zp, int v[4])
{
    v[0] = (int)(signed char)(x) + zp;
    v[1] = (int)(signed char)(x >> 8) + zp;
    v[2] = (int)(signed char)(x >> 16) + zp;
    v[3] = (x >> 24) + zp;
}
__device__ __forceinline__ unsigned pack4(const int v[4])
{
    return ((unsigned)v[0] & 255u) | (((unsigned)v[1] & 255u) << 8) | (((unsigned)v[2] & 255u) << 16) | ((unsigned)v[3] << 24);
}

// ref: src/Cell/PoolCell_Frame_Kernels.cpp:26-197 with the unit mapping PoolCell builds
// (one output per channel).  `flip` = 0x80808080 makes plain U8 bytes comparable as signed.
template <bool IS_MAX>
__global__ __launch_bounds__(256) void pool_kernel(const signed char* __restrict__ in, int cs, int B, int H, int W,
                                                   signed char* __restrict__ out, int OH, int OW, int poolW, int poolH,
                                                   int strideX, int strideY, int padX, int padY, int zp, unsigned flip)
{
    const int cq = cs >> 2;
    const long long total = (long long)B * OH * OW * cq;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
        const int c4 = (int)(idx % cq) * 4;
        long long r = idx / cq;
        const int ox = (int)(r % OW); r /= OW;
        const int oy = (int)(r % OH);
        const int b = (int)(r / OH);
        const int bx = ox * strideX - padX, by = oy * strideY - padY;
        // window limits as the reference clamps them
        const int sxMin = max(-bx, 0), syMin = max(-by, 0);
        const int sxMax = min(max(W - bx, 0), poolW), syMax = min(max(H - by, 0), poolH);
        int acc[4];
        bool valid = false;
        acc[0] = acc[1] = acc[2] = acc[3] = 0;
        for (int sy = syMin; sy < syMax; ++sy) {
            for (int sx = sxMin; sx < sxMax; ++sx) {
                const int xv = *(const int*)(in + (((long long)b * H + by + sy) * W + bx + sx) * cs + c4) ^ (int)flip;
                int v[4];
                unpack4(xv, zp, v);
                if (IS_MAX) {
                    if (!valid) { acc[0] = v[0]; acc[1] = v[1]; acc[2] = v[2]; acc[3] = v[3]; valid = true; }
                    else { acc[0] = max(acc[0], v[0]); acc[1] = max(acc[1], v[1]); acc[2] = max(acc[2], v[2]); acc[3] = max(acc[3], v[3]); }
                } else {
                    acc[0] += v[0]; acc[1] += v[1]; acc[2] += v[2]; acc[3] += v[3];
                }
            }
        }
        if (!IS_MAX) {
            const int count = poolW * poolH;      // countIncludePadding = true
#pragma unroll
            for (int t = 0; t < 4; ++t)
                acc[t] = acc[t] / count;           // C division truncates toward zero, as std::trunc(sum / count)
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[t] -= zp;
        *(unsigned*)(out + idx * 4) = pack4(acc) ^ flip;
    }
}

// Pooling with a connection map (ref: src/Cell/PoolCell_Frame_Kernels.cpp:60-75,150-185): output o pools the window over
// every channel c with maps[o * C + c] set: the largest value met, or the sum divided by window size x connected channels
// and truncated toward zero.  An output without a connected channel, or whose window lies outside the image, is 0.  One
// thread per output value; `bias` turns stored bytes into values (128 for the biased form, 0 otherwise).
template <bool IS_MAX, bool IS_SIGNED>
__global__ __launch_bounds__(256) void pool_mapped_kernel(const signed char* __restrict__ in, int cs, int C, int B, int H, int W,
                                                          const unsigned char* __restrict__ maps, signed char* __restrict__ out,
                                                          int out_cs, int O, int OH, int OW, int poolW, int poolH, int strideX,
                                                          int strideY, int padX, int padY, int bias)
{
    const long long total = (long long)B * OH * OW * out_cs;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
        const int o = (int)(idx % out_cs);
        long long r = idx / out_cs;
        const int ox = (int)(r % OW); r /= OW;
        const int oy = (int)(r % OH);
        const int b = (int)(r / OH);
        int result = 0;
        if (o < O) {
            const int bx = ox * strideX - padX, by = oy * strideY - padY;
            const int sxMin = max(-bx, 0), syMin = max(-by, 0);
            const int sxMax = min(max(W - bx, 0), poolW), syMax = min(max(H - by, 0), poolH);
            int acc = 0, count = 0;
            bool valid = false;
            for (int c = 0; c < C; ++c) {
                if (!maps[(long long)o * C + c])
                    continue;
                for (int sy = syMin; sy < syMax; ++sy)
                    for (int sx = sxMin; sx < sxMax; ++sx) {
                        const signed char raw = in[(((long long)b * H + by + sy) * W + bx + sx) * cs + c];
                        const int v = (IS_SIGNED ? (int)raw : (int)(unsigned char)raw) + bias;
                        if (IS_MAX) {
                            acc = valid ? max(acc, v) : v;
                            valid = true;
                        } else
                            acc += v;
                    }
                count += poolW * poolH;            // countIncludePadding = true
            }
            result = IS_MAX ? acc : (count > 0 ? acc / count : 0);
        }
        out[idx] = (signed char)(result - bias);    // channels between O and the channel stride hold the stored 0
    }
}

// Max pooling with a small compile-time window, 16 channels per thread.  The maximum of signed bytes is taken on the
// packed words themselves: even and odd bytes are moved to the high halves of two 16-bit pairs, where the packed
// 16-bit maximum orders them as bytes.  A tap outside the input is replaced by the nearest tap inside, which cannot
// change a maximum; the host guarantees that every window has one.  Every load of a window is issued before any use.
typedef short v2s __attribute__((ext_vector_type(2)));
template <int PW, int PH>
__global__ __launch_bounds__(256) void pool_max_fast_kernel(const signed char* __restrict__ in, int cs, int B, int H, int W,
                                                            signed char* __restrict__ out, int OH, int OW,
                                                            int strideX, int strideY, int padX, int padY, unsigned flip, int out_halo)
{
    const int cq = cs >> 4;
    const long long total = (long long)B * OH * OW * cq;
    // blocks 8 apart run on the same XCD: give an XCD consecutive logical blocks, so that the rows two neighbouring
    // windows share come out of that XCD's L2 (the grid is a multiple of 8)
    const long long lblock = (long long)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    for (long long idx = lblock * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
        const int c16 = (int)(idx % cq) * 16;
        long long r = idx / cq;
        const int ox = (int)(r % OW); r /= OW;
        const int oy = (int)(r % OH);
        const int b = (int)(r / OH);
        const int bx = ox * strideX - padX, by = oy * strideY - padY;
        const int xlo = max(bx, 0), xhi = min(bx + PW, W) - 1, ylo = max(by, 0), yhi = min(by + PH, H) - 1;
        const signed char* img = in + (long long)b * H * W * cs + c16;
        int4 v[PH][PW];
#pragma unroll
        for (int sy = 0; sy < PH; ++sy) {
            const int iy = min(max(by + sy, ylo), yhi);
#pragma unroll
            for (int sx = 0; sx < PW; ++sx) {
                const int ix = min(max(bx + sx, xlo), xhi);
                v[sy][sx] = *(const int4*)(img + ((long long)iy * W + ix) * cs);
            }
        }
        unsigned res[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v2s me, mo;
#pragma unroll
            for (int sy = 0; sy < PH; ++sy)
#pragma unroll
                for (int sx = 0; sx < PW; ++sx) {
                    const int4 t = v[sy][sx];
                    const unsigned w = (unsigned)(q == 0 ? t.x : q == 1 ? t.y : q == 2 ? t.z : t.w) ^ flip;
                    const unsigned ev = (w << 8) & 0xFF00FF00u, od = w & 0xFF00FF00u;
                    v2s e, o;
                    __builtin_memcpy(&e, &ev, 4);
                    __builtin_memcpy(&o, &od, 4);
                    if (sy == 0 && sx == 0) { me = e; mo = o; }
                    else { me = __builtin_elementwise_max(me, e); mo = __builtin_elementwise_max(mo, o); }
                }
            unsigned ue, uo;
            __builtin_memcpy(&ue, &me, 4);
            __builtin_memcpy(&uo, &mo, 4);
            res[q] = (((ue >> 8) & 0x00FF00FFu) | (uo & 0xFF00FF00u)) ^ flip;
        }
        // an output that carries its readers' padding: the interior of (OH + 2 halo) x (OW + 2 halo) pixels per image
        const long long opix = out_halo ? ((long long)b * (OH + 2 * out_halo) + oy + out_halo) * (OW + 2 * out_halo) + ox + out_halo
                                        : idx / cq;
        *(uint4*)(out + (opix * cq + idx % cq) * 16) = uint4{res[0], res[1], res[2], res[3]};
    }
}

// Global average pooling (the window is the whole input, no padding): a block takes 256 channels of one image, its four
// waves share the pixels and meet in LDS.  Same arithmetic as pool_kernel<false>: integer sum, division truncated
// toward zero (ref: src/Cell/PoolCell_Frame_Kernels.cpp:120-197 followed by the export's std::trunc).
__global__ __launch_bounds__(256) void global_avg_pool_kernel(const signed char* __restrict__ in, int cs, int npix,
                                                              signed char* __restrict__ out, int zp, unsigned flip)
{
    __shared__ int part[4][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slabs = (cs + 255) / 256;
    const int b = blockIdx.x / slabs, c4 = (blockIdx.x % slabs) * 256 + lane * 4;
    int acc[4] = {0, 0, 0, 0};
    if (c4 < cs) {
        const signed char* src = in + (long long)b * npix * cs + c4;
        // the loads of several pixels are issued before the first one is consumed
        int p = wave;
        for (; p + 12 < npix; p += 16) {
            int w[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                w[u] = *(const int*)(src + (long long)(p + 4 * u) * cs);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int v[4];
                unpack4(w[u] ^ (int)flip, zp, v);
                acc[0] += v[0]; acc[1] += v[1]; acc[2] += v[2]; acc[3] += v[3];
            }
        }
        for (; p < npix; p += 4) {
            int v[4];
            unpack4(*(const int*)(src + (long long)p * cs) ^ (int)flip, zp, v);
            acc[0] += v[0]; acc[1] += v[1]; acc[2] += v[2]; acc[3] += v[3];
        }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
        part[wave][lane][t] = acc[t];
    __syncthreads();
    if (wave == 0 && c4 < cs) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[t] = (part[0][lane][t] + part[1][lane][t] + part[2][lane][t] + part[3][lane][t]) / npix - zp;
        *(unsigned*)(out + (long long)b * cs + c4) = pack4(acc) ^ flip;
    }
}

constexpr int EW_MAX_INPUTS = 4;
struct ElemWiseArgs;
int run_elemwise(const ElemWiseArgs& a, bool fcoef, hipStream_t stream);
struct ElemWiseArgs {
    const signed char* in[EW_MAX_INPUTS];
    int zp[EW_MAX_INPUTS];
    unsigned flip[EW_MAX_INPUTS];
    int nb_inputs;
    const float* w;     // [nb_inputs][cpad] coefficient per input and channel
    const float* s;
    int cpad;
    void* out;
    int out_dtype;
    unsigned out_xor;
    int cs;
    long long npix;
    EpiArgs epi;
    int pre_input;      // input that carries a folded ScalingCell (-1: none)
    EpiArgs pre;        // its Scaling (EPI_I24 tables), applied to the input before the sum
};

// ref: src/Cell/ElemWiseCell_Frame.cpp:116-136 (Sum) followed by the cell's activation; with one input and unit
// coefficients it is ScalingCell_Frame::propagate (ref: src/Cell/ScalingCell_Frame.cpp:67-75).
// FCOEF: float32 arithmetic in the reference's order, products and sums rounded individually (no fused
// multiply-add).  !FCOEF: all weights are 1 and all shifts 0, the sum is formed in int32 (the same value: every
// float operation of the reference is exact on these operands).
// HOIST: the launch makes the grid stride a multiple of the dwords per pixel, so a thread keeps its 4 channels
// and loads their table rows once.
// PRE: one input is rescaled on the fly by the ScalingCell folded into this cell.
template <int KIND, bool FCOEF, bool HOIST, bool PRE>
__global__ __launch_bounds__(256) void elemwise_sum_kernel(ElemWiseArgs p)
{
    const int cq = p.cs >> 2;
    const long long total = p.npix * cq;
    const long long stride = (long long)gridDim.x * blockDim.x;
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    int c4 = (int)(idx % cq) * 4;
    int4 ta = {0, 0, 0, 0}, tb = ta, tc = ta, td = ta, te = ta;
    int4 pa = ta, pb = ta, pc = ta, pd = ta, pe = ta;
    auto load_tables = [&](int c) {
        if (PRE) {
            pa = *(const int4*)(p.pre.a + c);
            pb = *(const int4*)(p.pre.b + c);
            pc = *(const int4*)(p.pre.c + c);
            pd = *(const int4*)(p.pre.d + c);
            pe = *(const int4*)(p.pre.e + c);
        }
        if (KIND != EPI_RAW) {
            ta = *(const int4*)(p.epi.a + c);
            tb = *(const int4*)(p.epi.b + c);
            tc = *(const int4*)(p.epi.c + c);
            if (KIND == EPI_I24) td = *(const int4*)(p.epi.d + c);
            if (KIND != EPI_F32) te = *(const int4*)(p.epi.e + c);
        }
    };
    if (HOIST) load_tables(c4);
#pragma unroll 4
    for (; idx < total; idx += stride) {
        if (!HOIST) {
            c4 = (int)(idx % cq) * 4;
            load_tables(c4);
        }
        int r[4];
        if (FCOEF) {
            float o[4];
            {
                int v[4];
                unpack4(*(const int*)(p.in[0] + idx * 4) ^ (int)p.flip[0], p.zp[0], v);
                const float4 w = *(const float4*)(p.w + c4), s = *(const float4*)(p.s + c4);
                o[0] = __fadd_rn(__fmul_rn(w.x, (float)v[0]), s.x);
                o[1] = __fadd_rn(__fmul_rn(w.y, (float)v[1]), s.y);
                o[2] = __fadd_rn(__fmul_rn(w.z, (float)v[2]), s.z);
                o[3] = __fadd_rn(__fmul_rn(w.w, (float)v[3]), s.w);
            }
            for (int k = 1; k < p.nb_inputs; ++k) {
                int v[4];
                unpack4(*(const int*)(p.in[k] + idx * 4) ^ (int)p.flip[k], p.zp[k], v);
                const float4 w = *(const float4*)(p.w + (long long)k * p.cpad + c4), s = *(const float4*)(p.s + (long long)k * p.cpad + c4);
                o[0] = __fadd_rn(o[0], __fadd_rn(__fmul_rn(w.x, (float)v[0]), s.x));
                o[1] = __fadd_rn(o[1], __fadd_rn(__fmul_rn(w.y, (float)v[1]), s.y));
                o[2] = __fadd_rn(o[2], __fadd_rn(__fmul_rn(w.z, (float)v[2]), s.z));
                o[3] = __fadd_rn(o[3], __fadd_rn(__fmul_rn(w.w, (float)v[3]), s.w));
            }
            if (KIND == EPI_F32) {
                const int a4[4] = {ta.x, ta.y, ta.z, ta.w}, b4[4] = {tb.x, tb.y, tb.z, tb.w}, c4v[4] = {tc.x, tc.y, tc.z, tc.w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    float f = fminf(fmaxf(o[t], as_f32(a4[t])), as_f32(b4[t]));
                    f = round_half_away(__fmul_rn(f, as_f32(c4v[t])));
                    r[t] = (int)fminf(fmaxf(f, (float)p.epi.lo), (float)p.epi.hi);
                }
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    r[t] = (int)fminf(fmaxf(round_half_away(o[t]), -2147483520.0f), 2147483520.0f);   // round(realInput)
            }
        } else {
            auto prescale = [&](int v[4]) {
                v[0] = epi_apply<EPI_I24>(v[0], pa.x, pb.x, pc.x, pd.x, pe.x, p.pre.lo, p.pre.hi, 0);
                v[1] = epi_apply<EPI_I24>(v[1], pa.y, pb.y, pc.y, pd.y, pe.y, p.pre.lo, p.pre.hi, 0);
                v[2] = epi_apply<EPI_I24>(v[2], pa.z, pb.z, pc.z, pd.z, pe.z, p.pre.lo, p.pre.hi, 0);
                v[3] = epi_apply<EPI_I24>(v[3], pa.w, pb.w, pc.w, pd.w, pe.w, p.pre.lo, p.pre.hi, 0);
            };
            unpack4(*(const int*)(p.in[0] + idx * 4) ^ (int)p.flip[0], p.zp[0], r);
            if (PRE && p.pre_input == 0) prescale(r);
            for (int k = 1; k < p.nb_inputs; ++k) {
                int v[4];
                unpack4(*(const int*)(p.in[k] + idx * 4) ^ (int)p.flip[k], p.zp[k], v);
                if (PRE && p.pre_input == k) prescale(v);
                r[0] += v[0]; r[1] += v[1]; r[2] += v[2]; r[3] += v[3];
            }
        }
        if (!(FCOEF && KIND == EPI_F32)) {
            r[0] = epi_apply<KIND>(r[0], ta.x, tb.x, tc.x, td.x, te.x, p.epi.lo, p.epi.hi, p.epi.relu);
            r[1] = epi_apply<KIND>(r[1], ta.y, tb.y, tc.y, td.y, te.y, p.epi.lo, p.epi.hi, p.epi.relu);
            r[2] = epi_apply<KIND>(r[2], ta.z, tb.z, tc.z, td.z, te.z, p.epi.lo, p.epi.hi, p.epi.relu);
            r[3] = epi_apply<KIND>(r[3], ta.w, tb.w, tc.w, td.w, te.w, p.epi.lo, p.epi.hi, p.epi.relu);
        }
        if (p.out_dtype == N2D2HIP_I32)
            *(int4*)((int*)p.out + idx * 4) = int4{r[0], r[1], r[2], r[3]};
        else
            *(unsigned*)((signed char*)p.out + idx * 4) = pack4(r) ^ p.out_xor;
    }
}

template <bool FCOEF, bool HOIST, bool PRE>
static void launch_elemwise(const ElemWiseArgs& a, unsigned grid, hipStream_t stream)
{
    switch (a.epi.kind) {
    case EPI_RAW: N2D2HIP_LAUNCH_T(elemwise_sum_kernel, (EPI_RAW, FCOEF, HOIST, PRE), dim3(grid), dim3(256), 0, stream, a); break;
    case EPI_I24: N2D2HIP_LAUNCH_T(elemwise_sum_kernel, (EPI_I24, FCOEF, HOIST, PRE), dim3(grid), dim3(256), 0, stream, a); break;
    case EPI_I64: N2D2HIP_LAUNCH_T(elemwise_sum_kernel, (EPI_I64, FCOEF, HOIST, PRE), dim3(grid), dim3(256), 0, stream, a); break;
    default: N2D2HIP_LAUNCH_T(elemwise_sum_kernel, (EPI_F32, FCOEF, HOIST, PRE), dim3(grid), dim3(256), 0, stream, a); break;
    }
}

// Launches the sum / rescale kernel over NHWC byte tensors described by `a`.
int run_elemwise(const ElemWiseArgs& a, bool fcoef, hipStream_t stream)
{
    const int cq = a.cs >> 2;
    const long long total = a.npix * cq;
    long long want = std::max<long long>(1, std::min<long long>((total + 1023) / 1024, 256 * 16));   // ~4 dwords per thread and pass
    // grid stride (grid*256) must be a multiple of cq for the hoisted form
    int g = cq, b = 256;
    while (b) { const int t = g % b; g = b; b = t; }
    const long long unit = cq / g;                // grid must be a multiple of this
    bool hoist = unit <= want;
    unsigned grid = (unsigned)(hoist ? (want / unit) * unit : want);
    const bool pre = a.pre_input >= 0;
    if (fcoef) { if (hoist) launch_elemwise<true, true, false>(a, grid, stream); else launch_elemwise<true, false, false>(a, grid, stream); }
    else if (pre) { if (hoist) launch_elemwise<false, true, true>(a, grid, stream); else launch_elemwise<false, false, true>(a, grid, stream); }
    else { if (hoist) launch_elemwise<false, true, false>(a, grid, stream); else launch_elemwise<false, false, false>(a, grid, stream); }
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

// ScalingCell on an NHWC byte tensor: the one-input, unit-coefficient case of the kernel above.
int run_scaling_nhwc(const n2d2hip_act_s* act, const n2d2hip_tensor* in, const n2d2hip_tensor* out, hipStream_t stream)
{
    ElemWiseArgs a = {};
    a.in[0] = (const signed char*)in->data;
    a.flip[0] = in->dtype == N2D2HIP_U8 ? 0x80808080u : 0u;
    a.zp[0] = in->dtype == N2D2HIP_I8 ? 0 : 128;
    a.nb_inputs = 1;
    a.pre_input = -1;
    a.out = out->data;
    a.out_dtype = out->dtype;
    a.out_xor = out->dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    a.cs = out->cs;
    a.npix = (long long)out->B * out->H * out->W;
    a.epi = act->args;
    return run_elemwise(a, false, stream);
}

// ---------------------------------------------------------------- channel concatenation
// A cell with several inputs sees their channels one behind the other (ref: src/Cell/ConvCell_Frame.cpp:438-459: the
// weighted sums of the inputs are added up, each input with its own slice of the weights, which is the convolution of the
// concatenated channels).  One thread per pixel and group of 4 output channels; inputs may carry a halo (read past it).
constexpr int CONCAT_MAX = 8;
struct ConcatArgs {
    const signed char* in[CONCAT_MAX];
    int cs[CONCAT_MAX], halo[CONCAT_MAX];
    int first[CONCAT_MAX + 1];      // first output channel of each input; first[n] = all channels
    int n;
    signed char* out;
    int out_cs, out_halo;
    int B, H, W;
    unsigned fill;                  // storage form of 0, for the channels past the last one
};

__global__ __launch_bounds__(256) void concat_channels_kernel(ConcatArgs p)
{
    const int cq = p.out_cs >> 2;
    const long long total = (long long)p.B * p.H * p.W * cq;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int g = (int)(idx % cq);
        const long long pix = idx / cq;
        const int x = (int)(pix % p.W), y = (int)((pix / p.W) % p.H), b = (int)(pix / ((long long)p.W * p.H));
        unsigned v = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = 4 * g + j;
            unsigned byte = p.fill;
#pragma unroll
            for (int k = 0; k < CONCAT_MAX; ++k) {
                if (k < p.n && c >= p.first[k] && c < p.first[k + 1]) {
                    const int h = p.halo[k];
                    const long long at = (((long long)b * (p.H + 2 * h) + y + h) * (p.W + 2 * h) + x + h) * p.cs[k] + (c - p.first[k]);
                    byte = (unsigned char)p.in[k][at];
                }
            }
            v |= (byte & 0xffu) << (8 * j);
        }
        const int ho = p.out_halo;
        const long long at = (((long long)b * (p.H + 2 * ho) + y + ho) * (p.W + 2 * ho) + x + ho) * p.out_cs + 4 * g;
        *(unsigned*)(p.out + at) = v;
    }
}

} // namespace n2d2hip

using namespace n2d2hip;

extern "C" {

int n2d2hip_pool_out_dims(const n2d2hip_pool_desc* d, int H, int W, int* outH, int* outW)
{
    N2D2HIP_REQUIRE(d && outH && outW, N2D2HIP_ERR_INVALID, "pool_out_dims: null argument");
    N2D2HIP_REQUIRE(d->poolW > 0 && d->poolH > 0 && d->strideX > 0 && d->strideY > 0 && d->padX >= 0 && d->padY >= 0,
                    N2D2HIP_ERR_INVALID, "pool_out_dims: bad descriptor");
    // ref: src/Cell/PoolCell.cpp:219-240
    *outW = (int)((W + 2 * d->padX - d->poolW + d->strideX) / (double)d->strideX);
    *outH = (int)((H + 2 * d->padY - d->poolH + d->strideY) / (double)d->strideY);
    N2D2HIP_REQUIRE(*outW > 0 && *outH > 0, N2D2HIP_ERR_INVALID, "pool_out_dims: empty output");
    return N2D2HIP_OK;
}

// windows that all hold at least one input element, square 2x2 or 3x3, 16-byte channel groups: the kernel that may write
// its output with a border
static bool pool_fast(const n2d2hip_pool_desc* d, int H, int W, int cs, int OH, int OW)
{
    return d->pooling == N2D2HIP_POOL_MAX && cs % 16 == 0 && d->poolW == d->poolH && (d->poolW == 2 || d->poolW == 3)
        && d->padX < d->poolW && d->padY < d->poolH && (OW - 1) * d->strideX - d->padX < W && (OH - 1) * d->strideY - d->padY < H;
}

int n2d2hip_pool_writes_halo(const n2d2hip_pool_desc* d, int H, int W, int cs)
{
    int OH, OW;
    if (!d || n2d2hip_pool_out_dims(d, H, W, &OH, &OW) != N2D2HIP_OK)
        return 0;
    return pool_fast(d, H, W, cs, OH, OW) ? 1 : 0;
}

int n2d2hip_pool_forward(const n2d2hip_pool_desc* d, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc, OH, OW;
    N2D2HIP_REQUIRE(d != nullptr, N2D2HIP_ERR_INVALID, "pool_forward: null descriptor");
    N2D2HIP_REQUIRE(d->pooling == N2D2HIP_POOL_MAX || d->pooling == N2D2HIP_POOL_AVERAGE, N2D2HIP_ERR_INVALID, "pool_forward: bad pooling %d", d->pooling);
    if ((rc = check_tensor(in, "pool input")) || (rc = check_tensor(out, "pool output", true)) || (rc = n2d2hip_pool_out_dims(d, in->H, in->W, &OH, &OW)))
        return rc;
    N2D2HIP_REQUIRE(in->layout == N2D2HIP_NHWC && out->layout == N2D2HIP_NHWC, N2D2HIP_ERR_UNSUPPORTED, "pool_forward: tensors must be NHWC");
    N2D2HIP_REQUIRE(is_byte_type(in->dtype) && out->dtype == in->dtype, N2D2HIP_ERR_INVALID, "pool_forward: byte tensors of one dtype expected");
    N2D2HIP_REQUIRE(out->B == in->B && out->C == in->C && out->H == OH && out->W == OW && out->cs == in->cs, N2D2HIP_ERR_INVALID,
                    "pool_forward: output is %dx%dx%dx%d (cs %d), expected %dx%dx%dx%d (cs %d)", out->B, out->C, out->H, out->W, out->cs,
                    in->B, in->C, OH, OW, in->cs);
    const long long total = (long long)in->B * OH * OW * (in->cs / 4);
    const unsigned grid = (unsigned)std::max<long long>(1, std::min<long long>((total + 255) / 256, 256 * 64));
    const unsigned flip = in->dtype == N2D2HIP_U8 ? 0x80808080u : 0u;
    const int zp = in->dtype == N2D2HIP_I8 ? 0 : 128;      // after the flip, U8 bytes read as value-128 too
    const bool fast = pool_fast(d, in->H, in->W, in->cs, OH, OW);
    N2D2HIP_REQUIRE(out->halo == 0 || fast, N2D2HIP_ERR_UNSUPPORTED,
                    "pool_forward: only the 2x2 / 3x3 max pooling of 16-byte channel groups writes an output with a halo");
    if (d->pooling == N2D2HIP_POOL_AVERAGE && OH == 1 && OW == 1 && d->poolW == in->W && d->poolH == in->H && d->padX == 0 && d->padY == 0) {
        const int slabs = (in->cs + 255) / 256;
        N2D2HIP_LAUNCH(global_avg_pool_kernel, dim3((unsigned)(in->B * slabs)), dim3(256), 0, (hipStream_t)stream,
                           (const signed char*)in->data, in->cs, in->H * in->W, (signed char*)out->data, zp, flip);
    } else if (fast) {
        const long long total16 = (long long)in->B * OH * OW * (in->cs / 16);
        const unsigned g16 = (unsigned)round_up((int)std::max<long long>(1, std::min<long long>((total16 + 255) / 256, 256 * 64)), 8);
        if (d->poolW == 3)
            N2D2HIP_LAUNCH_T(pool_max_fast_kernel, (3, 3), dim3(g16), dim3(256), 0, (hipStream_t)stream, (const signed char*)in->data, in->cs,
                               in->B, in->H, in->W, (signed char*)out->data, OH, OW, d->strideX, d->strideY, d->padX, d->padY, flip, out->halo);
        else
            N2D2HIP_LAUNCH_T(pool_max_fast_kernel, (2, 2), dim3(g16), dim3(256), 0, (hipStream_t)stream, (const signed char*)in->data, in->cs,
                               in->B, in->H, in->W, (signed char*)out->data, OH, OW, d->strideX, d->strideY, d->padX, d->padY, flip, out->halo);
    } else if (d->pooling == N2D2HIP_POOL_MAX)
        N2D2HIP_LAUNCH_T(pool_kernel, (true), dim3(grid), dim3(256), 0, (hipStream_t)stream, (const signed char*)in->data, in->cs, in->B, in->H,
                           in->W, (signed char*)out->data, OH, OW, d->poolW, d->poolH, d->strideX, d->strideY, d->padX, d->padY, zp, flip);
    else
        N2D2HIP_LAUNCH_T(pool_kernel, (false), dim3(grid), dim3(256), 0, (hipStream_t)stream, (const signed char*)in->data, in->cs, in->B, in->H,
                           in->W, (signed char*)out->data, OH, OW, d->poolW, d->poolH, d->strideX, d->strideY, d->padX, d->padY, zp, flip);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_pool_forward_mapped(const n2d2hip_pool_desc* d, const unsigned char* maps, int map_outputs, int map_channels,
                                const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc, OH, OW;
    N2D2HIP_REQUIRE(d != nullptr && maps != nullptr, N2D2HIP_ERR_INVALID, "pool_forward_mapped: null descriptor or map");
    // the kernel reads maps[o * in->C + c] for every output and channel of the tensors: the map must have been built for them
    N2D2HIP_REQUIRE(in != nullptr && out != nullptr && map_outputs == out->C && map_channels == in->C, N2D2HIP_ERR_INVALID,
                    "pool_forward_mapped: the map is %d outputs x %d channels, the tensors have %d outputs and %d channels", map_outputs,
                    map_channels, out ? out->C : 0, in ? in->C : 0);
    N2D2HIP_REQUIRE(d->pooling == N2D2HIP_POOL_MAX || d->pooling == N2D2HIP_POOL_AVERAGE, N2D2HIP_ERR_INVALID, "pool_forward_mapped: bad pooling %d", d->pooling);
    if ((rc = check_tensor(in, "pool input")) || (rc = check_tensor(out, "pool output")) || (rc = n2d2hip_pool_out_dims(d, in->H, in->W, &OH, &OW)))
        return rc;
    N2D2HIP_REQUIRE(in->layout == N2D2HIP_NHWC && out->layout == N2D2HIP_NHWC, N2D2HIP_ERR_UNSUPPORTED, "pool_forward_mapped: tensors must be NHWC");
    N2D2HIP_REQUIRE(is_byte_type(in->dtype) && out->dtype == in->dtype, N2D2HIP_ERR_INVALID, "pool_forward_mapped: byte tensors of one dtype expected");
    N2D2HIP_REQUIRE(out->B == in->B && out->H == OH && out->W == OW, N2D2HIP_ERR_INVALID,
                    "pool_forward_mapped: output is %dx%dx%dx%d, expected %dxOx%dx%d", out->B, out->C, out->H, out->W, in->B, OH, OW);
    const long long total = (long long)in->B * OH * OW * out->cs;
    const unsigned grid = (unsigned)std::max<long long>(1, std::min<long long>((total + 255) / 256, 256 * 64));
    const int bias = in->dtype == N2D2HIP_U8B ? 128 : 0;
#define N2D2HIP_POOL_MAPPED(IS_MAX, IS_SIGNED)                                                                                      \
    N2D2HIP_LAUNCH_T(pool_mapped_kernel, (IS_MAX, IS_SIGNED), dim3(grid), dim3(256), 0, (hipStream_t)stream,                       \
                       (const signed char*)in->data, in->cs, in->C, in->B, in->H, in->W, maps, (signed char*)out->data, out->cs,     \
                       out->C, OH, OW, d->poolW, d->poolH, d->strideX, d->strideY, d->padX, d->padY, bias)
    const bool is_signed = in->dtype != N2D2HIP_U8;
    if (d->pooling == N2D2HIP_POOL_MAX) {
        if (is_signed) N2D2HIP_POOL_MAPPED(true, true); else N2D2HIP_POOL_MAPPED(true, false);
    } else {
        if (is_signed) N2D2HIP_POOL_MAPPED(false, true); else N2D2HIP_POOL_MAPPED(false, false);
    }
#undef N2D2HIP_POOL_MAPPED
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_elemwise_create(int nb_inputs, int nb_channels, int coeff_mode, const float* weights, const float* shifts,
                            n2d2hip_act_t act, n2d2hip_elemwise_t* ew)
{
    N2D2HIP_REQUIRE(act && ew, N2D2HIP_ERR_INVALID, "elemwise_create: null argument");
    N2D2HIP_REQUIRE(nb_inputs >= 1 && nb_inputs <= EW_MAX_INPUTS, N2D2HIP_ERR_UNSUPPORTED, "elemwise_create: %d inputs (1..%d)", nb_inputs, EW_MAX_INPUTS);
    N2D2HIP_REQUIRE(coeff_mode >= N2D2HIP_COEFF_PER_LAYER && coeff_mode <= N2D2HIP_COEFF_PER_CHANNEL, N2D2HIP_ERR_INVALID, "elemwise_create: bad coeff mode");
    N2D2HIP_REQUIRE(act->nb_channels == nb_channels, N2D2HIP_ERR_INVALID, "elemwise_create: activation built for %d channels, cell has %d", act->nb_channels, nb_channels);
    const int cpad = act->cpad;
    std::vector<float> h(2 * (size_t)nb_inputs * cpad);
    float* hw = h.data();
    float* hs = hw + (size_t)nb_inputs * cpad;
    for (int k = 0; k < nb_inputs; ++k)
        for (int c = 0; c < cpad; ++c) {
            const int cc = c < nb_channels ? c : nb_channels - 1;
            // ref: src/Cell/ElemWiseCell_Frame.cpp:121-130: input 0 uses index c0 (= channel when
            // PerChannel, else 0); input k >= 1 uses c0 when PerChannel, else k.
            const int c0 = coeff_mode == N2D2HIP_COEFF_PER_CHANNEL ? cc : 0;
            const int idx = (k == 0) ? c0 : (coeff_mode == N2D2HIP_COEFF_PER_CHANNEL ? c0 : k);
            hw[(size_t)k * cpad + c] = weights ? weights[idx] : 1.0f;
            hs[(size_t)k * cpad + c] = shifts ? shifts[idx] : 0.0f;
        }
    n2d2hip_elemwise_s* e = new n2d2hip_elemwise_s();
    e->unit_coeff = true;
    for (size_t i = 0; i < (size_t)nb_inputs * cpad; ++i)
        if (hw[i] != 1.0f || hs[i] != 0.0f) e->unit_coeff = false;
    e->pre_input = -1; e->pre_act = nullptr;
    e->nb_inputs = nb_inputs; e->nb_channels = nb_channels; e->cpad = cpad; e->act = act; e->d_coeff = nullptr;
    hipError_t herr = hipMalloc((void**)&e->d_coeff, h.size() * sizeof(float));
    if (herr == hipSuccess) herr = hipMemcpy(e->d_coeff, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice);
    if (herr != hipSuccess) {
        n2d2hip_elemwise_destroy(e);
        return fail(N2D2HIP_ERR_HIP, "elemwise_create: device upload failed: %s", hipGetErrorString(herr));
    }
    *ew = e;
    return N2D2HIP_OK;
}

int n2d2hip_elemwise_fold_input_scaling(n2d2hip_elemwise_t ew, int input_index, n2d2hip_act_t scaling)
{
    N2D2HIP_REQUIRE(ew != nullptr, N2D2HIP_ERR_INVALID, "elemwise_fold_input_scaling: null cell");
    if (!scaling) { ew->pre_input = -1; ew->pre_act = nullptr; return N2D2HIP_OK; }
    N2D2HIP_REQUIRE(input_index >= 0 && input_index < ew->nb_inputs, N2D2HIP_ERR_INVALID, "elemwise_fold_input_scaling: input %d of %d", input_index, ew->nb_inputs);
    N2D2HIP_REQUIRE(scaling->nb_channels == ew->nb_channels, N2D2HIP_ERR_INVALID, "elemwise_fold_input_scaling: channel count mismatch");
    N2D2HIP_REQUIRE(ew->unit_coeff && scaling->args.kind == EPI_I24 && scaling->min_out >= -128 && scaling->max_out <= 255, N2D2HIP_ERR_UNSUPPORTED,
                    "elemwise_fold_input_scaling: only an integer Scaling in front of a unit-coefficient sum can be folded");
    ew->pre_input = input_index;
    ew->pre_act = scaling;
    return N2D2HIP_OK;
}

int n2d2hip_elemwise_destroy(n2d2hip_elemwise_t ew)
{
    if (!ew) return N2D2HIP_OK;
    if (ew->d_coeff) (void)hipFree(ew->d_coeff);
    delete ew;
    return N2D2HIP_OK;
}

int n2d2hip_elemwise_forward(n2d2hip_elemwise_t ew, const n2d2hip_tensor* const* inputs, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc;
    N2D2HIP_REQUIRE(ew && inputs, N2D2HIP_ERR_INVALID, "elemwise_forward: null argument");
    if ((rc = check_tensor(out, "elemwise output")))
        return rc;
    N2D2HIP_REQUIRE(out->layout == N2D2HIP_NHWC && out->C == ew->nb_channels, N2D2HIP_ERR_INVALID, "elemwise_forward: NHWC output with %d channels expected", ew->nb_channels);
    ElemWiseArgs a = {};
    for (int k = 0; k < ew->nb_inputs; ++k) {
        const n2d2hip_tensor* t = inputs[k];
        if ((rc = check_tensor(t, "elemwise input")))
            return rc;
        N2D2HIP_REQUIRE(t->layout == N2D2HIP_NHWC && is_byte_type(t->dtype), N2D2HIP_ERR_UNSUPPORTED, "elemwise_forward: inputs must be NHWC byte tensors");
        N2D2HIP_REQUIRE(t->B == out->B && t->C == out->C && t->H == out->H && t->W == out->W && t->cs == out->cs, N2D2HIP_ERR_INVALID,
                        "elemwise_forward: input %d shape differs from the output", k);
        a.in[k] = (const signed char*)t->data;
        a.flip[k] = t->dtype == N2D2HIP_U8 ? 0x80808080u : 0u;
        a.zp[k] = t->dtype == N2D2HIP_I8 ? 0 : 128;
    }
    const n2d2hip_act_s* act = ew->act;
    if (is_byte_type(out->dtype)) {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(act->min_out >= lo && act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "elemwise_forward: activation range [%d,%d] does not fit output dtype %d", act->min_out, act->max_out, out->dtype);
    } else {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_UNSUPPORTED, "elemwise_forward: output must be a byte type or I32");
    }
    a.nb_inputs = ew->nb_inputs;
    a.pre_input = ew->pre_input;
    if (ew->pre_input >= 0) a.pre = ew->pre_act->args;
    a.w = ew->d_coeff;
    a.s = ew->d_coeff + (size_t)ew->nb_inputs * ew->cpad;
    a.cpad = ew->cpad;
    a.out = out->data;
    a.out_dtype = out->dtype;
    a.out_xor = out->dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    a.cs = out->cs;
    a.npix = (long long)out->B * out->H * out->W;
    a.epi = act->args;
    // EPI_RAW on float coefficients would emit non-integers: only the integer form is defined there
    if (act->args.kind == EPI_RAW)
        N2D2HIP_REQUIRE(ew->unit_coeff, N2D2HIP_ERR_UNSUPPORTED, "elemwise_forward: non-unit coefficients need a rescaling activation");
    return run_elemwise(a, !ew->unit_coeff, (hipStream_t)stream);
}

int n2d2hip_concat_channels(int nb_inputs, const n2d2hip_tensor* const* inputs, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc;
    N2D2HIP_REQUIRE(inputs != nullptr && nb_inputs >= 1 && nb_inputs <= CONCAT_MAX, N2D2HIP_ERR_INVALID,
                    "concat_channels: %d inputs (1 to %d)", nb_inputs, CONCAT_MAX);
    if ((rc = check_tensor(out, "concat output", true)))
        return rc;
    N2D2HIP_REQUIRE(out->layout == N2D2HIP_NHWC && is_byte_type(out->dtype), N2D2HIP_ERR_UNSUPPORTED, "concat_channels: NHWC byte tensors");
    ConcatArgs a = {};
    int channels = 0;
    for (int k = 0; k < nb_inputs; ++k) {
        const n2d2hip_tensor* t = inputs[k];
        if ((rc = check_tensor(t, "concat input", true)))
            return rc;
        N2D2HIP_REQUIRE(t->layout == N2D2HIP_NHWC && t->dtype == out->dtype, N2D2HIP_ERR_INVALID,
                        "concat_channels: input %d has dtype %d, the output %d (one byte type for all, NHWC)", k, t->dtype, out->dtype);
        N2D2HIP_REQUIRE(t->B == out->B && t->H == out->H && t->W == out->W, N2D2HIP_ERR_INVALID,
                        "concat_channels: input %d is %dx%dx%d, the output %dx%dx%d", k, t->B, t->H, t->W, out->B, out->H, out->W);
        a.in[k] = (const signed char*)t->data;
        a.cs[k] = t->cs;
        a.halo[k] = t->halo;
        a.first[k] = channels;
        channels += t->C;
    }
    N2D2HIP_REQUIRE(channels == out->C, N2D2HIP_ERR_INVALID, "concat_channels: the inputs hold %d channels, the output %d", channels, out->C);
    a.first[nb_inputs] = channels;
    a.n = nb_inputs;
    a.out = (signed char*)out->data;
    a.out_cs = out->cs;
    a.out_halo = out->halo;
    a.B = out->B; a.H = out->H; a.W = out->W;
    a.fill = out->dtype == N2D2HIP_U8B ? 0x80u : 0u;
    const long long total = (long long)out->B * out->H * out->W * (out->cs / 4);
    const unsigned grid = (unsigned)std::max<long long>(1, std::min<long long>((total + 255) / 256, 256 * 64));
    N2D2HIP_LAUNCH(concat_channels_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, a);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
