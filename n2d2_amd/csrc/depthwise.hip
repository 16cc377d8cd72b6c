// 3x3 depthwise convolution on NHWC bytes: groups == C == O, so there is no reduction over channels and no matrix core:
// the layer is bound by memory traffic and, behind it, by the vector ALU
// (ref: src/Cell/ConvCell_Frame_Kernels.cpp:26-179 with one channel per group).
//
// A thread owns 4 consecutive channels (one dword) of one output column and walks down a strip of output rows, so
// consecutive lanes read and write consecutive bytes.  Each input row it meets is loaded once as the three pixels left,
// middle and right of the column and transposed into four dwords, one per channel, of (left, middle, right, 0); every
// output row that uses the input row then needs one 4-way dot product per channel against (w[ky][0], w[ky][1], w[ky][2], 0).
// Taps outside the image read the stored form of 0, which lets the input's zero point live in the bias.
#include "depthwise.hpp"
#include "depthwise_math.hpp"
#include "epilogue.hpp"
#include "mfma_util.hpp"

namespace n2d2hip {

namespace {

// FAST (KIND == EPI_I24 only): the rescale is (v * c + d) >> e with the bias inside d, saturated to [0, 255] while packing.
template <int S, int KIND, bool FAST = false>
__global__ __launch_bounds__(256) void depthwise3x3_kernel(const DepthwiseArgs p)
{
    // Work-groups 8 apart run on the same XCD (they are dealt to the 8 XCDs in turn): a work-group's place in the tensor is
    // chosen so that each XCD walks one contiguous eighth of it, and the columns and rows that neighbouring work-groups
    // both read come out of that XCD's L2 instead of being fetched from memory once per XCD.
    const unsigned per_xcd = gridDim.x >> 3;
    const unsigned idx = ((blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3)) * 256u + threadIdx.x;
    if (idx >= p.nthreads)
        return;
    const unsigned cg = idx % p.cq;
    unsigned r = idx / p.cq;
    const int ox = (int)(r % (unsigned)p.OW);
    r /= (unsigned)p.OW;
    const int strip = (int)(r % (unsigned)p.nstrips);
    const int b = (int)(r / (unsigned)p.nstrips);
    const int c4 = (int)cg * 4;
    const int oy0 = strip * p.rows;
    const int nrows = min(p.rows, p.OH - oy0);

    int4 w0 = *(const int4*)(p.wb + c4);
    int4 w1 = *(const int4*)(p.wb + p.cs + c4);
    int4 w2 = *(const int4*)(p.wb + 2 * p.cs + c4);
    int4 bias = {};
    if (!FAST)
        bias = *(const int4*)(p.wb + 3 * p.cs + c4);
    int4 ta = {}, tb = {}, tc = {}, td = {}, te = {};
    if (FAST) {
        tc = *(const int4*)(p.fc + c4);
        td = *(const int4*)(p.fd + c4);
        te = *(const int4*)(p.fe + c4);
    } else if (KIND == EPI_I24 || KIND == EPI_I64) {
        ta = *(const int4*)(p.epi.a + c4);
        tb = *(const int4*)(p.epi.b + c4);
        tc = *(const int4*)(p.epi.c + c4);
        td = *(const int4*)(p.epi.d + c4);
        te = *(const int4*)(p.epi.e + c4);
    }

    const int ix0 = ox * S - p.padL;
    const bool vm = ix0 >= 0 && ix0 < p.W, v0 = ix0 + 1 >= 0 && ix0 + 1 < p.W, vp = ix0 + 2 >= 0 && ix0 + 2 < p.W;
    const unsigned fill = p.fill;
    // Every load is issued whatever the position (no branches in the loop): a tap outside the image reads the nearest pixel
    // inside and is replaced by the stored form of 0 afterwards.
    const signed char* img = p.in + (long long)b * p.H * p.W * p.cs + c4;
    const int om = min(max(ix0, 0), p.W - 1) * p.cs, oc = min(max(ix0 + 1, 0), p.W - 1) * p.cs, op = min(max(ix0 + 2, 0), p.W - 1) * p.cs;
    const long long row_bytes = (long long)p.W * p.cs;
    // an input row as loaded (left, middle, right pixel)
    struct Raw3 { unsigned m, c, p; };
    typedef const unsigned __attribute__((address_space(1))) * GlobalWord;
    // fetch_row only issues the loads; settle_row, called where the values are used, puts the stored form of 0 in place of
    // the taps outside the image (a select on a loaded value waits for it).
    auto fetch_row = [&](int iy) -> Raw3 {
        const signed char* rp = img + min(max(iy, 0), p.H - 1) * row_bytes;
        Raw3 r;
        r.m = *(GlobalWord)(rp + om);
        r.c = *(GlobalWord)(rp + oc);
        r.p = *(GlobalWord)(rp + op);
        return r;
    };
    auto settle_row = [&](const Raw3& r, int iy) -> Row4 {
        const bool row_ok = iy >= 0 && iy < p.H;
        return transpose3((row_ok && vm) ? r.m : fill, (row_ok && v0) ? r.c : fill, (row_ok && vp) ? r.p : fill);
    };
    auto load_row = [&](int iy) -> Row4 {
        return settle_row(fetch_row(iy), iy);
    };
    auto finish = [&](int v, int ch, int a, int bq, int c, int d, int e) -> int {
        if (KIND == EPI_I24 || KIND == EPI_I64)
            return epi_apply<KIND>(v, a, bq, c, d, e, p.epi.lo, p.epi.hi, 0);
        return epi_apply_dyn(p.epi, v, c4 + ch);
    };
    unsigned* outp = (unsigned*)((signed char*)p.out + (((long long)b * p.OH + oy0) * p.OW + ox) * p.cs + c4);
    const long long out_row = (long long)p.OW * p.cs / 4;

    const int iy0 = oy0 * S - p.padT;
    Row4 t0 = load_row(iy0);
    Row4 t1 = {};
    if (S == 1)
        t1 = load_row(iy0 + 1);
    // The per-channel tables were requested before the first rows and so have arrived by now; saying so here keeps the
    // loop free of waits for them (such a wait would also wait for the rows requested ahead).
#define N2D2HIP_DW_ARRIVED(v) asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w))
    N2D2HIP_DW_ARRIVED(w0); N2D2HIP_DW_ARRIVED(w1); N2D2HIP_DW_ARRIVED(w2); N2D2HIP_DW_ARRIVED(bias);
    if (FAST) {
        N2D2HIP_DW_ARRIVED(tc); N2D2HIP_DW_ARRIVED(td); N2D2HIP_DW_ARRIVED(te);
    } else if (KIND == EPI_I24 || KIND == EPI_I64) {
        N2D2HIP_DW_ARRIVED(ta); N2D2HIP_DW_ARRIVED(tb); N2D2HIP_DW_ARRIVED(tc); N2D2HIP_DW_ARRIVED(td); N2D2HIP_DW_ARRIVED(te);
    }
#undef N2D2HIP_DW_ARRIVED
    // R output rows per turn of the loop, all their input rows requested before the first is used: a thread has 12 loads
    // in flight, and meets the memory latency once per R rows.  Rows past the strip read a row inside the image and store
    // nothing.
    constexpr int R = S == 1 ? 4 : 2;
    for (int q = 0; q < nrows; q += R) {
        const int base = iy0 + S * q + (S == 1 ? 2 : 1);
        Raw3 raw[R * S];
#pragma unroll
        for (int i = 0; i < R * S; ++i)
            raw[i] = fetch_row(base + i);
#pragma unroll
        for (int i = 0; i < R; ++i) {
            if (S != 1)
                t1 = settle_row(raw[2 * i], base + 2 * i);
            const Row4 t2 = settle_row(raw[S * i + S - 1], base + S * i + S - 1);
            int a0 = __builtin_amdgcn_sdot4(t0.c[0], w0.x, bias.x, false);
            int a1 = __builtin_amdgcn_sdot4(t0.c[1], w0.y, bias.y, false);
            int a2 = __builtin_amdgcn_sdot4(t0.c[2], w0.z, bias.z, false);
            int a3 = __builtin_amdgcn_sdot4(t0.c[3], w0.w, bias.w, false);
            a0 = __builtin_amdgcn_sdot4(t1.c[0], w1.x, a0, false);
            a1 = __builtin_amdgcn_sdot4(t1.c[1], w1.y, a1, false);
            a2 = __builtin_amdgcn_sdot4(t1.c[2], w1.z, a2, false);
            a3 = __builtin_amdgcn_sdot4(t1.c[3], w1.w, a3, false);
            a0 = __builtin_amdgcn_sdot4(t2.c[0], w2.x, a0, false);
            a1 = __builtin_amdgcn_sdot4(t2.c[1], w2.y, a1, false);
            a2 = __builtin_amdgcn_sdot4(t2.c[2], w2.z, a2, false);
            a3 = __builtin_amdgcn_sdot4(t2.c[3], w2.w, a3, false);
            unsigned packed;
            if (FAST) {
                packed = sat_bytes_u8((__mul24(a0, tc.x) + td.x) >> te.x, (__mul24(a1, tc.y) + td.y) >> te.y,
                                      (__mul24(a2, tc.z) + td.z) >> te.z, (__mul24(a3, tc.w) + td.w) >> te.w);
            } else {
                const int r0 = finish(a0, 0, ta.x, tb.x, tc.x, td.x, te.x);
                const int r1 = finish(a1, 1, ta.y, tb.y, tc.y, td.y, te.y);
                const int r2 = finish(a2, 2, ta.z, tb.z, tc.z, td.z, te.z);
                const int r3 = finish(a3, 3, ta.w, tb.w, tc.w, td.w, te.w);
                packed = ((unsigned)r0 & 255u) | (((unsigned)r1 & 255u) << 8) | (((unsigned)r2 & 255u) << 16) | ((unsigned)r3 << 24);
            }
            if (q + i < nrows)
                outp[(q + i) * out_row] = packed ^ p.out_xor;
            if (S == 1) {
                t0 = t1;
                t1 = t2;
            } else {
                t0 = t2;
            }
        }
    }
}

} // namespace

void depthwise3x3_weight_layout(const signed char* w, const int* bias, int C, int cs, int* wb)
{
    for (int i = 0; i < 4 * cs; ++i)
        wb[i] = 0;
    for (int c = 0; c < C; ++c) {
        for (int ky = 0; ky < 3; ++ky) {
            const signed char* t = w + ((size_t)c * 3 + ky) * 3;
            wb[ky * cs + c] = (int)((unsigned)(unsigned char)t[0] | ((unsigned)(unsigned char)t[1] << 8) | ((unsigned)(unsigned char)t[2] << 16));
        }
        wb[3 * cs + c] = bias[c];
    }
}

int depthwise3x3_launch(DepthwiseArgs a, int stride, int num_cus, hipStream_t stream)
{
    N2D2HIP_REQUIRE((stride == 1 || stride == 2) && a.cs % 4 == 0, N2D2HIP_ERR_INVALID, "depthwise3x3: stride %d, channel stride %d", stride, a.cs);
    a.cq = (unsigned)(a.cs / 4);
    // Strips short enough that every compute unit holds about 1024 threads: a strip re-reads the two input rows above it.
    const long long columns = (long long)a.B * a.OW * a.cq;
    const long long want = (long long)num_cus * 1024;
    long long nstrips = std::min<long long>((want + columns - 1) / columns, (a.OH + 1) / 2);
    nstrips = std::max<long long>(nstrips, 1);
    a.rows = (int)((a.OH + nstrips - 1) / nstrips);
    a.nstrips = (a.OH + a.rows - 1) / a.rows;
    const long long nthreads = columns * a.nstrips;
    N2D2HIP_REQUIRE(nthreads < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED, "depthwise3x3: tensor too large");
    a.nthreads = (unsigned)nthreads;
    const unsigned grid = (unsigned)round_up((int)((nthreads + 255) / 256), 8);        // a multiple of the XCD count (see the kernel)
#define N2D2HIP_DW_LAUNCH(S, K) N2D2HIP_LAUNCH_T(depthwise3x3_kernel, (S, K), dim3(grid), dim3(256), 0, stream, a)
    if (a.epi.kind == EPI_I24 && a.fast) {
        if (stride == 1) N2D2HIP_LAUNCH_T(depthwise3x3_kernel, (1, EPI_I24, true), dim3(grid), dim3(256), 0, stream, a);
        else N2D2HIP_LAUNCH_T(depthwise3x3_kernel, (2, EPI_I24, true), dim3(grid), dim3(256), 0, stream, a);
    } else if (a.epi.kind == EPI_I24) {
        if (stride == 1) N2D2HIP_DW_LAUNCH(1, EPI_I24); else N2D2HIP_DW_LAUNCH(2, EPI_I24);
    } else if (a.epi.kind == EPI_I64) {
        if (stride == 1) N2D2HIP_DW_LAUNCH(1, EPI_I64); else N2D2HIP_DW_LAUNCH(2, EPI_I64);
    } else {
        if (stride == 1) N2D2HIP_DW_LAUNCH(1, EPI_RAW); else N2D2HIP_DW_LAUNCH(2, EPI_RAW);
    }
#undef N2D2HIP_DW_LAUNCH
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // namespace n2d2hip
