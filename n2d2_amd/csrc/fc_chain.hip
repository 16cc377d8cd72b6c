// Two or three small fully-connected cells, one reading the other, in one launch (a classifier head: LeNet's 400 -> 120 ->
// 84 -> 10).  Each of them is a few microseconds of work for a handful of work-groups, so launched one by one they cost
// their launches; here a work-group takes G images through all the cells, the vectors between them in LDS.
//
// A thread owns one output channel: for every dword of K it reads its channel's four weights (the host stores the weights
// K-major, so the 128 threads read 128 consecutive dwords) and multiplies them into the accumulators of the G images,
// whose input dwords every lane reads from the same LDS address (a broadcast).  Accumulation is in int32 on 4-way byte
// dot products, the rescale is the one every cell uses (epi_apply_dyn), so results are those of the cells run in turn.
#include <algorithm>
#include <cstring>
#include <vector>

#include "common.h"
#include "conv_handle.hpp"
#include "epilogue.hpp"

namespace n2d2hip {

enum { FC_CHAIN_MAX = 3, FC_CHAIN_K4 = 256 /* dwords of K per cell at most */, FC_CHAIN_O = 128 };

struct FcChainArgs {
    const signed char* in;      // B images of in_bytes contiguous bytes (NHWC with the channel stride equal to the channels)
    int in_bytes, B, n;
    const unsigned* wt[FC_CHAIN_MAX];       // [K / 4][128] dwords: the four weights of output o for bytes 4k .. 4k + 3
    const int* bias[FC_CHAIN_MAX];          // zero point of the cell's input folded in
    EpiArgs epi[FC_CHAIN_MAX];
    int k4[FC_CHAIN_MAX], O[FC_CHAIN_MAX];
    int store[FC_CHAIN_MAX];                // storage type of cell l's output (what cell l + 1 reads; the tensor's for the last)
    void* out;
    int out_cs;
};

template <int G>
__global__ __launch_bounds__(FC_CHAIN_O) void fc_chain_kernel(const FcChainArgs q)
{
    __shared__ unsigned xbuf[2][G][FC_CHAIN_K4];
    const int o = threadIdx.x;
    const int g0 = blockIdx.x * G;
    // ---- the images' input vectors; K past the input's own bytes meets zero weights
    for (int i = o; i < G * q.k4[0]; i += FC_CHAIN_O) {
        const int g = i / q.k4[0], k = i - g * q.k4[0];
        const int img = min(g0 + g, q.B - 1);
        xbuf[0][g][k] = 4 * k < q.in_bytes ? *(const unsigned*)(q.in + (size_t)img * q.in_bytes + 4 * k) : 0u;
    }
    __syncthreads();
    int cur = 0;
    for (int l = 0; l < q.n; ++l) {
        int acc[G];
        const int b = q.bias[l][o];
#pragma unroll
        for (int g = 0; g < G; ++g)
            acc[g] = b;
        const unsigned* w = q.wt[l] + o;
        const int k4 = q.k4[l];
#pragma unroll 8
        for (int k = 0; k < k4; ++k) {
            const int wv = (int)w[(size_t)k * FC_CHAIN_O];
#pragma unroll
            for (int g = 0; g < G; ++g)
                acc[g] = __builtin_amdgcn_sdot4((int)xbuf[cur][g][k], wv, acc[g], false);
        }
        const bool last = l + 1 == q.n;
        if (!last) {
            // the next cell's input: bytes in its storage form, the channels past this cell's outputs meet zero weights
            unsigned char* nx = (unsigned char*)xbuf[cur ^ 1];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                int v = 0;
                if (o < q.O[l]) {
                    v = epi_apply_dyn(q.epi[l], acc[g], o);
                    v = q.store[l] == N2D2HIP_U8B ? v - 128 : v;
                }
                nx[g * (FC_CHAIN_K4 * 4) + o] = (unsigned char)v;
            }
            // (the next cell may read more than 128 bytes of K: the rest is cleared)
            for (int i = o; i < G * (q.k4[l + 1] - FC_CHAIN_O / 4); i += FC_CHAIN_O) {
                const int per = q.k4[l + 1] - FC_CHAIN_O / 4;
                xbuf[cur ^ 1][i / per][FC_CHAIN_O / 4 + i % per] = 0u;
            }
        } else if (o < q.O[l]) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (g0 + g < q.B)
                    store_value(q.out, (size_t)(g0 + g) * q.out_cs + o, q.store[l], epi_apply_dyn(q.epi[l], acc[g], o));
            }
        }
        __syncthreads();
        cur ^= 1;
    }
}

} // namespace n2d2hip

using namespace n2d2hip;

struct n2d2hip_fc_chain_s {
    int n;
    n2d2hip_fc_t fc[FC_CHAIN_MAX];
    unsigned* d_wt[FC_CHAIN_MAX];
    int k4[FC_CHAIN_MAX];
};

extern "C" {

int n2d2hip_fc_chain_destroy(n2d2hip_fc_chain_t h)
{
    if (!h) return N2D2HIP_OK;
    for (int l = 0; l < h->n; ++l)
        if (h->d_wt[l]) (void)hipFree(h->d_wt[l]);
    delete h;
    return N2D2HIP_OK;
}

int n2d2hip_fc_chain_create(int n, const n2d2hip_fc_t* fcs, n2d2hip_fc_chain_t* out)
{
    N2D2HIP_REQUIRE(fcs && out, N2D2HIP_ERR_INVALID, "fc_chain_create: null argument");
    bool ok = n >= 2 && n <= FC_CHAIN_MAX;
    for (int l = 0; ok && l < n; ++l) {
        const n2d2hip_conv_s* c = fcs[l];
        ok = c && c->is_fc && c->desc.weight_bits == 8 && !c->depthwise && !c->pix4 && c->ktot % 4 == 0 && c->ktot <= 4 * FC_CHAIN_K4
            && c->desc.O <= FC_CHAIN_O && c->d_w && c->d_bias && !c->sum;
        // the cell reads what the one before it writes: a vector of that cell's outputs, stored as this cell's input type
        if (ok && l > 0)
            ok = c->fcH == 1 && c->fcW == 1 && c->desc.C == fcs[l - 1]->desc.O && c->ktot >= c->desc.C
                && fcs[l - 1]->act->min_out >= (c->in_dtype == N2D2HIP_I8 ? -128 : 0) && fcs[l - 1]->act->max_out <= (c->in_dtype == N2D2HIP_I8 ? 127 : 255);
    }
    N2D2HIP_REQUIRE(ok, N2D2HIP_ERR_UNSUPPORTED,
                    "fc_chain_create: needs two or three 8-bit fully-connected cells, each after the first reading the 1 x 1 output of "
                    "the one before, with at most 1024 inputs and 128 outputs each");
    n2d2hip_fc_chain_s* h = new n2d2hip_fc_chain_s();
    h->n = n;
    for (int l = 0; l < FC_CHAIN_MAX; ++l) { h->fc[l] = nullptr; h->d_wt[l] = nullptr; h->k4[l] = 0; }
    for (int l = 0; l < n; ++l) {
        const n2d2hip_conv_s* c = fcs[l];
        h->fc[l] = fcs[l];
        h->k4[l] = c->ktot / 4;
        std::vector<signed char> w((size_t)c->opad * c->ktot);
        hipError_t e = hipMemcpy(w.data(), c->d_w, w.size(), hipMemcpyDeviceToHost);
        std::vector<unsigned> wt((size_t)h->k4[l] * FC_CHAIN_O, 0u);
        if (e == hipSuccess) {
            for (int o = 0; o < c->desc.O; ++o)
                for (int k = 0; k < h->k4[l]; ++k)
                    memcpy(&wt[(size_t)k * FC_CHAIN_O + o], w.data() + (size_t)o * c->ktot + 4 * k, 4);
            e = hipMalloc((void**)&h->d_wt[l], wt.size() * sizeof(unsigned));
        }
        if (e == hipSuccess) e = hipMemcpy(h->d_wt[l], wt.data(), wt.size() * sizeof(unsigned), hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            n2d2hip_fc_chain_destroy(h);
            return fail(N2D2HIP_ERR_HIP, "fc_chain_create: moving the weights failed: %s", hipGetErrorString(e));
        }
    }
    *out = h;
    return N2D2HIP_OK;
}

int n2d2hip_fc_chain_forward(n2d2hip_fc_chain_t h, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream_)
{
    int rc;
    N2D2HIP_REQUIRE(h != nullptr, N2D2HIP_ERR_INVALID, "fc_chain_forward: null handle");
    if ((rc = check_tensor(in, "fc_chain input")) || (rc = check_tensor(out, "fc_chain output")))
        return rc;
    const n2d2hip_conv_s* first = h->fc[0];
    const n2d2hip_conv_s* last = h->fc[h->n - 1];
    N2D2HIP_REQUIRE(in->layout == N2D2HIP_NHWC && in->dtype == first->in_dtype && in->C == first->desc.C && in->cs == first->in_cs
                        && in->H == first->fcH && in->W == first->fcW,
                    N2D2HIP_ERR_INVALID, "fc_chain_forward: input is %dx%dx%d (stride %d) of type %d, the first cell was built for %dx%dx%d of type %d",
                    in->C, in->H, in->W, in->cs, in->dtype, first->desc.C, first->fcH, first->fcW, first->in_dtype);
    const int in_bytes = in->H * in->W * in->cs;
    N2D2HIP_REQUIRE(in_bytes % 4 == 0 && in_bytes <= first->ktot, N2D2HIP_ERR_UNSUPPORTED, "fc_chain_forward: %d input bytes per image", in_bytes);
    N2D2HIP_REQUIRE(out->layout == N2D2HIP_NHWC && out->B == in->B && out->C == last->desc.O && out->H == 1 && out->W == 1
                        && out->cs >= last->desc.O,
                    N2D2HIP_ERR_INVALID, "fc_chain_forward: output must be %dx%dx1x1", in->B, last->desc.O);
    if (last->act->args.kind == EPI_RAW) {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_INVALID, "fc_chain_forward: without a rescale the last cell outputs raw sums; the output dtype must be I32");
    } else if (is_byte_type(out->dtype)) {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(last->act->min_out >= lo && last->act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "fc_chain_forward: activation range [%d,%d] does not fit output dtype %d", last->act->min_out, last->act->max_out, out->dtype);
    } else {
        N2D2HIP_REQUIRE(out->dtype == N2D2HIP_I32, N2D2HIP_ERR_UNSUPPORTED, "fc_chain_forward: F32 outputs are produced with n2d2hip_convert");
    }
    FcChainArgs a = {};
    a.in = (const signed char*)in->data; a.in_bytes = in_bytes; a.B = in->B; a.n = h->n;
    for (int l = 0; l < h->n; ++l) {
        const n2d2hip_conv_s* c = h->fc[l];
        a.wt[l] = h->d_wt[l]; a.bias[l] = c->d_bias; a.epi[l] = c->act->args; a.k4[l] = h->k4[l]; a.O[l] = c->desc.O;
        a.store[l] = l + 1 < h->n ? h->fc[l + 1]->in_dtype : out->dtype;
    }
    a.out = out->data; a.out_cs = out->cs;
    // two images per work-group: the launch is bound by latency, not by the weights every work-group reads again
    constexpr int G = 2;
    N2D2HIP_LAUNCH_T(fc_chain_kernel, (G), dim3((in->B + G - 1) / G), dim3(FC_CHAIN_O), 0, (hipStream_t)stream_, a);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
