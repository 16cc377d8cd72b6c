// A 3x3 depthwise convolution and the 1x1 convolution that reads it, in one launch (the building block of the MobileNets).
// Launched cell by cell, the depthwise output is written by one launch and read back by the next, and at 14 x 14 and
// below both launches are mostly their fixed cost.  Here a work-group owns a tile of 8 rows x 16 columns of output pixels:
// for each chunk of 64 (or 32) channels it computes the depthwise convolution on the vector ALU exactly as the stand-alone
// kernel does (a thread owns 4 channels of one column and walks down the rows, every tap a byte of a 4-way dot product),
// rescales it to bytes, writes them to LDS as the pixel operand of the matrix cores and multiplies them into the 1x1
// convolution's accumulators, of which that chunk is one slice of K; the depthwise output never reaches memory.
//
// LDS: the pixel operand (128 pixels x 64 bytes, 16-byte slots XOR-swizzled by the row so that the 32 rows of a fragment
// read spread over the banks) and the 1x1 weights of the chunk in matrix-core fragment order (copied by direct-to-LDS
// loads while the vector ALU works on the chunk), both twice, so that a chunk is written while slower waves still
// multiply the one before: one barrier per chunk.  The 1x1 convolution's tables are resident in LDS.
#include <algorithm>
#include <vector>

#include "common.h"
#include "conv_handle.hpp"
#include "depthwise_math.hpp"
#include "epilogue.hpp"
#include "mfma_util.hpp"

namespace n2d2hip {

struct DwPwArgs {
    const signed char* in;    // B x H x W x C bytes
    signed char* out;         // B x OH x OW x O bytes
    const int* wdw;           // depthwise: [3][C] dwords (w[ky][0], w[ky][1], w[ky][2], 0), then [C] biases, zero point folded in
    EpiArgs dwe;              // depthwise rescale, tables by channel
    const signed char* wpw;   // 1x1 weights: [channel tile of 32*NB][chunk][K step of 32][32-channel block][lane][16 bytes]
    const int* pwt;           // 1x1 rescale with the bias folded in: a, b, c, d, e, each [O]
    int C, O;
    int B, H, W, OH, OW, padL, padT;
    int tw;                   // valid columns of a tile (at most 16)
    int tiles_x, tiles_y, ntiles;
    unsigned fill;            // the stored form of 0 in all four bytes of the input
    unsigned mid_xor;         // 0x80808080 when the depthwise output is stored as value - 128
    unsigned out_xor;
    int pw_lo, pw_hi;
    unsigned out_bytes;
};

namespace {

// S: stride of the depthwise convolution; KC: channels per chunk (64, or 32 for a 32-channel layer); NB: 32-channel blocks
// of the 1x1 convolution's outputs a work-group computes (blockIdx.y selects which 32 * NB of them); WAVES: 4, or 8 with
// the channel blocks split between the two halves of the work-group (half the accumulators per wave, half the rows per
// thread in the depthwise part).
// FAST: neither cell needs a clamp before its multiply and both saturate to [0, 255]: the depthwise tables c, d, e are then
// the ones with the bias folded in (accumulators start from zero), and both rescales saturate while they pack.
template <int S, int KC, int NB, int WAVES, bool FAST>
__global__ __launch_bounds__(64 * WAVES) void dw_pw_kernel(const DwPwArgs q)
{
    constexpr int THREADS = 64 * WAVES;
    constexpr int NBW = NB / (WAVES / 4);    // channel blocks of a wave
    static_assert(NBW >= 2 && NBW % 2 == 0, "a wave stores pairs of channel blocks");
    constexpr int CG = KC / 4;               // channel groups of a chunk
    constexpr int RH = THREADS / (CG * 16);  // the tile's rows are split over this many groups of threads
    constexpr int ROWS = 8 / RH;             // output rows a thread walks down
    constexpr int KS = KC / 32;
    constexpr int A_BYTES = 128 * 64;
    constexpr int B_BYTES = KC * NB * 32;
    constexpr int NT = NB * 32;              // output channels of the work-group
    constexpr int A_OFF = 0, B_OFF = 2 * A_BYTES, T_OFF = B_OFF + 2 * B_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[T_OFF + 5 * NT * 4];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;

    // blocks 8 apart run on the same XCD: give each XCD a run of consecutive tiles (neighbours share input rows)
    const int per_xcd = (q.ntiles + 7) / 8;
    const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (tile >= q.ntiles)
        return;
    const int n0 = (int)blockIdx.y * NT;
    const int tx = tile % q.tiles_x;
    const int ty = (tile / q.tiles_x) % q.tiles_y;
    const int b = tile / (q.tiles_x * q.tiles_y);

    // ---- the 1x1 convolution's tables
    {
        int* tab = (int*)(smem + T_OFF);
        for (int i = tid; i < 5 * NT; i += THREADS) {
            const int row = i / NT, ch = i - row * NT;
            tab[i] = q.pwt[row * q.O + n0 + ch];
        }
    }

    // ---- depthwise side: this thread's column and channel group
    const int cg = tid % CG;
    const int x = (tid / CG) % 16;
    const int rh = tid / (CG * 16);
    const int ox = min(tx * q.tw + x, q.OW - 1);
    const int oy0 = ty * 8 + rh * ROWS;
    const int ix0 = ox * S - q.padL;
    const bool vm = ix0 >= 0 && ix0 < q.W, v0 = ix0 + 1 >= 0 && ix0 + 1 < q.W, vp = ix0 + 2 >= 0 && ix0 + 2 < q.W;
    const unsigned fill = q.fill;
    const int om = min(max(ix0, 0), q.W - 1) * q.C, oc = min(max(ix0 + 1, 0), q.W - 1) * q.C, op = min(max(ix0 + 2, 0), q.W - 1) * q.C;
    const long long row_bytes = (long long)q.W * q.C;
    const signed char* img = q.in + (long long)b * q.H * row_bytes + cg * 4;
    const int iy0 = oy0 * S - q.padT;
    typedef const unsigned __attribute__((address_space(1))) * GlobalWord;
    struct Raw3 { unsigned m, c, p; };

    const int wm = wave & 3, wn = wave >> 2;     // this wave's 32 pixels and its run of channel blocks
    v16i acc[NBW];
#pragma unroll
    for (int i = 0; i < NBW; ++i)
        acc[i] = v16i{};

    const int nchunks = q.C / KC;
    for (int kc = 0; kc < nchunks; ++kc) {
        unsigned char* abuf = smem + A_OFF + (kc & 1) * A_BYTES;
        unsigned char* bbuf = smem + B_OFF + (kc & 1) * B_BYTES;
        // ---- the chunk's 1x1 weights: B_BYTES contiguous bytes, 1 KB per load
        {
            const signed char* src = q.wpw + ((long long)blockIdx.y * nchunks + kc) * B_BYTES;
#pragma unroll
            for (int j = 0; j < (B_BYTES / 1024 + WAVES - 1) / WAVES; ++j) {
                const int c = wave + WAVES * j;
                if (c < B_BYTES / 1024)
                    __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + c * 1024 + lane * 16), (lds_ptr_t)(bbuf + c * 1024), 16, 0, 0);
            }
        }
        // ---- depthwise convolution of the chunk's channels
        {
            const int ch = kc * KC + cg * 4;
            const signed char* cimg = img + kc * KC;
            const int4 w0 = *(const int4*)(q.wdw + ch);
            const int4 w1 = *(const int4*)(q.wdw + q.C + ch);
            const int4 w2 = *(const int4*)(q.wdw + 2 * q.C + ch);
            int4 bias = {}, ta = {}, tb = {};
            if (!FAST) {
                bias = *(const int4*)(q.wdw + 3 * q.C + ch);
                ta = *(const int4*)(q.dwe.a + ch);
                tb = *(const int4*)(q.dwe.b + ch);
            }
            const int4 tc = *(const int4*)(q.dwe.c + ch);
            const int4 td = *(const int4*)(q.dwe.d + ch);
            const int4 te = *(const int4*)(q.dwe.e + ch);
            auto fetch_row = [&](int iy) -> Raw3 {
                const signed char* rp = cimg + min(max(iy, 0), q.H - 1) * row_bytes;
                Raw3 r;
                r.m = *(GlobalWord)(rp + om);
                r.c = *(GlobalWord)(rp + oc);
                r.p = *(GlobalWord)(rp + op);
                return r;
            };
            auto settle_row = [&](const Raw3& r, int iy) -> Row4 {
                const bool row_ok = iy >= 0 && iy < q.H;
                return transpose3((row_ok && vm) ? r.m : fill, (row_ok && v0) ? r.c : fill, (row_ok && vp) ? r.p : fill);
            };
            Row4 t0 = settle_row(fetch_row(iy0), iy0);
            Row4 t1 = {};
            if (S == 1)
                t1 = settle_row(fetch_row(iy0 + 1), iy0 + 1);
            // this thread's dword of row m of the pixel operand: slot (cg / 4) of the row, swizzled, byte 4 * (cg % 4)
            constexpr int R = S == 1 ? (ROWS < 4 ? ROWS : 4) : 2;
#pragma unroll
            for (int r0 = 0; r0 < ROWS; r0 += R) {
                const int base = iy0 + S * r0 + (S == 1 ? 2 : 1);
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
                        const int v0r = epi_apply<EPI_I24>(a0, ta.x, tb.x, tc.x, td.x, te.x, q.dwe.lo, q.dwe.hi, 0);
                        const int v1r = epi_apply<EPI_I24>(a1, ta.y, tb.y, tc.y, td.y, te.y, q.dwe.lo, q.dwe.hi, 0);
                        const int v2r = epi_apply<EPI_I24>(a2, ta.z, tb.z, tc.z, td.z, te.z, q.dwe.lo, q.dwe.hi, 0);
                        const int v3r = epi_apply<EPI_I24>(a3, ta.w, tb.w, tc.w, td.w, te.w, q.dwe.lo, q.dwe.hi, 0);
                        packed = ((unsigned)v0r & 255u) | (((unsigned)v1r & 255u) << 8) | (((unsigned)v2r & 255u) << 16) | ((unsigned)v3r << 24);
                    }
                    packed ^= q.mid_xor;
                    const int m = (rh * ROWS + r0 + i) * 16 + x;
                    *(unsigned*)(abuf + m * 64 + (((cg >> 2) ^ ((m >> 1) & 3)) << 4) + ((cg & 3) << 2)) = packed;
                    if (S == 1) {
                        t0 = t1;
                        t1 = t2;
                    } else {
                        t0 = t2;
                    }
                }
            }
        }
        // the chunk's pixel bytes and weights are in LDS for every wave; the chunk before this one has been multiplied by
        // every wave, so its buffers may be written again after this barrier
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // ---- multiply: this wave's 32 pixels against all NB channel blocks
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int m = 32 * wm + l32;
            const v4i pf = *(const v4i*)(abuf + m * 64 + (((2 * ks + lh) ^ ((m >> 1) & 3)) << 4));
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) {
                const v4i wf = *(const v4i*)(bbuf + ((ks * NB + wn * NBW + nb) * 64 + lane) * 16);
                acc[nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf, pf, acc[nb], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: lane (l32, lh) holds, for pixel 32 * wm + l32, channels 32 * (wn * NBW + nb) + 8 * g + 4 * lh + e in
    // acc[nb][4 * g + e]
    const int m = 32 * wm + l32;
    const int px = m & 15, py = m >> 4;
    const int oxo = tx * q.tw + px, oyo = ty * 8 + py;
    const bool pix_ok = px < q.tw && oxo < q.OW && oyo < q.OH;
    const int* tab = (const int*)(smem + T_OFF);
    signed char* orow = q.out + (((long long)b * q.OH + oyo) * q.OW + oxo) * q.O + n0 + wn * NBW * 32 + 32 * lh;
#pragma unroll
    for (int j = 0; j < NBW / 2; ++j) {
        unsigned pk[2][4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ch = (wn * NBW + 2 * j + i) * 32 + 8 * g + 4 * lh;
                const v4i tc = *(const v4i*)(tab + 2 * NT + ch), td = *(const v4i*)(tab + 3 * NT + ch), te = *(const v4i*)(tab + 4 * NT + ch);
                int r[4];
                if (FAST) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        r[e] = (__mul24(acc[2 * j + i][4 * g + e], tc[e]) + td[e]) >> te[e];
                    pk[i][g] = sat_bytes_u8(r[0], r[1], r[2], r[3]) ^ q.out_xor;
                } else {
                    const v4i ta = *(const v4i*)(tab + ch), tb = *(const v4i*)(tab + NT + ch);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int t = med3_i32(acc[2 * j + i][4 * g + e], ta[e], tb[e]);
                        r[e] = med3_i32((__mul24(t, tc[e]) + td[e]) >> te[e], q.pw_lo, q.pw_hi);
                    }
                    pk[i][g] = pack_bytes(r[0], r[1], r[2], r[3]) ^ q.out_xor;
                }
            }
        }
        // exchange between the lane halves until a lane owns 32 consecutive channels of the pair of blocks
        unsigned qd[2][4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const auto s02 = __builtin_amdgcn_permlane32_swap(pk[i][0], pk[i][2], false, false);
            const auto s13 = __builtin_amdgcn_permlane32_swap(pk[i][1], pk[i][3], false, false);
            qd[i][0] = s02[0]; qd[i][1] = s02[1]; qd[i][2] = s13[0]; qd[i][3] = s13[1];
        }
        v4i first, second;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const auto xw = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[1][e], false, false);
            first[e] = (int)xw[0];
            second[e] = (int)xw[1];
        }
        if (pix_ok) {
            *(v4i*)(orow + 64 * j) = first;
            *(v4i*)(orow + 64 * j + 16) = second;
        }
    }
}

bool plain_1x1(const n2d2hip_conv_desc& d)
{
    return d.kW == 1 && d.kH == 1 && d.strideX == 1 && d.strideY == 1 && d.padL == 0 && d.padT == 0 && d.padR == 0 && d.padB == 0
        && d.dilX == 1 && d.dilY == 1 && d.groups == 1 && d.weight_bits == 8;
}

int byte_type_of(const n2d2hip_act_s* a) { return a->min_out >= 0 ? N2D2HIP_U8B : N2D2HIP_I8; }

template <int S, int KC, bool FAST>
void launch_nb(const DwPwArgs& a, int nb, dim3 grid, hipStream_t stream)
{
    if (nb == 8) N2D2HIP_LAUNCH_T(dw_pw_kernel, (S, KC, 8, 8, FAST), grid, dim3(512), 0, stream, a);
    else if (nb == 4) N2D2HIP_LAUNCH_T(dw_pw_kernel, (S, KC, 4, 4, FAST), grid, dim3(256), 0, stream, a);
    else N2D2HIP_LAUNCH_T(dw_pw_kernel, (S, KC, 2, 4, FAST), grid, dim3(256), 0, stream, a);
}

template <int S, int KC>
void launch_fast(const DwPwArgs& a, bool fast, int nb, dim3 grid, hipStream_t stream)
{
    if (fast) launch_nb<S, KC, true>(a, nb, grid, stream); else launch_nb<S, KC, false>(a, nb, grid, stream);
}

} // namespace
} // namespace n2d2hip

using namespace n2d2hip;

struct n2d2hip_dw_pw_s {
    n2d2hip_conv_t dw, pw;
    int kc, nb;               // channels per chunk, 32-channel blocks per work-group
    bool fast;                // neither rescale clamps before its multiply, both saturate to [0, 255]
    signed char* d_w;
    int* d_tab;
};

extern "C" {

int n2d2hip_dw_pw_destroy(n2d2hip_dw_pw_t h)
{
    if (!h) return N2D2HIP_OK;
    if (h->d_w) (void)hipFree(h->d_w);
    if (h->d_tab) (void)hipFree(h->d_tab);
    delete h;
    return N2D2HIP_OK;
}

int n2d2hip_dw_pw_create(n2d2hip_conv_t dw, n2d2hip_conv_t pw, n2d2hip_dw_pw_t* out)
{
    N2D2HIP_REQUIRE(dw && pw && out, N2D2HIP_ERR_INVALID, "dw_pw_create: null argument");
    const n2d2hip_conv_desc& dd = dw->desc;
    const n2d2hip_conv_desc& dp = pw->desc;
    const int C = dd.C, O = dp.O;
    const bool ok = dw->depthwise && dw->d_wdw && dd.kW == 3 && dd.kH == 3 && dd.dilX == 1 && dd.dilY == 1 && dd.strideX == dd.strideY
        && (dd.strideX == 1 || dd.strideX == 2) && dw->act->args.kind == EPI_I24 && dw->act->cpad >= C && dw->in_cs == C
        && (C == 32 || C % 64 == 0) && dw->act->min_out >= -128 && dw->act->max_out <= 255
        && plain_1x1(dp) && dp.C == C && pw->in_cs == C && pw->in_dtype == byte_type_of(dw->act) && (O == 64 || O == 128 || O % 256 == 0)
        && pw->act->args.kind == EPI_I24 && pw->bias_folded && pw->d_epi_tab && pw->act->min_out >= -128 && pw->act->max_out <= 255
        && !pw->sum && pw->ktot >= C;
    N2D2HIP_REQUIRE(ok, N2D2HIP_ERR_UNSUPPORTED,
                    "dw_pw_create: needs a 3x3 undilated depthwise convolution of stride 1 or 2 over 32 or a multiple of 64 channels and an "
                    "unpadded 1x1 convolution of stride 1 reading it, to 64, 128 or a multiple of 256 channels, both 8-bit with integer "
                    "rescales (32-bit multiply-add) and byte outputs, the second without a folded sum");
    const int kc = C == 32 ? 32 : 64, nb = std::min(O, 256) / 32, nt = nb * 32;
    const int nchunks = C / kc, ks = kc / 32;
    std::vector<signed char> w((size_t)pw->opad * pw->ktot);
    const int cp = pw->act->cpad;
    std::vector<int> tab5(5 * (size_t)cp);
    hipError_t e = hipMemcpy(w.data(), pw->d_w, w.size(), hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemcpy(tab5.data(), pw->d_epi_tab, tab5.size() * sizeof(int), hipMemcpyDeviceToHost);
    if (e != hipSuccess)
        return fail(N2D2HIP_ERR_HIP, "dw_pw_create: reading the 1x1 convolution back failed: %s", hipGetErrorString(e));
    // [channel tile][chunk][K step][32-channel block][lane][16 bytes]: lane l holds channel l % 32 of the block,
    // bytes K step * 32 + 16 * (l / 32) .. of the chunk
    auto fragment_image = [&](int blocks) {
        std::vector<signed char> img((size_t)O * C);
        const int tile = blocks * 32;
        for (int t = 0; t < O / tile; ++t)
            for (int c = 0; c < nchunks; ++c)
                for (int s = 0; s < ks; ++s)
                    for (int blk = 0; blk < blocks; ++blk)
                        for (int l = 0; l < 64; ++l)
                            memcpy(img.data() + ((((size_t)(t * nchunks + c) * ks + s) * blocks + blk) * 64 + l) * 16,
                                   w.data() + (size_t)(t * tile + blk * 32 + (l & 31)) * pw->ktot + c * kc + s * 32 + 16 * (l >> 5), 16);
        return img;
    };
    const std::vector<signed char> img = fragment_image(nb);
    (void)nt;
    // a, b, c, d, e by channel; a cell that needs no clamp before its multiply gets bounds that clamp nothing
    std::vector<int> tab(5 * (size_t)O);
    for (int r = 0; r < 5; ++r)
        for (int o = 0; o < O; ++o)
            tab[(size_t)r * O + o] = tab5[(size_t)r * cp + o];
    if (!pw->preclamp)
        for (int o = 0; o < O; ++o) {
            tab[o] = std::numeric_limits<int>::min();
            tab[(size_t)O + o] = std::numeric_limits<int>::max();
        }
    n2d2hip_dw_pw_s* h = new n2d2hip_dw_pw_s();
    h->dw = dw; h->pw = pw; h->kc = kc; h->nb = nb; h->d_w = nullptr; h->d_tab = nullptr;
    h->fast = dw->bias_folded && dw->d_epi_tab && !dw->preclamp && dw->act->args.lo == 0 && dw->act->args.hi == 255
        && !pw->preclamp && pw->act->args.lo == 0 && pw->act->args.hi == 255;
    e = hipMalloc((void**)&h->d_w, img.size());
    if (e == hipSuccess) e = hipMemcpy(h->d_w, img.data(), img.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void**)&h->d_tab, tab.size() * sizeof(int));
    if (e == hipSuccess) e = hipMemcpy(h->d_tab, tab.data(), tab.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        n2d2hip_dw_pw_destroy(h);
        return fail(N2D2HIP_ERR_HIP, "dw_pw_create: device upload failed: %s", hipGetErrorString(e));
    }
    *out = h;
    return N2D2HIP_OK;
}

int n2d2hip_dw_pw_pays(n2d2hip_dw_pw_t h, int batch, int in_h, int in_w)
{
    if (!h || batch <= 0)
        return 0;
    int OH, OW;
    if (n2d2hip_conv_out_dims(&h->dw->desc, in_h, in_w, &OH, &OW) != N2D2HIP_OK)
        return 0;
    const long long pixels = (long long)batch * OH * OW;
    // One work-group holds all output channels of its pixels and the tensor between the cells is large: with more than 256
    // output channels the depthwise part is computed once per 256 of them, and on small images the launch has too few
    // work-groups to fill the chip.
    return h->pw->desc.O <= 256 && pixels >= 32768 ? 1 : 0;
}

int n2d2hip_dw_pw_forward(n2d2hip_dw_pw_t h, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    N2D2HIP_REQUIRE(h && in && out && in->data && out->data, N2D2HIP_ERR_INVALID, "dw_pw_forward: null argument");
    const n2d2hip_conv_desc& dd = h->dw->desc;
    const n2d2hip_conv_desc& dp = h->pw->desc;
    int OH, OW;
    int rc = n2d2hip_conv_out_dims(&dd, in->H, in->W, &OH, &OW);
    if (rc != N2D2HIP_OK)
        return rc;
    const int out_dtype = byte_type_of(h->pw->act);
    N2D2HIP_REQUIRE(in->layout == N2D2HIP_NHWC && out->layout == N2D2HIP_NHWC && in->halo == 0 && out->halo == 0, N2D2HIP_ERR_UNSUPPORTED,
                    "dw_pw_forward: tensors must be NHWC without a border");
    N2D2HIP_REQUIRE(in->dtype == h->dw->in_dtype && in->C == dd.C && in->cs == dd.C, N2D2HIP_ERR_INVALID,
                    "dw_pw_forward: input has %d channels (stride %d) of type %d, the depthwise convolution expects %d of type %d", in->C,
                    in->cs, in->dtype, dd.C, h->dw->in_dtype);
    N2D2HIP_REQUIRE(out->B == in->B && out->C == dp.O && out->cs == dp.O && out->H == OH && out->W == OW && out->dtype == out_dtype,
                    N2D2HIP_ERR_INVALID, "dw_pw_forward: output must be %dx%dx%dx%d bytes of type %d with a channel stride of %d", in->B, dp.O,
                    OH, OW, out_dtype, dp.O);
    N2D2HIP_REQUIRE((long long)in->B * in->H * in->W * in->cs < (1ll << 31) && (long long)out->B * OH * OW * out->cs < (1ll << 31),
                    N2D2HIP_ERR_UNSUPPORTED, "dw_pw_forward: tensor too large");
    DwPwArgs a;
    a.in = (const signed char*)in->data; a.out = (signed char*)out->data;
    a.wdw = h->dw->d_wdw; a.dwe = h->dw->act->args;
    if (h->fast) {
        const int cpd = h->dw->act->cpad;
        a.dwe.c = h->dw->d_epi_tab + 2 * cpd; a.dwe.d = h->dw->d_epi_tab + 3 * cpd; a.dwe.e = h->dw->d_epi_tab + 4 * cpd;
    }
    a.wpw = h->d_w; a.pwt = h->d_tab;
    a.C = dd.C; a.O = dp.O;
    a.B = in->B; a.H = in->H; a.W = in->W; a.OH = OH; a.OW = OW; a.padL = dd.padL; a.padT = dd.padT;
    // columns of a tile: 16, or fewer when that leaves fewer idle columns in the last tile of a row
    int best_tw = 16;
    long long best_cols = ((OW + 15) / 16) * 16;
    for (int tw = 15; tw >= 8; --tw) {
        const long long cols = (long long)((OW + tw - 1) / tw) * 16;
        if (cols < best_cols) { best_cols = cols; best_tw = tw; }
    }
    a.tw = best_tw;
    a.tiles_x = (OW + a.tw - 1) / a.tw;
    a.tiles_y = (OH + 7) / 8;
    const long long ntiles = (long long)in->B * a.tiles_y * a.tiles_x;
    N2D2HIP_REQUIRE(ntiles < (1 << 28), N2D2HIP_ERR_UNSUPPORTED, "dw_pw_forward: tensor too large");
    a.ntiles = (int)ntiles;
    a.fill = zero_point(in->dtype) ? 0x80808080u : 0u;
    a.mid_xor = h->pw->in_dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    a.out_xor = out_dtype == N2D2HIP_U8B ? 0x80808080u : 0u;
    a.pw_lo = h->pw->act->args.lo; a.pw_hi = h->pw->act->args.hi;
    a.out_bytes = (unsigned)((long long)out->B * OH * OW * out->cs);
    const dim3 grid((unsigned)(((a.ntiles + 7) / 8) * 8), (unsigned)(dp.O / (h->nb * 32)));
    if (dd.strideX == 1) {
        if (h->kc == 32) launch_fast<1, 32>(a, h->fast, h->nb, grid, stream); else launch_fast<1, 64>(a, h->fast, h->nb, grid, stream);
    } else {
        if (h->kc == 32) launch_fast<2, 32>(a, h->fast, h->nb, grid, stream); else launch_fast<2, 64>(a, h->fast, h->nb, grid, stream);
    }
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
