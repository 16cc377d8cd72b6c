// The end of one residual bottleneck and the start of the next in one launch: the expanding 1x1 convolution (C -> 4C) with
// the block's ElemWise sum in its epilogue, and the reducing 1x1 convolution (4C -> C) of the block that follows, which
// reads nothing but that sum.  Launched cell by cell the block's output is written by one launch and read back by the
// next, and the reducing convolution (about 1 us of matrix work at 14 x 14) pays a whole launch.  Here a work-group owns
// 128 pixels and ALL 4C channels of them: for each tile of 128 output channels it computes the expansion, adds the
// residual input and rescales (the pipelined kernel's folded sum, on 16-bit pairs), writes the bytes to memory (the next
// block's shortcut needs them) and to LDS, and at once multiplies them into the reducing convolution's accumulators,
// of which that channel tile is one 128-wide slice of K.  After the last channel tile those accumulators are rescaled and
// stored, into a tensor that may carry the border of zeros the following 3x3 convolution wants.
//
// Operands: the expansion's pixel operand (128 pixels x C bytes) lives in registers for the whole tile (each wave loads
// the fragments of its 32 pixels straight from global memory); both weight sets stream through a three-stage LDS ring
// as one sequence of stages in the order they are consumed (per channel tile: the expansion's 128 x C weights, then the
// reduction's C x 128 slice), in matrix-core fragment order, copied by direct-to-LDS loads two stages ahead; the tables
// of all channels are resident in LDS.  Two barriers per channel tile.  Vector memory operations complete in issue order,
// so every wait is a count of the operations issued after the one needed (the counts are written next to the waits).
#include <algorithm>
#include <type_traits>
#include <utility>
#include <vector>

#include "common.h"
#include "conv_handle.hpp"
#include "mfma_util.hpp"

namespace n2d2hip {

struct ExpandReduceArgs {
    const signed char* x;        // [M][C] bytes: input of the expansion
    const signed char* res;      // [M][4C] bytes: the sum's other input
    signed char* y;              // [M][4C] bytes: the sum
    signed char* z;              // the reducing convolution's output, C channels, NHWC, may carry a border
    const signed char* wstream;  // per channel tile: 128 x C expansion weights, C x 128 reduction weights, fragment order
    const int* tab;              // expansion c, d; other input's c, d (each [4C]); sum c, d, e as 16-bit pairs (each [2C] ints);
                                 // reduction c, d (each [C])
    int M, ntiles;
    int HW, W, z_halo, z_cs, ZHp, ZWp;
    unsigned y_bytes, z_bytes;
    unsigned hw_mul, hw_sh, w_mul, w_sh;
    int c_lo, c_hi;              // saturation of the expansion
    int p_lo, p_hi;              // of the ScalingCell on the other input
    unsigned res_flip, y_xor, z_xor;
};

namespace {

__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
__device__ __forceinline__ void gload128(v4i& dst, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(dst) : "v"(p) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f)
{
    (f(std::integral_constant<int, I>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(std::make_integer_sequence<int, N>(), f);
}

// CMID: channels of the expansion's input and of the reduction's output (128 or 256); the sum has 4 * CMID.
// PRE: the sum's other input is taken as it is (0), goes through a folded ScalingCell whose result cannot leave its range (1)
// or can (2).  The sum and the reduction saturate to [0, 255] (Rectifier cells with unsigned outputs), which has an
// instruction of its own; the expansion saturates to the range given.
template <int CMID, int PRE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void expand_reduce_kernel(ExpandReduceArgs q)
{
    constexpr bool HAS_PRE = PRE != 0;
    constexpr int COUT = 4 * CMID;
    constexpr int NCT = COUT / 128;            // channel tiles of the sum
    constexpr int KS = CMID / 32;              // K steps of the expansion
    constexpr int NI2 = CMID / 64;             // 32-channel tiles of the reduction per wave
    constexpr int SB = 128 * CMID;             // bytes of a ring stage
    constexpr int NL = SB / (512 * 16);        // direct loads per thread and stage
    constexpr int RING_OFF = 0, YT_OFF = 3 * SB, T1_OFF = YT_OFF + 128 * 128;
    constexpr int T1_INTS = 4 * COUT + 3 * (COUT / 2), T2_INTS = 2 * CMID;
    constexpr int P16_OFF = T1_OFF + 16 * COUT;          // the 16-bit pairs behind the four int arrays
    constexpr int T2_OFF = T1_OFF + 4 * T1_INTS;
    static_assert(CMID == 128 || CMID == 256, "128 or 256 middle channels");
    static_assert(NI2 >= 2, "the next tile's pixel loads need two younger stores behind them");
    __shared__ __attribute__((aligned(16))) unsigned char smem[T2_OFF + 4 * T2_INTS];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wc = wave & 1, wp = wave >> 1;   // channel half, pixel quarter
    const int l32 = lane & 31, lh = lane >> 5;

    const int G = gridDim.x;
    const int ntile = ((int)blockIdx.x < q.ntiles) ? (q.ntiles - (int)blockIdx.x + G - 1) / G : 0;
    if (ntile == 0)
        return;
    for (int i = tid; i < T1_INTS + T2_INTS; i += 512)
        ((int*)(smem + T1_OFF))[i] = q.tab[i];

    // the weight ring: stage s of the stream goes to slot s % 3
    int r_stage = 0, r_slot = 0;
    auto issue_ring = [&]() {
        const signed char* src = q.wstream + (size_t)r_stage * SB + tid * 16;
        unsigned char* dst = smem + RING_OFF + r_slot * SB + wave * 1024;
#pragma unroll
        for (int j = 0; j < NL; ++j)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + j * 8192), (lds_ptr_t)(dst + j * 8192), 16, 0, 0);
        r_stage = (r_stage + 1 == 2 * NCT) ? 0 : r_stage + 1;
        r_slot = (r_slot + 1 == 3) ? 0 : r_slot + 1;
    };
    // pixel row of this lane in tile k of this block (tiles past the block's last repeat it; rows past the end read row 0)
    auto row_of = [&](int k) -> int {
        const int m = ((int)blockIdx.x + min(k, ntile - 1) * G) * 128 + wp * 32 + l32;
        return m < q.M ? m : 0;
    };
    v4i xf[KS];
    auto issue_x = [&](int k) {
        const signed char* p = q.x + (size_t)row_of(k) * CMID + 16 * lh;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)
            gload128(xf[kk], p + kk * 32);
    };
    v4i rfirst, rsecond;
    auto issue_r = [&](int k, int ct) {
        const signed char* p = q.res + (size_t)row_of(k) * COUT + ct * 128 + wc * 64 + 32 * lh;
        gload128(rfirst, p);
        gload128(rsecond, p + 16);
    };
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(q.y, 0, q.y_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t z_rsrc = __builtin_amdgcn_make_buffer_rsrc(q.z, 0, q.z_bytes, 0x00020000);

    v16i acc1[2], acc2[NI2];
#pragma unroll
    for (int i = 0; i < NI2; ++i)
        acc2[i] = v16i{};
    const v2s lo1 = splat_v2s(q.c_lo), hi1 = splat_v2s(q.c_hi);
    const v2s lo3 = splat_v2s(q.p_lo), hi3 = splat_v2s(q.p_hi);

    // ---- prologue: the first tile's pixels and residual, two ring stages
    issue_x(0);
    issue_r(0, 0);
    issue_ring();
    issue_ring();
    wait_vm<NL>();                     // everything but the second stage has landed
    int c_slot = 0;                    // ring slot consumed next
    int k = 0, ct = 0;
    unsigned yoff = 0, zoff = 0;       // byte offsets of this lane's pixel in y and z (out of range: nothing is stored)
    const int nit = ntile * NCT;
    for (int it = 0; it < nit; ++it) {
        // ---- the expansion's stage has landed (issued two barriers ago; behind it: 2 residual loads, 2 stores of the
        // sum, NL loads of the following stage) and everybody is done with the previous reduction step
        wait_vm<4 + NL>();
        lds_barrier();
        issue_ring();
        if (ct == 0) {
#pragma unroll
            for (int kk = 0; kk < KS; ++kk)
                tie(xf[kk]);
            const int m = ((int)blockIdx.x + k * G) * 128 + wp * 32 + l32;
            if (m < q.M) {
                yoff = (unsigned)m * COUT;
                const int b = div_magic(m, q.hw_mul, q.hw_sh);
                const int rem = m - b * q.HW;
                const int yy = div_magic(rem, q.w_mul, q.w_sh);
                const int xx = rem - yy * q.W;
                zoff = (unsigned)(((b * q.ZHp + yy + q.z_halo) * q.ZWp + xx + q.z_halo) * q.z_cs);
            } else {
                yoff = 0x80000000u;
                zoff = 0x80000000u;
            }
        }
        // ---- expansion: acc1[i] = W[channel tile 2 wc + i] . x, K = CMID
        {
            const unsigned base = lds0 + RING_OFF + c_slot * SB + ((2 * wc) * KS * 64 + lane) * 16;
            v4i fa[2][2];
            lds_read128_nowait<0>(fa[0][0], base);
            lds_read128_nowait<KS * 1024>(fa[0][1], base);
            static_for<KS>([&](auto kkc) {
                constexpr int kk = decltype(kkc)::value;
                constexpr int set = kk & 1;
                wait_lgkm<0>();
                tie(fa[set][0]); tie(fa[set][1]);
                if constexpr (kk + 1 < KS) {
                    lds_read128_nowait<(kk + 1) * 1024>(fa[set ^ 1][0], base);
                    lds_read128_nowait<(KS + kk + 1) * 1024>(fa[set ^ 1][1], base);
                }
                if constexpr (kk == 0) {
                    acc1[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][0], xf[kk], v16i{}, 0, 0, 0);
                    acc1[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][1], xf[kk], v16i{}, 0, 0, 0);
                } else {
                    acc1[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][0], xf[kk], acc1[0], 0, 0, 0);
                    acc1[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][1], xf[kk], acc1[1], 0, 0, 0);
                }
            });
            c_slot = (c_slot + 1 == 3) ? 0 : c_slot + 1;
        }
        // ---- the residual input of this channel tile (issued a channel tile ago; behind it: 2 stores, 2 NL ring loads)
        // into the accumulators' layout: the output's lane-half exchanges run backwards
        unsigned resw[8];
        wait_vm<2 + 2 * NL>();
        tie(rfirst); tie(rsecond);
        {
            unsigned qd[2][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const auto yv = __builtin_amdgcn_permlane32_swap((unsigned)rfirst[e], (unsigned)rsecond[e], false, false);
                qd[0][e] = yv[0]; qd[1][e] = yv[1];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const auto s02 = __builtin_amdgcn_permlane32_swap(qd[i][0], qd[i][1], false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(qd[i][2], qd[i][3], false, false);
                resw[i * 4 + 0] = s02[0]; resw[i * 4 + 2] = s02[1];
                resw[i * 4 + 1] = s13[0]; resw[i * 4 + 3] = s13[1];
            }
        }
        // the next channel tile's residual (the next tile's first one behind the last)
        const bool last_ct = ct == NCT - 1;
        {
            const int nct = last_ct ? 0 : ct + 1, nk = last_ct ? k + 1 : k;
            issue_r(nk, nct);
        }
        // ---- rescale, add, rescale: the folded sum on pairs of 16-bit values
        unsigned pk[2][4];
        {
            const unsigned t32 = lds0 + T1_OFF + (unsigned)(ct * 128 + wc * 64 + 4 * lh) * 4u;
            const unsigned t16 = lds0 + P16_OFF + (unsigned)(ct * 128 + wc * 64 + 4 * lh) * 2u;
            static_for<8>([&](auto idxc) {
                constexpr int idx = decltype(idxc)::value;
                constexpr int i = idx / 4, g = idx % 4;
                constexpr int o32 = (i * 32 + 8 * g) * 4, o16 = (i * 32 + 8 * g) * 2;
                v4i tc, td, xc, xd;
                v2i c16, d16, e16;
                lds_read128_nowait<o32>(tc, t32);
                lds_read128_nowait<4 * COUT + o32>(td, t32);
                if (HAS_PRE) {
                    lds_read128_nowait<8 * COUT + o32>(xc, t32);
                    lds_read128_nowait<12 * COUT + o32>(xd, t32);
                }
                lds_read64_nowait<o16>(c16, t16);
                lds_read64_nowait<2 * COUT + o16>(d16, t16);
                lds_read64_nowait<4 * COUT + o16>(e16, t16);
                wait_lgkm<0>();
                tie(tc); tie(td);
                if (HAS_PRE) { tie(xc); tie(xd); }
                tie(c16); tie(d16); tie(e16);
                v2s pq[2], oq[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int t0 = __mul24(acc1[i][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                    const int t1 = __mul24(acc1[i][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                    pq[h] = clamp_v2s(as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u)), lo1, hi1);
                }
                const unsigned w = resw[idx] ^ q.res_flip;
                if (HAS_PRE) {
                    unsigned u[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        u[t] = __umul24((w >> (8 * t)) & 0xffu, (unsigned)xc[t]) + (unsigned)xd[t];
                    oq[0] = as_v2s((int)__builtin_amdgcn_perm(u[1], u[0], 0x07060302u));
                    oq[1] = as_v2s((int)__builtin_amdgcn_perm(u[3], u[2], 0x07060302u));
                    if (PRE == 2) {
                        oq[0] = clamp_v2s(oq[0], lo3, hi3);
                        oq[1] = clamp_v2s(oq[1], lo3, hi3);
                    }
                } else {
                    oq[0] = as_v2s((int)__builtin_amdgcn_perm(w, w, 0x0c010c00u));
                    oq[1] = as_v2s((int)__builtin_amdgcn_perm(w, w, 0x0c030c02u));
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    v2s v = pq[h] + oq[h];
                    v = v * as_v2s(c16[h]) + as_v2s(d16[h]);
                    pq[h] = v >> as_v2s(e16[h]);
                }
                pk[i][g] = (sat_pk_u8(pq[0]) | (sat_pk_u8(pq[1]) << 16)) ^ q.y_xor;
                asm volatile("" : "+v"(pk[i][g]));
            });
        }
        // the expansion's accumulators have all been read, so its pixel fragments are free: the next tile's are requested
        if (last_ct)
            issue_x(k + 1);
        // ---- 32 consecutive channels per lane: to memory, and to LDS as the reduction's pixel operand
        {
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
                const auto xv = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[1][e], false, false);
                first[e] = (int)xv[0];
                second[e] = (int)xv[1];
            }
            const unsigned off = yoff + (unsigned)(ct * 128 + wc * 64 + 32 * lh);
            __builtin_amdgcn_raw_buffer_store_b128(first, y_rsrc, off, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b128(second, y_rsrc, off + 16u, 0, 0);
            unsigned char* yt = smem + YT_OFF + ((wp * 4 + 2 * wc + lh) * 64 + l32) * 16;
            *(v4i*)yt = first;
            *(v4i*)(yt + 512) = second;
        }
        // ---- the reduction's stage has landed (behind it: NL ring loads, 2 residual loads, 2 stores) and this channel
        // tile's bytes are in LDS for everybody
        wait_vm<4 + NL>();
        lds_barrier();
        issue_ring();
        {
            const unsigned base = lds0 + RING_OFF + c_slot * SB + ((wc * NI2) * 4 * 64 + lane) * 16;
            const unsigned ybase = lds0 + YT_OFF + ((wp * 4) * 64 + lane) * 16;
            v4i fb[2][NI2], fy[2];
            static_for<NI2>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                lds_read128_nowait<(i * 4) * 1024>(fb[0][i], base);
            });
            lds_read128_nowait<0>(fy[0], ybase);
            static_for<4>([&](auto kkc) {
                constexpr int kk = decltype(kkc)::value;
                constexpr int set = kk & 1;
                wait_lgkm<0>();
#pragma unroll
                for (int i = 0; i < NI2; ++i)
                    tie(fb[set][i]);
                tie(fy[set]);
                if constexpr (kk + 1 < 4) {
                    static_for<NI2>([&](auto ic) {
                        constexpr int i = decltype(ic)::value;
                        lds_read128_nowait<(i * 4 + kk + 1) * 1024>(fb[set ^ 1][i], base);
                    });
                    lds_read128_nowait<(kk + 1) * 1024>(fy[set ^ 1], ybase);
                }
#pragma unroll
                for (int i = 0; i < NI2; ++i)
                    acc2[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[set][i], fy[set], acc2[i], 0, 0, 0);
            });
            c_slot = (c_slot + 1 == 3) ? 0 : c_slot + 1;
        }
        if (last_ct) {
            // ---- the reduction is complete: rescale, saturate, 32 consecutive channels per lane, store
            const unsigned t2 = lds0 + T2_OFF + (unsigned)(wc * NI2 * 32 + 4 * lh) * 4u;
            unsigned pz[NI2][4];
            static_for<NI2 * 4>([&](auto idxc) {
                constexpr int idx = decltype(idxc)::value;
                constexpr int i = idx / 4, g = idx % 4;
                constexpr int o32 = (i * 32 + 8 * g) * 4;
                v4i tc, td;
                lds_read128_nowait<o32>(tc, t2);
                lds_read128_nowait<4 * CMID + o32>(td, t2);
                wait_lgkm<0>();
                tie(tc); tie(td);
                v2s pq[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int t0 = __mul24(acc2[i][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                    const int t1 = __mul24(acc2[i][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                    pq[h] = as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u));
                }
                pz[i][g] = (sat_pk_u8(pq[0]) | (sat_pk_u8(pq[1]) << 16)) ^ q.z_xor;
                asm volatile("" : "+v"(pz[i][g]));
            });
#pragma unroll
            for (int p = 0; p < NI2 / 2; ++p) {
                unsigned qd[2][4];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const auto s02 = __builtin_amdgcn_permlane32_swap(pz[2 * p + i][0], pz[2 * p + i][2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(pz[2 * p + i][1], pz[2 * p + i][3], false, false);
                    qd[i][0] = s02[0]; qd[i][1] = s02[1]; qd[i][2] = s13[0]; qd[i][3] = s13[1];
                }
                v4i first, second;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const auto xv = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[1][e], false, false);
                    first[e] = (int)xv[0];
                    second[e] = (int)xv[1];
                }
                const unsigned off = zoff + (unsigned)(wc * NI2 * 32 + p * 64 + 32 * lh);
                __builtin_amdgcn_raw_buffer_store_b128(first, z_rsrc, off, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(second, z_rsrc, off + 16u, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < NI2; ++i)
                acc2[i] = v16i{};
            ct = 0;
            ++k;
        } else {
            ++ct;
        }
    }
    // no direct load may still be writing into LDS when the block's LDS is handed to another block
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
}

bool one_by_one(const n2d2hip_conv_desc& d)
{
    return d.kW == 1 && d.kH == 1 && d.strideX == 1 && d.strideY == 1 && d.padL == 0 && d.padT == 0 && d.padR == 0 && d.padB == 0
        && d.dilX == 1 && d.dilY == 1 && d.groups == 1 && d.weight_bits == 8;
}
bool hi16_cell(const n2d2hip_conv_s* c)
{
    return c->act->args.kind == EPI_I24 && c->bias_folded && c->hi16 && c->d_epi_tab && c->act->min_out >= -128 && c->act->max_out <= 255;
}
int byte_dtype_of(const n2d2hip_act_s* a) { return a->min_out >= 0 ? N2D2HIP_U8B : N2D2HIP_I8; }
unsigned xor_of(int dtype) { return dtype == N2D2HIP_U8B ? 0x80808080u : 0u; }
void magic(unsigned d, unsigned* mul, unsigned* sh)
{
    if (d <= 1) { *mul = 0; *sh = 0; return; }
    unsigned s = 0;
    while ((1ull << s) < d) ++s;
    *mul = (unsigned)((1ull << (31 + s)) / d + 1);
    *sh = s - 1;
}
int device_cus()
{
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
        return prop.multiProcessorCount;
    return 256;
}

// rows x K weights (row stride `stride`) -> [32-row tile][K step of 32][lane][16 bytes]: lane l holds row tile * 32 + l % 32,
// bytes K step * 32 + 16 * (l / 32) ..
void to_fragments(const signed char* w, int row0, int rows, int k0, int ksteps, int stride, signed char* out)
{
    for (int t = 0; t < rows / 32; ++t)
        for (int kk = 0; kk < ksteps; ++kk)
            for (int l = 0; l < 64; ++l)
                for (int b = 0; b < 16; ++b)
                    out[(((size_t)t * ksteps + kk) * 64 + l) * 16 + b] =
                        w[(size_t)(row0 + t * 32 + (l & 31)) * stride + k0 + kk * 32 + 16 * (l >> 5) + b];
}

} // namespace
} // namespace n2d2hip

using namespace n2d2hip;

struct n2d2hip_expand_reduce_s {
    n2d2hip_conv_t expand, reduce;
    int cmid;
    signed char* d_w;
    int* d_tab;
};

extern "C" {

int n2d2hip_expand_reduce_create(n2d2hip_conv_t expand, n2d2hip_conv_t reduce, n2d2hip_expand_reduce_t* out)
{
    N2D2HIP_REQUIRE(expand && reduce && out, N2D2HIP_ERR_INVALID, "expand_reduce_create: null argument");
    const n2d2hip_conv_desc& de = expand->desc;
    const n2d2hip_conv_desc& dr = reduce->desc;
    const int cmid = de.C, cout = de.O;
    const bool ok = one_by_one(de) && one_by_one(dr) && (cmid == 128 || cmid == 256) && cout == 4 * cmid && dr.C == cout && dr.O == cmid
        && expand->in_cs == cmid && reduce->in_cs == cout && hi16_cell(expand) && hi16_cell(reduce) && !reduce->preclamp && !reduce->sum
        && expand->sum && expand->d_res_tab && expand->sum16 && expand->sum->act->cpad == cout && expand->act->cpad == cout
        && expand->sum->act->args.lo == 0 && expand->sum->act->args.hi == 255 && reduce->act->args.lo == 0 && reduce->act->args.hi == 255
        && reduce->in_dtype == byte_dtype_of(expand->sum->act) && reduce->act->cpad >= cmid
        && expand->ktot == cmid && reduce->ktot == cout;
    N2D2HIP_REQUIRE(ok, N2D2HIP_ERR_UNSUPPORTED,
                    "expand_reduce_create: needs a 1x1 convolution C -> 4C (C = 128 or 256) with its sum folded in on 16-bit pairs and a 1x1 "
                    "convolution 4C -> C reading that sum, both 8-bit with integer rescales that fit the scaled-up tables, the sum and the "
                    "second convolution saturating to [0, 255]");
    const int nct = cout / 128, ks = cmid / 32;
    const size_t sb = (size_t)128 * cmid;
    std::vector<signed char> we((size_t)expand->opad * expand->ktot), wr((size_t)reduce->opad * reduce->ktot);
    hipError_t e = hipMemcpy(we.data(), expand->d_w, we.size(), hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemcpy(wr.data(), reduce->d_w, wr.size(), hipMemcpyDeviceToHost);
    if (e != hipSuccess)
        return fail(N2D2HIP_ERR_HIP, "expand_reduce_create: reading the weights back failed: %s", hipGetErrorString(e));
    std::vector<signed char> stream(2 * (size_t)nct * sb);
    for (int ct = 0; ct < nct; ++ct) {
        to_fragments(we.data(), ct * 128, 128, 0, ks, expand->ktot, stream.data() + (size_t)(2 * ct) * sb);
        to_fragments(wr.data(), 0, cmid, ct * 128, 4, reduce->ktot, stream.data() + (size_t)(2 * ct + 1) * sb);
    }
    std::vector<int> tab((size_t)4 * cout + 3 * (cout / 2) + 2 * cmid, 0);
    {
        const int cp = cout;
        e = hipMemcpy(tab.data(), expand->d_epi_tab + 5 * cp, cout * sizeof(int), hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(tab.data() + cout, expand->d_epi_tab + 6 * cp, cout * sizeof(int), hipMemcpyDeviceToHost);
        if (e == hipSuccess && expand->has_pre) {
            e = hipMemcpy(tab.data() + 2 * cout, expand->d_res_tab + 12 * cp, cout * sizeof(int), hipMemcpyDeviceToHost);
            if (e == hipSuccess) e = hipMemcpy(tab.data() + 3 * cout, expand->d_res_tab + 13 * cp, cout * sizeof(int), hipMemcpyDeviceToHost);
        }
        if (e == hipSuccess) e = hipMemcpy(tab.data() + 4 * cout, expand->d_res_tab + 10 * cp, 3 * (cp / 2) * sizeof(int), hipMemcpyDeviceToHost);
        const int cpr = reduce->act->cpad;
        int* t2 = tab.data() + 4 * cout + 3 * (cout / 2);
        if (e == hipSuccess) e = hipMemcpy(t2, reduce->d_epi_tab + 5 * cpr, cmid * sizeof(int), hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(t2 + cmid, reduce->d_epi_tab + 6 * cpr, cmid * sizeof(int), hipMemcpyDeviceToHost);
    }
    if (e != hipSuccess)
        return fail(N2D2HIP_ERR_HIP, "expand_reduce_create: reading the tables back failed: %s", hipGetErrorString(e));
    n2d2hip_expand_reduce_s* h = new n2d2hip_expand_reduce_s();
    h->expand = expand; h->reduce = reduce; h->cmid = cmid; h->d_w = nullptr; h->d_tab = nullptr;
    e = hipMalloc((void**)&h->d_w, stream.size());
    if (e == hipSuccess) e = hipMemcpy(h->d_w, stream.data(), stream.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void**)&h->d_tab, tab.size() * sizeof(int));
    if (e == hipSuccess) e = hipMemcpy(h->d_tab, tab.data(), tab.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        n2d2hip_expand_reduce_destroy(h);
        return fail(N2D2HIP_ERR_HIP, "expand_reduce_create: device upload failed: %s", hipGetErrorString(e));
    }
    *out = h;
    return N2D2HIP_OK;
}

int n2d2hip_expand_reduce_destroy(n2d2hip_expand_reduce_t h)
{
    if (!h) return N2D2HIP_OK;
    if (h->d_w) (void)hipFree(h->d_w);
    if (h->d_tab) (void)hipFree(h->d_tab);
    delete h;
    return N2D2HIP_OK;
}

int n2d2hip_expand_reduce_forward(n2d2hip_expand_reduce_t h, const n2d2hip_tensor* x, const n2d2hip_tensor* other, const n2d2hip_tensor* sum,
                                  const n2d2hip_tensor* reduced, n2d2hip_stream_t stream_)
{
    int rc;
    N2D2HIP_REQUIRE(h != nullptr, N2D2HIP_ERR_INVALID, "expand_reduce_forward: null handle");
    if ((rc = check_tensor(x, "expand_reduce input")) || (rc = check_tensor(other, "expand_reduce other input"))
        || (rc = check_tensor(sum, "expand_reduce sum")) || (rc = check_tensor(reduced, "expand_reduce output", true)))
        return rc;
    const int cmid = h->cmid, cout = 4 * cmid;
    const n2d2hip_conv_s* ce = h->expand;
    const n2d2hip_conv_s* cr = h->reduce;
    const n2d2hip_act_s* sa = ce->sum->act;
    N2D2HIP_REQUIRE(x->layout == N2D2HIP_NHWC && other->layout == N2D2HIP_NHWC && sum->layout == N2D2HIP_NHWC && reduced->layout == N2D2HIP_NHWC,
                    N2D2HIP_ERR_UNSUPPORTED, "expand_reduce_forward: NHWC tensors");
    N2D2HIP_REQUIRE(x->dtype == ce->in_dtype && x->C == cmid && x->cs == cmid, N2D2HIP_ERR_INVALID,
                    "expand_reduce_forward: input must have %d channels of the type the expansion was created for", cmid);
    N2D2HIP_REQUIRE(other->dtype == ce->sum_other_dtype && other->C == cout && other->cs == cout && other->B == x->B && other->H == x->H
                        && other->W == x->W,
                    N2D2HIP_ERR_INVALID, "expand_reduce_forward: the sum's other input must be %dx%dx%dx%d of the type given when the sum was folded",
                    x->B, cout, x->H, x->W);
    N2D2HIP_REQUIRE(sum->B == x->B && sum->H == x->H && sum->W == x->W && sum->C == cout && sum->cs == cout && sum->dtype == byte_dtype_of(sa),
                    N2D2HIP_ERR_INVALID, "expand_reduce_forward: the sum must be %dx%dx%dx%d bytes", x->B, cout, x->H, x->W);
    N2D2HIP_REQUIRE(reduced->B == x->B && reduced->H == x->H && reduced->W == x->W && reduced->C == cmid && reduced->cs == cmid
                        && reduced->dtype == byte_dtype_of(cr->act),
                    N2D2HIP_ERR_INVALID, "expand_reduce_forward: the output must be %dx%dx%dx%d bytes", x->B, cmid, x->H, x->W);
    const long long M = (long long)x->B * x->H * x->W;
    const long long zpix = (long long)x->B * (x->H + 2 * reduced->halo) * (x->W + 2 * reduced->halo);
    N2D2HIP_REQUIRE(M * cout < (1ll << 31) && zpix * cmid < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED, "expand_reduce_forward: tensor too large");

    ExpandReduceArgs q = {};
    q.x = (const signed char*)x->data; q.res = (const signed char*)other->data;
    q.y = (signed char*)sum->data; q.z = (signed char*)reduced->data;
    q.wstream = h->d_w; q.tab = h->d_tab;
    q.M = (int)M; q.ntiles = (int)((M + 127) / 128);
    q.HW = x->H * x->W; q.W = x->W; q.z_halo = reduced->halo; q.z_cs = reduced->cs;
    q.ZHp = x->H + 2 * reduced->halo; q.ZWp = x->W + 2 * reduced->halo;
    q.y_bytes = (unsigned)(M * cout); q.z_bytes = (unsigned)(zpix * cmid);
    magic((unsigned)q.HW, &q.hw_mul, &q.hw_sh);
    magic((unsigned)q.W, &q.w_mul, &q.w_sh);
    q.c_lo = ce->act->args.lo; q.c_hi = ce->act->args.hi;
    if (ce->has_pre) { q.p_lo = ce->sum->pre_act->args.lo; q.p_hi = ce->sum->pre_act->args.hi; }
    q.res_flip = other->dtype == N2D2HIP_U8 ? 0u : 0x80808080u;
    q.y_xor = xor_of(sum->dtype); q.z_xor = xor_of(reduced->dtype);
    // as many blocks as finish together: ceil(tiles / rounds) with rounds = ceil(tiles / compute units)
    const int cus = device_cus();
    const int rounds = (q.ntiles + cus - 1) / cus;
    const int grid = (q.ntiles + rounds - 1) / rounds;
    hipStream_t stream = (hipStream_t)stream_;
#define N2D2HIP_ER_LAUNCH(C, P) N2D2HIP_LAUNCH_T(expand_reduce_kernel, (C, P), dim3(grid), dim3(512), 0, stream, q)
    const int pre = !ce->has_pre ? 0 : ce->pre_in_range ? 1 : 2;
    if (cmid == 128) {
        if (pre == 0) N2D2HIP_ER_LAUNCH(128, 0); else if (pre == 1) N2D2HIP_ER_LAUNCH(128, 1); else N2D2HIP_ER_LAUNCH(128, 2);
    } else {
        if (pre == 0) N2D2HIP_ER_LAUNCH(256, 0); else if (pre == 1) N2D2HIP_ER_LAUNCH(256, 1); else N2D2HIP_ER_LAUNCH(256, 2);
    }
#undef N2D2HIP_ER_LAUNCH
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
