// Second half of a residual bottleneck in one launch: 3x3 convolution (CM -> CM channels, CM = 64, 128 or 256), 1x1
// expansion (CM -> 4 CM) and the two-input sum with the block's shortcut.  Launched cell by cell, the middle tensor goes
// to memory and back and the expansion, a matrix product over only CM of K, pays a launch's fill and drain for very few
// matrix instructions; here the middle tensor of a tile lives in LDS and the expansion starts from there.
//
// A work-group of four waves walks tiles of BM output pixels:
//  phase A  t2[BM][CM] = conv3x3(in): the pipelined kernel's loop (operands global -> LDS by direct loads into an S-stage
//           ring, fragments LDS -> registers one K step ahead, one barrier per stage) over ALL CM output channels, on an
//           input that carries its padding as a border; rescaled (result in the upper half of the multiply-add),
//           saturated, packed, and written to LDS as rows of CM bytes, where the ring was: the ring is filled per tile.
//  phase B  out[BM][4 CM] = sum(expand(t2), other): a wave takes 64 pixels and walks chunks of 64 output channels.  Pixel
//           fragments come from t2, weight fragments straight from memory (the host stores them in fragment order) into a
//           small ring of register sets that runs RD K steps ahead, across chunk boundaries; the other input of the sum is
//           requested one chunk ahead.  The three rescales run on pairs of 16-bit values, exactly as in the pipelined
//           kernel's folded sum, whose tables (here for all 4 CM channels) are copied to LDS behind t2.
// Vector memory operations of a wave complete in issue order; every wait below is s_waitcnt vmcnt(n) with n = the number
// of operations issued after the one needed, computed at compile time from the fixed order in which a wave issues them.
#include <algorithm>
#include <cstring>
#include <utility>

#include "conv_chain.hpp"

namespace n2d2hip {

namespace {

__device__ __forceinline__ void chain_gload128(v4i& dst, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(dst) : "v"(p) : "memory");
}
template <int OFF>
__device__ __forceinline__ void chain_gload128_at(v4i& dst, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=&v"(dst) : "v"(p), "n"(OFF) : "memory");
}
template <int N>
__device__ __forceinline__ void chain_wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void chain_lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
__device__ __forceinline__ void lds_write128(unsigned addr, const v4i& v)
{
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>());
}

// Phase B's vector memory operations of one wave, in issue order:
//   W(0) .. W(RD-1) (2 loads each), R(0) (4 loads);
//   chunk c: for every K step kk: [wait W(c KS + kk)] ... W(c KS + kk + RD) if there is one;
//            [wait R(c)], 4 stores, with R(c + 1), if there is one, in front of them or (late) behind them.
// Returns the number of operations issued between the one waited for (kk < 0: R(qc)) and its wait.
constexpr int chain_after(int KS, int NCH, int RD, bool late, int qc, int qkk)
{
    int n = 0;
    int w_at[64] = {};
    int r_at[16] = {};
    for (int G = 0; G < RD; ++G) { n += 2; w_at[G] = n; }
    n += 4; r_at[0] = n;
    for (int c = 0; c < NCH; ++c) {
        for (int kk = 0; kk < KS; ++kk) {
            const int G = c * KS + kk;
            if (c == qc && kk == qkk) return n - w_at[G];
            if (G + RD < NCH * KS) { n += 2; w_at[G + RD] = n; }
        }
        if (c == qc && qkk < 0) return n - r_at[c];
        if (!late && c + 1 < NCH) { n += 4; r_at[c + 1] = n; }
        n += 4;
        if (late && c + 1 < NCH) { n += 4; r_at[c + 1] = n; }
    }
    return 0;
}

} // namespace

// CM: middle channels = 64 * (4 / WGM); BK, S: bytes of K per ring stage and ring depth of phase A; a wave of phase A owns
// NJ x 2 tiles of 32 pixels x 32 channels, WGM waves side by side along the pixels.
// PRE: the sum's other input goes through a folded ScalingCell.
// WPE: waves per SIMD the registers are budgeted for: 2, or 3 where three work-groups of four waves fit a compute unit's LDS
// (64 middle channels on a three-stage ring): the third work-group fills units the other two leave idle while they rescale.
template <int CM, int BK, int S, int NJ, int WGM, bool PRE, int WPE = 2>
__global__ __launch_bounds__(WGM * (CM / 64) * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void conv_chain_kernel(ConvChainArgs g)
{
    const ConvPipeArgs& q = g.p;
    const ConvArgs& p = q.c;
    constexpr int NI = 2;
    constexpr int WGN = CM / 64;                       // every wave column owns 64 of the middle channels
    constexpr int NW = WGM * WGN, NT = NW * 64;
    static_assert(NW == 4 || NW == 8, "four waves (two or three work-groups per compute unit) or eight (one)");
    constexpr int TM = 32 * NJ, TN = 32 * NI;
    constexpr int BM = TM * WGM, BN = CM;
    constexpr int LPR = BK / 16, RPC = 64 / LPR, KH = BK / 32, TOFF = 32 * BK;
    constexpr int A_CH = BM / RPC, B_CH = BN / RPC;
    constexpr int A_J = (A_CH + NW - 1) / NW, B_J = (B_CH + NW - 1) / NW;
    constexpr int LPI = A_J + B_J;
    constexpr int STAGE = BM * BK + BN * BK;
    static_assert(BK == 64 || BK == 128, "K bytes per stage");
    static_assert(A_CH % NW == 0 && B_CH % NW == 0, "every wave loads whole chunks, none twice");
    static_assert(LPI * (S - 1) < 60, "vmcnt is a 6-bit counter");
    // phase B
    constexpr int OC = 4 * CM;
    static_assert(BM % 64 == 0, "a wave of phase B owns 64 pixels");
    constexpr int WGM_B = BM / 64, WGN_B = NW / WGM_B;
    constexpr int NCH = (OC / 64) / WGN_B;             // chunks of 64 output channels per wave
    constexpr int KS = CM / 32;                        // K steps of the expansion
    constexpr int RD = KS >= 4 ? 4 : 2;                // weight register sets
    // The sum's other input of the next chunk is requested before this chunk's rescales where the K loop is too short to
    // hide the request (its registers are then live through the rescales), else behind them.
    constexpr bool RES_LATE = KS >= 4;
    static_assert(KS % RD == 0 && NCH * KS <= 64 && NCH <= 16, "the register ring's index is a compile-time value");
    constexpr int SH = CM == 64 ? 2 : CM == 128 ? 1 : 0;      // t2 rows are XOR-swizzled like the ring's
    // LDS: the ring, where t2 goes once a tile's K loop is done; behind it the 3x3 convolution's multiplier and addend and
    // the tables of the expansion and the sum
    constexpr int T2_OFF = 0, TABB_BYTES = 22 * OC;
    constexpr int TABA_OFF = S * STAGE, TABB_OFF = TABA_OFF + 2 * CM * 4;
    static_assert(BM * CM <= S * STAGE, "t2 takes the ring's place");
    static_assert(TABB_OFF + TABB_BYTES <= (NW == 4 ? (WPE == 3 ? 53 : 80) : 160) * 1024, "three or two work-groups of four waves per compute unit, or one of eight");
    __shared__ __attribute__((aligned(1024))) unsigned char smem[TABB_OFF + TABB_BYTES];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane_k = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int wmB = wave % WGM_B, wnB = wave / WGM_B;

    // ---- tiles of this block: every mlanes-th pixel tile of its XCD's run (blocks 8 apart share an XCD)
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int mlane = xcd * q.xcd_tiles + slot;
    const int mend = min((xcd + 1) * q.xcd_tiles, q.mtiles);
    const int ntile = (mlane < mend) ? (mend - mlane + q.mlanes - 1) / q.mlanes : 0;
    if (ntile == 0)
        return;
    const int niter = p.niter;
#ifdef N2D2HIP_PROFILE
    long long pr[6] = {0, 0, 0, 0, 0, 0}, pr_t0 = clock64(), pr_t2 = 0, pr_w0 = wall_clock64();
#define CHAIN_MARK(k) do { const long long now__ = clock64(); pr[k] += now__ - pr_last; pr_last = now__; } while (0)
#else
#define CHAIN_MARK(k) do { } while (0)
#endif

    // ---- resident tables: the 3x3 convolution's, the expansion's, the sum's
    if (tid < CM) {
        int* ta = (int*)(smem + TABA_OFF);
        ta[tid] = p.epi.c[tid];
        ta[CM + tid] = p.epi.d[tid];
    }
    {
        int* tb = (int*)(smem + TABB_OFF);
        for (int i = tid; i < OC; i += NT) {
            tb[i] = g.etc[i];
            tb[OC + i] = g.etd[i];
            if (PRE) {
                tb[2 * OC + i] = q.pre.c[i];
                tb[3 * OC + i] = q.pre.d[i];
            }
        }
        for (int i = tid; i < OC / 2; i += NT) {
            tb[4 * OC + i] = q.sum16[i];
            tb[4 * OC + OC / 2 + i] = q.sum16[q.sum16_stride + i];
            tb[4 * OC + OC + i] = q.sum16[2 * q.sum16_stride + i];
        }
    }

    for (int t = 0; t < ntile; ++t) {
        const int m0 = (mlane + t * q.mlanes) * BM;
        // The lane's coordinates are made opaque once per tile: every address below is then formed inside the tile instead
        // of being formed before the loop, by the hundred, and spilled.
        int lane = lane_k;
        asm volatile("" : "+v"(lane));
        const int l32 = lane & 31, lh = lane >> 5;
        // ---- phase A's loader: lane l of a wave fills 16-byte slot l of a 1 KB chunk (see the pipelined kernel)
        const int lrow = lane / LPR;
        const int lq = BK == 64 ? (lane & 3) ^ ((lane >> 4) & 3) : (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4));
        unsigned woff[B_J];
    #pragma unroll
        for (int j = 0; j < B_J; ++j)
            woff[j] = (unsigned)((((wave + NW * j) % B_CH) * RPC + lrow) * p.ktot + lq * 16);
        int rowoff[A_J];
        int l_it, l_koff, l_stage, l_c, l_kx, l_ky, l_tapoff;
        auto loader_new_tile = [&](int m0) {
    #pragma unroll
            for (int j = 0; j < A_J; ++j) {
                const int m = m0 + ((wave + NW * j) % A_CH) * RPC + lrow;
                const int mm = m < p.M ? m : 0;            // rows past the end are computed like pixel 0 and never stored
                const int b = div_magic(mm, q.ohw_mul, q.ohw_sh);
                const int rem = mm - b * (p.OH * p.OW);
                const int oy = div_magic(rem, q.ow_mul, q.ow_sh);
                const int ox = rem - oy * p.OW;
                const int by = oy * p.strideY - p.padT, bx = ox * p.strideX - p.padL;
                rowoff[j] = ((b * p.H + by) * p.W + bx) * p.in_cs + lq * 16;
            }
            l_it = 0; l_koff = 0; l_stage = 0; l_c = 0; l_kx = 0; l_ky = 0; l_tapoff = 0;
        };
        auto issue = [&]() {
            unsigned char* sbase = smem + l_stage * STAGE;
            const signed char* ibase = p.in + l_tapoff;
    #pragma unroll
            for (int j = 0; j < A_J; ++j)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(ibase + (unsigned)rowoff[j]), (lds_ptr_t)(sbase + ((wave + NW * j) % A_CH) * 1024), 16, 0, 0);
            const signed char* wbase = p.w + l_koff;
    #pragma unroll
            for (int j = 0; j < B_J; ++j)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(wbase + woff[j]), (lds_ptr_t)(sbase + BM * BK + ((wave + NW * j) % B_CH) * 1024), 16, 0, 0);
            l_stage = (l_stage + 1 == S) ? 0 : l_stage + 1;
            l_koff += BK;
            ++l_it;
            l_tapoff += BK;
            if (++l_c == q.cper) {
                l_c = 0;
                if (++l_kx == q.kW) { l_kx = 0; ++l_ky; }
                l_tapoff = (l_ky * p.W + l_kx) * p.in_cs;
            }
        };

        // ---- phase A's fragment reads, two register sets
        unsigned pa[KH], wa[KH];
        int r_stage;
        v4i fw[2][NI], fp[2][NJ];
        auto reader_reset = [&]() {
    #pragma unroll
            for (int kk = 0; kk < KH; ++kk) {
                pa[kk] = lds0 + swz_k<BK>(wm * TM + l32, 2 * kk + lh);
                wa[kk] = lds0 + BM * BK + swz_k<BK>(wn * TN + l32, 2 * kk + lh);
            }
            r_stage = 0;
        };
        auto read_k = [&](auto kkc) {
            constexpr int kk = decltype(kkc)::value;
            constexpr int set = kk & 1;
            lds_read128_nowait<0>(fw[set][0], wa[kk]);
            lds_read128_nowait<TOFF>(fw[set][1], wa[kk]);
            lds_read128_nowait<0>(fp[set][0], pa[kk]);
            if (NJ > 1) lds_read128_nowait<TOFF>(fp[set][NJ > 1 ? 1 : 0], pa[kk]);
            if (NJ > 2) lds_read128_nowait<2 * TOFF>(fp[set][NJ > 2 ? 2 : 0], pa[kk]);
            if (NJ > 3) lds_read128_nowait<3 * TOFF>(fp[set][NJ > 3 ? 3 : 0], pa[kk]);
            if (kk == KH - 1) {
                const bool wrap = r_stage + 1 == S;
                const unsigned inc = wrap ? (unsigned)(-(S - 1) * STAGE) : (unsigned)STAGE;
                r_stage = wrap ? 0 : r_stage + 1;
    #pragma unroll
                for (int k2 = 0; k2 < KH; ++k2) { pa[k2] += inc; wa[k2] += inc; }
            }
        };

        const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, q.out_pixels * p.out_cs, 0x00020000);
        const int vlo = p.epi.lo, vhi = p.epi.hi;
        const unsigned tabA = lds0 + TABA_OFF + (unsigned)(wn * TN + 4 * lh) * 4u;
        // phase B: chunk c of the wave is chunk c * WGN_B + wnB of the output channels
        constexpr int WCHUNK = KS * 2048;                  // bytes of a chunk's weights: [K step][channel tile][lane][16]

#ifdef N2D2HIP_PROFILE
        long long pr_last = clock64();
#endif
        // =========================================================== phase A
        loader_new_tile(m0);
        reader_reset();
#pragma unroll
        for (int s = 0; s < S; ++s)
            issue();
        wait_loads_and_barrier<LPI*(S - 1)>();         // step 0 has landed
#ifdef N2D2HIP_PROFILE
        if (t == 0) pr_t2 = clock64();
#endif
        // (cleared here, not by a first matrix instruction that starts from zero: the accumulators' registers would
        // otherwise count as occupied from one tile's K loop to the next, through phase B)
        v16i acc[NI][NJ];
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                acc[i][j] = v16i{};
        read_k(std::integral_constant<int, 0>());
        for (int it = 0; it < niter; ++it) {
            auto kstep = [&](auto kkc) {
                constexpr int kk = decltype(kkc)::value;
                constexpr int set = kk & 1;
                wait_lgkm<0>();
#pragma unroll
                for (int i = 0; i < NI; ++i) tie(fw[set][i]);
#pragma unroll
                for (int j = 0; j < NJ; ++j) tie(fp[set][j]);
                if (kk == KH - 1) {
                    // every wave has its last fragments of this stage; the next stage has landed for every wave.  The ring
                    // stops at the tile's end: its last steps wait for everything that is still on its way.
                    if (l_it < niter) {
                        wait_loads_and_barrier<LPI*(S - 2)>();
                        issue();
                    } else {
                        wait_loads_and_barrier<0>();
                    }
                }
                read_k(std::integral_constant<int, (kk + 1) % KH>());
#pragma unroll
                for (int i = 0; i < NI; ++i)
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[set][i], fp[set][j], acc[i][j], 0, 0, 0);
            };
            kstep(std::integral_constant<int, 0>());
            kstep(std::integral_constant<int, 1>());
            if constexpr (KH > 2) {
                kstep(std::integral_constant<int, 2 % KH>());
                kstep(std::integral_constant<int, 3 % KH>());
            }
        }
        // (the last K step requested fragments of a stage that holds nothing new: they are dropped once they have arrived)
        wait_lgkm<0>();
        tie(fw[0][0]); tie(fw[0][1]);
#pragma unroll
        for (int j = 0; j < NJ; ++j) tie(fp[0][j]);
        CHAIN_MARK(0);

        // ---- phase B's first requests: its weights run RD K steps ahead, the sum's other input one chunk ahead.
        // Addresses are formed here, once per tile, and advanced as the loads are issued: left to itself the compiler
        // would form the address of every load of every chunk before the tile loop and keep them all in registers.
        v4i wfB[RD][2], rfirst[2], rsecond[2];
        const int laneB = lane, l32B = l32, lhB = lh;
        const signed char* wptr = g.we + ((size_t)wnB * WCHUNK + laneB * 16);
        asm volatile("" : "+v"(wptr));
        auto issue_wB = [&](auto Gc) {
            constexpr int G = decltype(Gc)::value;
            chain_gload128_at<0>(wfB[G % RD][0], wptr);
            chain_gload128_at<1024>(wfB[G % RD][1], wptr);
            wptr += (G % KS == KS - 1) ? 2048 + (WGN_B - 1) * WCHUNK : 2048;
            asm volatile("" : "+v"(wptr));
        };
        int opix[2];
        bool live[2];
        const signed char* rptr[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = m0 + wmB * 64 + j * 32 + l32B;
            live[j] = m < p.M;
            const int mm = live[j] ? m : 0;
            const int b = div_magic(mm, q.ohw_mul, q.ohw_sh);
            const int rem = mm - b * (p.OH * p.OW);
            const int oy = div_magic(rem, q.ow_mul, q.ow_sh);
            const int ox = rem - oy * p.OW;
            opix[j] = ((b * (p.OH + 2 * q.out_halo) + oy + q.out_halo) * (p.OW + 2 * q.out_halo) + ox + q.out_halo) * p.out_cs
                + wnB * 64 + 16 * lhB;
            const int rpix = (b * (p.OH + 2 * q.res_halo) + oy + q.res_halo) * (p.OW + 2 * q.res_halo) + ox + q.res_halo;
            rptr[j] = q.res + (long long)rpix * q.res_cs + (wnB * 64 + 32 * lhB);
            asm volatile("" : "+v"(rptr[j]));
        }
        auto issue_res = [&](auto cc) {
            constexpr int c = decltype(cc)::value;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                chain_gload128_at<c * WGN_B * 64>(rfirst[j], rptr[j]);
                chain_gload128_at<c * WGN_B * 64 + 16>(rsecond[j], rptr[j]);
            }
        };
        static_for<RD>([&](auto Gc) { issue_wB(Gc); });
        issue_res(std::integral_constant<int, 0>());

        // ---- the tile's 3x3 outputs -> t2 (every wave has read the ring's last stage: see the last barrier above)
        {
            unsigned pk[NI][NJ][4];
#pragma unroll
            for (int i = 0; i < NI; ++i) {
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const unsigned trow = tabA + (unsigned)(i * 32 + 8 * gq) * 4u;
                    v4i tc, td;
                    lds_read128_nowait<0>(tc, trow);
                    lds_read128_nowait<CM * 4>(td, trow);
                    wait_lgkm<0>();
                    tie(tc); tie(td);
                    v2s pq[NJ][2];
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int t0 = __mul24(acc[i][j][4 * gq + 2 * h], tc[2 * h]) + td[2 * h];
                            const int t1 = __mul24(acc[i][j][4 * gq + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                            pq[j][h] = as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u));
                        }
                    if (vlo == 0 && vhi == 255) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][gq] = (sat_pk_u8(pq[j][0]) | (sat_pk_u8(pq[j][1]) << 16)) ^ g.t2_xor;
                    } else {
                        const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][gq] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][1], lo1, hi1)),
                                                                 (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][0], lo1, hi1)), 0x06040200u) ^ g.t2_xor;
                    }
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        asm volatile("" : "+v"(pk[i][j][gq]));
                }
            }
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                unsigned qd[NI][4];
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    const auto s02 = __builtin_amdgcn_permlane32_swap(pk[i][j][0], pk[i][j][2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(pk[i][j][1], pk[i][j][3], false, false);
                    qd[i][0] = s02[0]; qd[i][1] = s02[1]; qd[i][2] = s13[0]; qd[i][3] = s13[1];
                }
                v4i first, second;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const auto x = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[1][e], false, false);
                    first[e] = (int)x[0];
                    second[e] = (int)x[1];
                }
                // the lane's 32 channels (wn * 64 + 32 * lh ..) of row r: 16-byte slots wn * 4 + 2 * lh and the next one
                const int r = wm * TM + j * 32 + l32;
                const unsigned sw = (unsigned)(r >> SH) & (unsigned)(CM / 16 - 1);
                const unsigned rowa = lds0 + T2_OFF + (unsigned)r * CM;
                lds_write128(rowa + ((((unsigned)(wn * 4 + 2 * lh)) ^ sw) << 4), first);
                lds_write128(rowa + ((((unsigned)(wn * 4 + 2 * lh + 1)) ^ sw) << 4), second);
            }
        }
        chain_lds_barrier();
        CHAIN_MARK(1);

        // =========================================================== phase B
        const int plo = q.pre.lo, phi = q.pre.hi, slo = q.sum.lo, shi = q.sum.hi;
        const int r0B = wmB * 64 + l32B;
        const unsigned t2row = lds0 + T2_OFF + (unsigned)r0B * CM;
        const unsigned tabB = lds0 + TABB_OFF + (unsigned)(wnB * 64 + 4 * lhB) * 4u;
        const unsigned tabB16 = lds0 + TABB_OFF + 16u * OC + (unsigned)(wnB * 64 + 4 * lhB) * 2u;
        static_for<NCH>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            v16i accB[2][2];
            v4i pf[2][2];
            // (the swizzle is formed again in every chunk: eight fragment addresses kept for the whole phase cost more)
            unsigned swB = ((unsigned)(r0B >> SH) & (unsigned)(CM / 16 - 1)) ^ (unsigned)lhB;
            asm volatile("" : "+v"(swB));
            auto read_t2 = [&](int kk, v4i* dst) {
                const unsigned a = t2row + ((((unsigned)(2 * kk)) ^ swB) << 4);
                lds_read128_nowait<0>(dst[0], a);
                lds_read128_nowait<32 * CM>(dst[1], a);
            };
            read_t2(0, pf[0]);
            static_for<KS>([&](auto kkc) {
                constexpr int kk = decltype(kkc)::value;
                constexpr int G = c * KS + kk;
                wait_lgkm<0>();
                tie(pf[kk & 1][0]); tie(pf[kk & 1][1]);
                if (kk + 1 < KS)
                    read_t2(kk + 1, pf[(kk + 1) & 1]);
                chain_wait_vm<chain_after(KS, NCH, RD, RES_LATE, c, kk)>();
                tie(wfB[G % RD][0]); tie(wfB[G % RD][1]);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        accB[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wfB[G % RD][i], pf[kk & 1][j], kk == 0 ? v16i{} : accB[i][j], 0, 0, 0);
                if constexpr (G + RD < NCH * KS) {
                    // the set is free once its matrix instructions have read it: the compiler orders the load's write
                    // behind them (the load's destination is an output operand of the asm statement)
                    issue_wB(std::integral_constant<int, G + RD>());
                }
                // (keeps the K steps apart: matrix instructions moved later would keep their weight registers with them)
                __builtin_amdgcn_sched_barrier(0);
            });

            CHAIN_MARK(2);
            // ---- the sum's other input, brought into the accumulators' layout (the output's lane-half exchanges backwards)
            unsigned resw[8][2];
            chain_wait_vm<chain_after(KS, NCH, RD, RES_LATE, c, -1)>();
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                tie(rfirst[j]); tie(rsecond[j]);
                unsigned qd[2][4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const auto y = __builtin_amdgcn_permlane32_swap((unsigned)rfirst[j][e], (unsigned)rsecond[j][e], false, false);
                    qd[0][e] = y[0]; qd[1][e] = y[1];
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const auto s02 = __builtin_amdgcn_permlane32_swap(qd[i][0], qd[i][1], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(qd[i][2], qd[i][3], false, false);
                    resw[i * 4 + 0][j] = s02[0];
                    resw[i * 4 + 2][j] = s02[1];
                    resw[i * 4 + 1][j] = s13[0];
                    resw[i * 4 + 3][j] = s13[1];
                }
            }
            if constexpr (!RES_LATE && c + 1 < NCH)
                issue_res(std::integral_constant<int, c + 1>());
            CHAIN_MARK(3);

            // ---- the three rescales on pairs of 16-bit values (see the pipelined kernel's folded sum); the tables of the
            // next channel group are requested before this one is computed
            unsigned pk[2][4];
            // (at three waves per SIMD there are no registers for a second set: a group's tables are requested when it starts)
            constexpr int NSET = WPE == 3 ? 1 : 2;
            v4i rq4[NSET][PRE ? 4 : 2];
            v2i rq2[NSET][3];
            auto request_tables = [&](auto groupc) {
                constexpr int group = decltype(groupc)::value;
                constexpr int set = group & (NSET - 1);
                constexpr int ch = c * WGN_B * 64 + (group / 4) * 32 + 8 * (group % 4);
                lds_read128_nowait<ch * 4>(rq4[set][0], tabB);
                lds_read128_nowait<OC * 4 + ch * 4>(rq4[set][1], tabB);
                if (PRE) {
                    lds_read128_nowait<2 * OC * 4 + ch * 4>(rq4[set][PRE ? 2 : 0], tabB);
                    lds_read128_nowait<3 * OC * 4 + ch * 4>(rq4[set][PRE ? 3 : 0], tabB);
                }
                lds_read64_nowait<ch * 2>(rq2[set][0], tabB16);
                lds_read64_nowait<OC * 2 + ch * 2>(rq2[set][1], tabB16);
                lds_read64_nowait<OC * 4 + ch * 2>(rq2[set][2], tabB16);
            };
            constexpr int NTR = PRE ? 7 : 5;           // reads per request
            request_tables(std::integral_constant<int, 0>());
            const v2s lo1 = splat_v2s(g.e_lo), hi1 = splat_v2s(g.e_hi);
            const v2s lo3 = splat_v2s(plo), hi3 = splat_v2s(phi);
            static_for<8>([&](auto idxc) {
                constexpr int idx = decltype(idxc)::value;
                constexpr int i = idx / 4, gq = idx % 4;
                constexpr int cur = idx & (NSET - 1);
                if constexpr (NSET == 1) {
                    if constexpr (idx > 0)
                        request_tables(std::integral_constant<int, idx>());
                    wait_lgkm<0>();
                } else if constexpr (idx + 1 < 8) {
                    request_tables(std::integral_constant<int, idx + 1>());
                    wait_lgkm<NTR>();
                } else {
                    wait_lgkm<0>();
                }
                tie(rq4[cur][0]); tie(rq4[cur][1]);
                if (PRE) { tie(rq4[cur][PRE ? 2 : 0]); tie(rq4[cur][PRE ? 3 : 0]); }
                tie(rq2[cur][0]); tie(rq2[cur][1]); tie(rq2[cur][2]);
                const v4i tc = rq4[cur][0], td = rq4[cur][1];
                const v2i c16 = rq2[cur][0], d16 = rq2[cur][1], e16 = rq2[cur][2];
                v2s pq[2][2];
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int t0 = __mul24(accB[i][j][4 * gq + 2 * h], tc[2 * h]) + td[2 * h];
                        const int t1 = __mul24(accB[i][j][4 * gq + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                        pq[j][h] = clamp_v2s(as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u)), lo1, hi1);
                    }
                v2s oq[2][2];
                if constexpr (PRE) {
                    const v4i xc = rq4[cur][PRE ? 2 : 0], xd = rq4[cur][PRE ? 3 : 0];
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const unsigned w = resw[idx][j] ^ q.res_flip;
                        unsigned u[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            u[e] = __umul24((w >> (8 * e)) & 0xffu, (unsigned)xc[e]) + (unsigned)xd[e];
                        oq[j][0] = as_v2s((int)__builtin_amdgcn_perm(u[1], u[0], 0x07060302u));
                        oq[j][1] = as_v2s((int)__builtin_amdgcn_perm(u[3], u[2], 0x07060302u));
                    }
                    if (!q.pre_in_range) {
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            oq[j][0] = clamp_v2s(oq[j][0], lo3, hi3);
                            oq[j][1] = clamp_v2s(oq[j][1], lo3, hi3);
                        }
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const unsigned w = resw[idx][j] ^ q.res_flip;
                        oq[j][0] = as_v2s((int)__builtin_amdgcn_perm(w, w, 0x0c010c00u));
                        oq[j][1] = as_v2s((int)__builtin_amdgcn_perm(w, w, 0x0c030c02u));
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        v2s v = pq[j][h] + oq[j][h];
                        v = v * as_v2s(c16[h]) + as_v2s(d16[h]);
                        pq[j][h] = v >> as_v2s(e16[h]);
                    }
                if (slo == 0 && shi == 255) {
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        pk[j][gq] = (sat_pk_u8(pq[j][0]) | (sat_pk_u8(pq[j][1]) << 16)) ^ p.out_xor;
                } else {
                    const v2s lo2 = splat_v2s(slo), hi2 = splat_v2s(shi);
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        pk[j][gq] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][1], lo2, hi2)),
                                                          (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][0], lo2, hi2)), 0x06040200u) ^ p.out_xor;
                }
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    asm volatile("" : "+v"(pk[j][gq]));
                if constexpr (gq == 3) {
                    // a 32-channel tile is done: one exchange between the lane halves leaves every lane with 16 consecutive
                    // channels (16 * lh ..) of its pixel; the two halves of a lane pair write 32 consecutive bytes
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const auto s02 = __builtin_amdgcn_permlane32_swap(pk[j][0], pk[j][2], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(pk[j][1], pk[j][3], false, false);
                        const v4i piece = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
                        const unsigned off = live[j] ? (unsigned)(opix[j] + c * WGN_B * 64 + i * 32) : 0x80000000u;
                        __builtin_amdgcn_raw_buffer_store_b128(piece, out_rsrc, off, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);      // one group's tables at a time
            });
            if constexpr (RES_LATE && c + 1 < NCH)
                issue_res(std::integral_constant<int, c + 1>());
            CHAIN_MARK(4);
        });
        // every wave has read t2: the next tile's ring may take its place
        chain_lds_barrier();
        CHAIN_MARK(5);
    }
#ifdef N2D2HIP_PROFILE
    if (tid == 0 && g.prof) {
        // the common record, then the time in: the 3x3 loop; the hand-over through LDS; the expansion's K loops; the wait
        // for the sum's other input; the rescales and stores; the last barrier
        long long* o = g.prof + (long long)blockIdx.x * 16;
        o[0] = pr_t0; o[1] = pr_t0; o[2] = pr_t2; o[3] = clock64(); o[4] = pr[3] + pr[4]; o[5] = pr_w0; o[6] = wall_clock64(); o[7] = ntile;
        for (int k = 0; k < 6; ++k) o[8 + k] = pr[k];
    }
#endif
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
}

bool conv_chain_channels(int cmid) { return cmid == 64 || cmid == 128 || cmid == 256; }

size_t conv_chain_weight_bytes(int C, int O) { return (size_t)C * O; }

void conv_chain_weight_layout(const signed char* w, int row_bytes, int C, int O, signed char* frag)
{
    // [chunk of 64 outputs][K step][32-output tile of the chunk][lane]: a wave reads a chunk's fragments in this order
    const int ks = C / 32;
    for (int chunk = 0; chunk < O / 64; ++chunk)
        for (int kk = 0; kk < ks; ++kk)
            for (int i = 0; i < 2; ++i)
                for (int lane = 0; lane < 64; ++lane) {
                    const int o = chunk * 64 + i * 32 + (lane & 31), ch = kk * 32 + (lane >> 5) * 16;
                    memcpy(frag + ((((size_t)chunk * ks + kk) * 2 + i) * 64 + lane) * 16, w + (size_t)o * row_bytes + ch, 16);
                }
}

int conv_chain_launch(ConvChainArgs a, int num_cus, hipStream_t stream)
{
    const int cm = a.p.c.in_cs;
    N2D2HIP_REQUIRE(conv_chain_channels(cm), N2D2HIP_ERR_INVALID, "conv_chain: %d middle channels", cm);
    const int BM = 128, BK = cm == 128 ? 128 : 64;
    N2D2HIP_REQUIRE(a.p.c.ktot % BK == 0 && a.p.c.ktot / BK >= 4, N2D2HIP_ERR_INVALID, "conv_chain: K of %d bytes", a.p.c.ktot);
    a.p.c.niter = a.p.c.ktot / BK;
    a.p.cper = cm / BK;
    a.p.mtiles = (a.p.c.M + BM - 1) / BM;
    // three (64 middle channels) or two work-groups of four waves per compute unit, or one of eight
    const int per_xcd = std::max(1, std::min((a.p.mtiles + 7) / 8, (cm == 256 ? 1 : cm == 64 ? 3 : 2) * num_cus / 8));
    a.p.mlanes = per_xcd;
    a.p.xcd_tiles = (a.p.mtiles + 7) / 8;
    const int grid = 8 * per_xcd;
#ifdef N2D2HIP_PROFILE
    a.prof = nullptr;      // probe builds: launch_kernel() points it at this launch's records
#endif
    const bool pre = a.p.has_pre != 0;
    if (cm == 256) {
        if (pre) N2D2HIP_LAUNCH_T(conv_chain_kernel, (256, 64, 4, 2, 2, true), dim3(grid), dim3(512), 0, stream, a);
        else N2D2HIP_LAUNCH_T(conv_chain_kernel, (256, 64, 4, 2, 2, false), dim3(grid), dim3(512), 0, stream, a);
    } else if (cm == 128) {
        if (pre) N2D2HIP_LAUNCH_T(conv_chain_kernel, (128, 128, 2, 2, 2, true), dim3(grid), dim3(256), 0, stream, a);
        else N2D2HIP_LAUNCH_T(conv_chain_kernel, (128, 128, 2, 2, 2, false), dim3(grid), dim3(256), 0, stream, a);
    } else {
        if (pre) N2D2HIP_LAUNCH_T(conv_chain_kernel, (64, 64, 3, 1, 4, true, 3), dim3(grid), dim3(256), 0, stream, a);
        else N2D2HIP_LAUNCH_T(conv_chain_kernel, (64, 64, 3, 1, 4, false, 3), dim3(grid), dim3(256), 0, stream, a);
    }
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // namespace n2d2hip
