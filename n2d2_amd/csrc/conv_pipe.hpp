// Persistent, software-pipelined implicit-GEMM convolution for int8 weights
// and activations whose channel count is a multiple of 64.
//
// What bounds such a layer on this chip is not memory but instruction issue:
// a 32x32x32 int8 MFMA keeps a SIMD's matrix core busy for 32 cycles, every
// other vector instruction costs 4 cycles of the same SIMD, and rescaling one
// accumulator to a byte takes 4-5 of them.  The kernel is organised so that the
// matrix core never waits for anything that can be had earlier:
//  * operands go global -> LDS by direct loads (global_load_lds_dwordx4) into an
//    S-stage ring that runs across tile boundaries; the loads of a step are
//    issued S-1 steps before they are consumed, so S-1 stages are in flight;
//  * fragments go LDS -> registers one MFMA K step (32 of K) ahead: while the
//    MFMAs of one K step run, the ds_reads of the next are in flight, into the
//    other of two register sets;
//  * one barrier per stage, at its last K step, hands a stage over in both
//    directions (the next stage has landed for everybody; this stage has been
//    read by everybody and is refilled at once);
//  * a block keeps one channel tile for its whole life and walks pixel tiles:
//    bias lives in registers and is the C operand of a tile's first MFMAs, the
//    rescale tables live in LDS;
//  * the epilogue has no LDS staging and no barrier: rescaled values are packed
//    to bytes, exchanged between the two lane halves (v_permlane32_swap) until
//    a lane owns 16 or 32 consecutive channels of its pixel, and stored;
//  * the steady state carries no address arithmetic for 1x1 kernels (uniform
//    base + constant per-lane offset), and for KxK kernels one validity bit
//    per tap and row, computed once per tile.
//
// Because the loads complete asynchronously, LDS accesses are explicit inline
// ds_* instructions and the waits are written by hand.  s_waitcnt vmcnt(n)
// counts the youngest operations that may still be outstanding; loads return
// in order, so "at most n outstanding" implies every load older than the
// youngest n has landed, whatever the epilogue's stores (which also count) do.
// A thread issues the same number of loads at every step: steps past the end
// of its work fetch rows that are marked invalid.
#pragma once

#include "conv_args.hpp"
#include "epilogue.hpp"
#include "mfma_util.hpp"

namespace n2d2hip {

struct ConvPipeArgs {
    ConvArgs c;
    const signed char* fill16;   // 16 bytes of the input's logical zero (device)
    int mtiles;                  // pixel tiles
    int xcd_tiles;               // consecutive pixel tiles given to one XCD
    int mlanes;                  // blocks of one XCD (and channel tile) that share its pixel tiles
    int cper;                    // 64-byte K steps per kernel tap (C / 64)
    int kW, kH;
    unsigned ohw_mul, ohw_sh, ow_mul, ow_sh;     // division by OH*OW and by OW
    int preclamp;                // I24: clamp before the multiply; F32: the cell has a Clip
    int out_halo;                // border pixels around every output image (byte outputs only)
    int out_pixels;              // pixels of the output buffer, borders included
    // Folded residual sum (RES kernels): out = sum_act(conv_act(conv) + pre(other)), all EPI_I24
    const signed char* res;      // the sum's other input, NHWC bytes
    int res_cs;
    int res_halo;                // border of zeros around every image of the other input
    unsigned res_flip;           // turns a stored byte into an unsigned one (0x80808080 unless plain U8 storage)
    EpiArgs sum;                 // the sum cell's rescale; its d table has the other input's zero point folded in
    EpiArgs pre;                 // ScalingCell folded onto the other input (d table with the zero point folded in)
    int has_pre, pre_clamp, sum_clamp;
    // The sum's multiplier, addend and shift as pairs of 16-bit values (channels 2k, 2k+1 in one dword), three arrays of
    // sum16_stride dwords, when the host has shown that the sum's arithmetic stays inside 16 bits; else null.
    const int* sum16;
    int sum16_stride;
    int pre_in_range;            // with sum16: the ScalingCell's result cannot leave its range, no saturation needed
#ifdef N2D2HIP_PROFILE
    long long* prof;             // one 16-counter record per block
#endif
};

// 16-byte slot of (row, logical slot s) in a [rows][BK bytes] tile.  The XOR spreads the rows that one
// ds_read_b128 touches for a fixed s over all banks.
template <int BK>
__device__ __forceinline__ int swz_k(int row, int s)
{
    return BK == 64 ? ((row << 2) + (s ^ ((row >> 2) & 3))) << 4 : ((row << 3) + (s ^ ((row >> 1) & 7))) << 4;
}

// NW waves as WGM (pixels) x NW/WGM (channels); a wave owns NJ x NI MFMA tiles of 32 pixels x 32 channels.
// BK: bytes of K per ring stage and row (64 or 128); 128 makes every row segment a whole 128-byte line, which is
// what the L2 -> LDS path moves fastest.
// RES: the residual sum that follows the convolution is computed in the epilogue (1x1 convolutions, EPI_I24).
// P16: the integer rescale's tables come scaled up so that the result is the upper half of a 32-bit register (no
// shift), and what follows runs on pairs of 16-bit values: with RES the whole sum, without it the saturation and the
// pack.  The host chooses it when it has shown that nothing overflows.
// VALID: 0 = windows may reach outside the input (per-tap validity bits), 1 = 1x1 kernel without padding, 2 = any kernel
// without padding (every tap of every window inside the input: a tap only moves the uniform base address).
// W4: 4-bit weights.  They stay packed two per byte in memory and in LDS (p.w is then an image of the ring's weight
// tiles: per 32 channels and 64 of K one 1 KB chunk, laid out as the LDS wants it) and are widened to bytes on their way
// from LDS to the matrix core, as 16 times their value: the nibble becomes the upper half of its byte, which one AND
// (upper nibbles) or a shift and an AND (lower nibbles) do for four weights at once.  The accumulators are divided by
// 16, exactly, before they are rescaled.
template <int NW, int BK, int NI, int NJ, int WGM, int EPI, int S, int VALID, bool RES = false, bool P16 = false, bool W4 = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_pipe_kernel(ConvPipeArgs q)
{
    const ConvArgs& p = q.c;
    constexpr int NT = NW * 64;                        // threads
    constexpr int WGN = NW / WGM;
    constexpr int TM = 32 * NJ, TN = 32 * NI;          // pixels x channels of a wave
    constexpr int BM = TM * WGM, BN = TN * WGN;        // of the block
    constexpr int LPR = BK / 16;                       // lanes (16-byte slots) per row
    constexpr int RPC = 64 / LPR;                      // rows per 1 KB chunk = per wave-wide load
    constexpr int KH = BK / 32;                        // MFMA K steps per stage
    constexpr int TOFF = 32 * BK;                      // LDS bytes between MFMA tiles of one operand
    // chunks each wave loads per step; when there are fewer chunks than waves some are loaded twice
    constexpr int WROW = W4 ? BK / 2 : BK;             // bytes of a weight row per stage
    constexpr int KCH = BK / 64;                       // W4: 1 KB weight chunks (32 channels x 64 of K) per channel block and stage
    constexpr int A_CH = BM / RPC, B_CH = W4 ? (BN / 32) * KCH : BN / RPC;
    constexpr int A_J = (A_CH + NW - 1) / NW, B_J = (B_CH + NW - 1) / NW;
    constexpr int LPI = A_J + B_J;                     // loads per thread and step
    constexpr int STAGE = BM * BK + BN * WROW;
    constexpr int TAB_OFF = S * STAGE;                 // 6 int arrays of BN entries: bias, a, b, c, d, e
    // RES: + a..e of the sum cell, + a..e of the folded ScalingCell.  When the sum runs on 16-bit pairs, its c, d, e in
    // that form take the place of the bias and the convolution's a, which that path does not use.
    constexpr int NTAB = RES ? 16 : 6;
    static_assert(!RES || EPI == EPI_I24, "the folded sum is integer arithmetic");
    constexpr int NF = NI + NJ;                        // fragment reads per MFMA K step
    constexpr bool BIAS_REG = EPI != EPI_I24;          // the integer rescale carries the bias in its tables
    static_assert(BK == 64 || BK == 128, "K bytes per stage");
    static_assert(WGM * WGN == NW && BM % RPC == 0 && BN % RPC == 0, "wave grid");
    static_assert(BK == 64 || (NW % 2 == 0 && A_CH % 2 == 0 && B_CH % 2 == 0), "a wave's chunks keep their parity");
    static_assert(S >= 2, "ring depth");
    static_assert(!W4 || EPI == EPI_I24, "packed weights: integer rescale with the bias in its tables");
    static_assert(LPI * (S - 1) < 60, "vmcnt is a 6-bit counter");
    static_assert((NJ - 1) * TOFF < 65536 && NTAB * BN * 4 + 256 < 65536, "ds_read immediate offsets are 16 bits");

    __shared__ __attribute__((aligned(16))) unsigned char smem[TAB_OFF + NTAB * BN * 4];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int l32 = lane & 31, lh = lane >> 5;

    // ---- which tiles this block walks: one channel tile, every mlanes-th pixel tile of its XCD's run.
    // Blocks 8 apart run on the same XCD; they take the same pixel tiles for neighbouring channel tiles.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % p.ntiles_n;
    // An XCD gets a run of consecutive pixel tiles (neighbouring tiles share their window halo through that XCD's L2)
    // and its blocks take them in turn.
    const int mlane = xcd * q.xcd_tiles + slot / p.ntiles_n;
    const int mend = min((xcd + 1) * q.xcd_tiles, q.mtiles);
    const int n0 = tile_n * BN;
    const int ntile = (mlane < mend) ? (mend - mlane + q.mlanes - 1) / q.mlanes : 0;
    const int niter = p.niter;
#ifdef N2D2HIP_PROFILE
    long long pr_t0 = clock64(), pr_t1 = 0, pr_t2 = 0, pr_t3 = 0, pr_epi = 0, pr_w0 = wall_clock64();
#endif

    // ---- loader state.  Lane l of a wave fills 16-byte slot l of a 1 KB chunk: row l/LPR of the chunk,
    // physical slot l%LPR, which holds the logical slot swz_k() maps there (chunk parity is the wave's parity).
    const int lrow = lane / LPR;
    const int lq = BK == 64 ? (lane & 3) ^ ((lane >> 4) & 3) : (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4));
    unsigned woff[B_J];            // byte offset of this thread's weight rows (without the K offset)
#pragma unroll
    for (int j = 0; j < B_J; ++j)
        woff[j] = W4 ? (unsigned)(((n0 / 32 + ((wave + NW * j) % B_CH) / KCH) * (p.niter * KCH) + ((wave + NW * j) % B_CH) % KCH) * 1024 + lane * 16)
                     : (unsigned)((n0 + ((wave + NW * j) % B_CH) * RPC + lrow) * p.ktot + lq * 16);
    int rowoff[A_J];               // byte offset of the window origin of this thread's pixel rows (+ sub-chunk)
    unsigned rowmask[A_J];         // bit t < 31: kernel tap t of the row reads inside the input; bit 31: undilated window
    int l_tile = 0, l_it = 0, l_koff = 0, l_stage = 0;
    int l_c = 0, l_kx = 0, l_ky = 0, l_tap = 0, l_tapoff = 0, l_ctapoff = 0;
    const bool dilated = p.dilX != 1 || p.dilY != 1;
    const int dil_kw = q.kW + (p.dilX - 1) * (q.kW - 1), dil_kh = q.kH + (p.dilY - 1) * (q.kH - 1);
    constexpr bool ALLVALID = VALID != 0;
    constexpr bool kxk = VALID == 2;
    auto loader_new_tile = [&]() {
        const int m0 = (mlane + l_tile * q.mlanes) * BM;
#pragma unroll
        for (int j = 0; j < A_J; ++j) {
            const int m = m0 + ((wave + NW * j) % A_CH) * RPC + lrow;
            // branch-free (the block-uniform loader state must stay in scalar registers): rows past the end of
            // the work are computed like pixel 0 and then masked
            const bool live = (l_tile < ntile) & (m < p.M);
            const int mm = live ? m : 0;
            const int b = div_magic(mm, q.ohw_mul, q.ohw_sh);
            const int rem = mm - b * (p.OH * p.OW);
            const int oy = div_magic(rem, q.ow_mul, q.ow_sh);
            const int ox = rem - oy * p.OW;
            const int by = oy * p.strideY - p.padT, bx = ox * p.strideX - p.padL;
            rowoff[j] = ((b * p.H + by) * p.W + bx) * p.in_cs + lq * 16;
            rowmask[j] = 0u;
            if (!ALLVALID) {
                // tap index >= max(pad - o*stride, 0) and dilated offset inside the input
                // (ref: src/Cell/ConvCell_Frame_Kernels.cpp:72-83)
                unsigned xmask = 0u;
                for (int kx = 0; kx < q.kW; ++kx)
                    xmask |= (unsigned)((kx >= -bx) & (kx * p.dilX < p.W - bx)) << kx;
                unsigned mk = 0u;
                for (int ky = 0; ky < q.kH; ++ky)
                    mk |= ((ky >= -by) & (ky * p.dilY < p.H - by)) ? (xmask << (ky * q.kW)) : 0u;
                // The reference unrolls "a 3x3 window fully inside" by hand, recognising it by its tap bounds alone
                // (ref: src/Cell/ConvCell_Frame_Kernels.cpp:95-117): a dilated kernel whose bounds happen to be
                // [0,3) x [0,3) is evaluated there with its first 3x3 taps at undilated offsets.
                const int sx_max = min(max(p.W - bx, 0), dil_kw), sy_max = min(max(p.H - by, 0), dil_kh);
                if (dilated && bx >= 0 && by >= 0 && sx_max == 3 && sy_max == 3)
                    mk = 0x80000000u | 7u | (7u << q.kW) | (7u << (2 * q.kW));
                rowmask[j] = live ? mk : 0u;
            }
        }
    };
    loader_new_tile();

    // Issues the LPI loads of the loader's current step into its current ring stage, then advances the loader.
    auto issue = [&]() {
        unsigned char* sbase = smem + l_stage * STAGE;
        if (ALLVALID) {
            // uniform; rows past the end read pixel 0.  Without padding every tap of every window lies inside the
            // input, whatever the kernel size: a tap only moves the uniform base.
            const signed char* ibase = p.in + (kxk ? l_tapoff : l_koff);
#pragma unroll
            for (int j = 0; j < A_J; ++j)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(ibase + (unsigned)rowoff[j]), (lds_ptr_t)(sbase + ((wave + NW * j) % A_CH) * 1024), 16, 0, 0);
        } else {
            const unsigned tapbit = 1u << l_tap;
#pragma unroll
            for (int j = 0; j < A_J; ++j) {
                const int toff = (int)rowmask[j] < 0 ? l_ctapoff : l_tapoff;
                const signed char* src = (rowmask[j] & tapbit) ? p.in + (rowoff[j] + toff) : q.fill16;
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)(sbase + ((wave + NW * j) % A_CH) * 1024), 16, 0, 0);
            }
        }
        const signed char* wbase = p.w + (W4 ? l_it * (KCH * 1024) : l_koff);
#pragma unroll
        for (int j = 0; j < B_J; ++j)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(wbase + woff[j]), (lds_ptr_t)(sbase + BM * BK + ((wave + NW * j) % B_CH) * 1024), 16, 0, 0);
        l_stage = (l_stage + 1 == S) ? 0 : l_stage + 1;
        l_koff += BK;
        if (++l_it == niter) {
            l_it = 0; l_koff = 0;
            l_c = 0; l_kx = 0; l_ky = 0; l_tap = 0; l_tapoff = 0; l_ctapoff = 0;
            ++l_tile;
            loader_new_tile();
        } else if (!ALLVALID || kxk) {
            l_tapoff += BK;
            l_ctapoff += BK;
            if (++l_c == q.cper) {
                l_c = 0;
                ++l_tap;
                if (++l_kx == q.kW) { l_kx = 0; ++l_ky; }
                l_tapoff = (l_ky * p.dilY * p.W + l_kx * p.dilX) * p.in_cs;
                l_ctapoff = (l_ky * p.W + l_kx) * p.in_cs;
            }
        }
    };

    // ---- fragment addresses of the stage to read next: (operand, MFMA K step); tiles are immediates
    unsigned pa[KH], wa[KH];
#pragma unroll
    for (int kk = 0; kk < KH; ++kk) {
        pa[kk] = lds0 + swz_k<BK>(wm * TM + l32, 2 * kk + lh);
        // (W4: the chunk of this wave's first channel block that holds K step kk, then the lane's row and 8-byte slot in it)
        wa[kk] = W4 ? lds0 + BM * BK + (wn * NI * KCH + kk / 2) * 1024 + l32 * 32 + (((2 * (kk % 2) + lh) ^ ((l32 >> 3) & 3)) << 3)
                    : lds0 + BM * BK + swz_k<BK>(wn * TN + l32, 2 * kk + lh);
    }
    int r_stage = 0;
    const unsigned tab = lds0 + TAB_OFF + (unsigned)(wn * TN + 4 * lh) * 4u;      // this lane's first channel in the tables
    const unsigned tab16 = lds0 + TAB_OFF + (unsigned)(wn * TN + 4 * lh) * 2u;    // and in the 16-bit pairs
    constexpr bool p16 = RES && P16;
    static_assert(!P16 || EPI == EPI_I24, "16-bit pairs follow the integer rescale");

    // two fragment sets: while the MFMAs of K step g run from set g%2, the reads of step g+1 fly into the other
    v4i fw[2][NI], fp[2][NJ];
    v2i fw4[2][W4 ? NI : 1];       // W4: the packed fragments as they come from LDS
    auto read_k = [&](auto kkc) {
        constexpr int kk = decltype(kkc)::value;
        constexpr int set = kk & 1;
        if (W4) {
            lds_read64_nowait<0>(fw4[set][0], wa[kk]);
            if (NI > 1) lds_read64_nowait<KCH * 1024>(fw4[set][W4 && NI > 1 ? 1 : 0], wa[kk]);
        } else {
            lds_read128_nowait<0>(fw[set][0], wa[kk]);
            if (NI > 1) lds_read128_nowait<TOFF>(fw[set][NI > 1 ? 1 : 0], wa[kk]);
        }
        lds_read128_nowait<0>(fp[set][0], pa[kk]);
        if (NJ > 1) lds_read128_nowait<TOFF>(fp[set][NJ > 1 ? 1 : 0], pa[kk]);
        if (NJ > 2) lds_read128_nowait<2 * TOFF>(fp[set][NJ > 2 ? 2 : 0], pa[kk]);
        if (NJ > 3) lds_read128_nowait<3 * TOFF>(fp[set][NJ > 3 ? 3 : 0], pa[kk]);
        if (kk == KH - 1) {
            // every K step of this stage is requested: move on to the next stage of the ring
            const bool wrap = r_stage + 1 == S;
            const unsigned inc = wrap ? (unsigned)(-(S - 1) * STAGE) : (unsigned)STAGE;
            r_stage = wrap ? 0 : r_stage + 1;
#pragma unroll
            for (int k2 = 0; k2 < KH; ++k2) { pa[k2] += inc; wa[k2] += inc; }
        }
    };

    // RES: the other input's bytes for this lane's accumulators.  They are read the way the output is written, 32
    // consecutive channels of a pixel per lane (whole 32-byte sectors, every line touched once), one tile ahead: the
    // loads of tile t+1 are issued at the start of tile t's epilogue and have a whole epilogue and K loop to arrive.
    // Rows past the end read pixel 0, so the number of loads issued never depends on the data.
    constexpr int NST = 2 * NJ;                        // RES: stores per thread and tile
    static_assert(!RES || (S * LPI >= NST && NST + LPI < 60), "enough younger operations behind the first tile's residual loads");
    v4i rfirst[RES ? NJ : 1], rsecond[RES ? NJ : 1];
    auto issue_res = [&](int c_tile) {
        const int m0 = (mlane + c_tile * q.mlanes) * BM;
#pragma unroll
        for (int j = 0; j < (RES ? NJ : 0); ++j) {
            const int m = m0 + wm * TM + j * 32 + l32;
            int rpix = m < p.M ? m : 0;
            if (q.res_halo != 0) {
                // the other input carries a border: its pixel sits past the borders of its image
                const int b = div_magic(rpix, q.ohw_mul, q.ohw_sh);
                const int rem = rpix - b * (p.OH * p.OW);
                const int oy = div_magic(rem, q.ow_mul, q.ow_sh);
                const int ox = rem - oy * p.OW;
                rpix = (b * (p.OH + 2 * q.res_halo) + oy + q.res_halo) * (p.OW + 2 * q.res_halo) + ox + q.res_halo;
            }
            const signed char* rp = q.res + (long long)rpix * q.res_cs + (n0 + wn * TN + 32 * lh);
            asm volatile("global_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %1, %2, off offset:16"
                         : "=&v"(rfirst[j]), "=&v"(rsecond[j]) : "v"(rp) : "memory");
        }
    };
    // RES: the output goes through a buffer descriptor whose bounds check drops the rows past the end, so that every
    // thread issues the same number of stores
    __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, RES ? q.out_pixels * p.out_cs : 0, 0x00020000);
    // Position of output pixel m in the output buffer: m itself, or past the borders of a tensor with a halo
    auto out_pix = [&](int m) -> int {
        if (q.out_halo == 0)
            return m;
        const int mm = m < p.M ? m : 0;
        const int b = div_magic(mm, q.ohw_mul, q.ohw_sh);
        const int rem = mm - b * (p.OH * p.OW);
        const int oy = div_magic(rem, q.ow_mul, q.ow_sh);
        const int ox = rem - oy * p.OW;
        return (b * (p.OH + 2 * q.out_halo) + oy + q.out_halo) * (p.OW + 2 * q.out_halo) + ox + q.out_halo;
    };

    v16i acc[NI][NJ];
    const bool out_bytes = p.out_dtype != N2D2HIP_I32;
    const int vlo = p.epi.lo, vhi = p.epi.hi;
    const float flo = (float)p.epi.lo, fhi = (float)p.epi.hi;
    const int plo = q.pre.lo, phi = q.pre.hi, slo = q.sum.lo, shi = q.sum.hi;

    // ---- rescale, pack and store the finished tile
    auto epilogue = [&](int c_tile) {
        const int m0 = (mlane + c_tile * q.mlanes) * BM;
        if (W4) {
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        acc[i][j][e] >>= 4;
        }
        unsigned pk[NI][NJ][4];
        // RES: the other input's bytes, 4 channels per dword, are brought into the accumulators' layout by running the
        // output's lane-half exchanges backwards (the exchange is its own inverse).  Memory operations complete in
        // issue order: behind this tile's residual loads came the previous tile's NST stores and at least one step of
        // ring loads (for the first tile, the ring's fill), so they have landed once no more than that is in flight.
        unsigned resw[RES ? NI * 4 : 1][RES ? NJ : 1];
        if (RES) {
            static_assert(!RES || NI == 2, "the folded sum is written for two channel tiles per wave");
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NST + LPI) : "memory");
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                tie(rfirst[RES ? j : 0]); tie(rsecond[RES ? j : 0]);
                unsigned qd[2][4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const auto y = __builtin_amdgcn_permlane32_swap((unsigned)rfirst[RES ? j : 0][e], (unsigned)rsecond[RES ? j : 0][e], false, false);
                    qd[0][e] = y[0]; qd[1][e] = y[1];
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const auto s02 = __builtin_amdgcn_permlane32_swap(qd[i][0], qd[i][1], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(qd[i][2], qd[i][3], false, false);
                    resw[RES ? i * 4 + 0 : 0][RES ? j : 0] = s02[0];
                    resw[RES ? i * 4 + 2 : 0][RES ? j : 0] = s02[1];
                    resw[RES ? i * 4 + 1 : 0][RES ? j : 0] = s13[0];
                    resw[RES ? i * 4 + 3 : 0][RES ? j : 0] = s13[1];
                }
            }
            issue_res(c_tile + 1);
        }
        // Without a folded sum, the convolution's tables of the next channel group are requested before this group is
        // rescaled (two register sets), so that their LDS latency is hidden behind the arithmetic.
        v4i tq[2][5];
        // Every register such a read fills must be tied after the wait, used or not: a register the compiler takes for
        // dead is handed to other values while the read is still on its way.  So only what is used is requested.
        auto request_tables = [&](v4i* t, unsigned trow) {
            if (!P16) lds_read128_nowait<BN * 4>(t[0], trow);
            if (!P16) lds_read128_nowait<2 * BN * 4>(t[1], trow);
            lds_read128_nowait<3 * BN * 4>(t[2], trow);
            if (EPI == EPI_I24) lds_read128_nowait<4 * BN * 4>(t[3], trow);
            if (EPI != EPI_F32 && !P16) lds_read128_nowait<5 * BN * 4>(t[4], trow);
        };
        constexpr int NTR = P16 ? 2 : 3 + (EPI == EPI_I24 ? 1 : 0) + (EPI != EPI_F32 ? 1 : 0);      // reads per request
        if (!RES && EPI != EPI_RAW)
            request_tables(tq[0], tab);
        // The folded sum on 16-bit pairs reads seven tables per channel group: they too are requested one group ahead.
        v4i rq4[2][4];
        v2i rq2[2][3];
        auto request_sum_tables = [&](int set, int group) {
            const unsigned t32 = tab + (unsigned)((group / 4) * 32 + 8 * (group % 4)) * 4u;
            const unsigned t16 = tab16 + (unsigned)((group / 4) * 32 + 8 * (group % 4)) * 2u;
            lds_read128_nowait<3 * BN * 4>(rq4[set][0], t32);
            lds_read128_nowait<4 * BN * 4>(rq4[set][1], t32);
            // (the ScalingCell's tables are read whether there is one or not: two reads of whatever the LDS holds cost less
            // than a branch here)
            lds_read128_nowait<13 * BN * 4>(rq4[set][2], t32);
            lds_read128_nowait<14 * BN * 4>(rq4[set][3], t32);
            lds_read64_nowait<0>(rq2[set][0], t16);
            lds_read64_nowait<BN * 2>(rq2[set][1], t16);
            lds_read64_nowait<BN * 4>(rq2[set][2], t16);
        };
        if (RES && P16)
            request_sum_tables(0, 0);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int idx = i * 4 + g;
                const unsigned trow = tab + (unsigned)(i * 32 + 8 * g) * 4u;
                if constexpr (RES && P16) {
                    // ---- the same three rescales with everything behind the convolution's shift held as pairs of
                    // 16-bit values (channels 2h, 2h+1 of the lane's four): half the instructions per value.  The host
                    // has shown that no intermediate leaves 16 bits and that none of the optional clamps is needed.
                    // The convolution's and the ScalingCell's multipliers and addends come scaled up by 2^(16 - shift):
                    // the rescaled value is the upper half of the 32-bit result and needs no shift of its own.
                    constexpr int SET = (RES && P16) ? 1 : 0;     // (keeps the other instantiations' indices in range)
                    const int cur = (idx & 1) * SET;
                    if (idx + 1 < NI * 4) {
                        request_sum_tables(((idx + 1) & 1) * SET, idx + 1);
                        wait_lgkm<7>();        // the LDS answers in order: this group's seven reads have arrived
                    } else {
                        wait_lgkm<0>();
                    }
                    // (every register a read fills is tied after the wait: see above)
                    tie(rq4[cur][0]); tie(rq4[cur][1]); tie(rq4[cur][2]); tie(rq4[cur][3]);
                    tie(rq2[cur][0]); tie(rq2[cur][1]); tie(rq2[cur][2]);
                    const v4i tc = rq4[cur][0], td = rq4[cur][1], xc = rq4[cur][2], xd = rq4[cur][3];
                    const v2i c16 = rq2[cur][0], d16 = rq2[cur][1], e16 = rq2[cur][2];
                    const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
                    v2s pq[NJ][2];
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int t0 = __mul24(acc[i][j][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                            const int t1 = __mul24(acc[i][j][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                            pq[j][h] = clamp_v2s(as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u)), lo1, hi1);
                        }
                    v2s oq[NJ][2];
                    if (q.has_pre) {
                        const v2s lo3 = splat_v2s(plo), hi3 = splat_v2s(phi);
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
                            const unsigned w = resw[RES ? idx : 0][RES ? j : 0] ^ q.res_flip;
                            unsigned u[4];
#pragma unroll
                            for (int t = 0; t < 4; ++t)
                                u[t] = __umul24((w >> (8 * t)) & 0xffu, (unsigned)xc[t]) + (unsigned)xd[t];
                            oq[j][0] = as_v2s((int)__builtin_amdgcn_perm(u[1], u[0], 0x07060302u));
                            oq[j][1] = as_v2s((int)__builtin_amdgcn_perm(u[3], u[2], 0x07060302u));
                        }
                        if (!q.pre_in_range) {
#pragma unroll
                            for (int j = 0; j < NJ; ++j) {
                                oq[j][0] = clamp_v2s(oq[j][0], lo3, hi3);
                                oq[j][1] = clamp_v2s(oq[j][1], lo3, hi3);
                            }
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
                            const unsigned w = resw[RES ? idx : 0][RES ? j : 0] ^ q.res_flip;
                            oq[j][0] = as_v2s((int)__builtin_amdgcn_perm(w, w, 0x0c010c00u));
                            oq[j][1] = as_v2s((int)__builtin_amdgcn_perm(w, w, 0x0c030c02u));
                        }
                    }
                    const v2s lo2 = splat_v2s(slo), hi2 = splat_v2s(shi);
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            v2s v = pq[j][h] + oq[j][h];
                            v = v * as_v2s(c16[h]) + as_v2s(d16[h]);
                            pq[j][h] = v >> as_v2s(e16[h]);
                        }
                    if (slo == 0 && shi == 255) {
                        // the usual range of a rectified sum has an instruction of its own
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][g] = (sat_pk_u8(pq[j][0]) | (sat_pk_u8(pq[j][1]) << 16)) ^ p.out_xor;
                    } else {
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][g] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][1], lo2, hi2)),
                                                                (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][0], lo2, hi2)), 0x06040200u) ^ p.out_xor;
                    }
                    // Keeps the groups apart (their results are needed only after the last one, and the compiler would
                    // otherwise compute them all there, with every group's tables live at once).
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        asm volatile("" : "+v"(pk[i][j][g]));
                } else if constexpr (P16) {
                    // ---- plain convolution, byte output: multiply-add, take the upper halves, saturate and pack.  The
                    // tables of the next channel group are requested before this one is rescaled.
                    if (idx + 1 < NI * 4) {
                        const int nx = idx + 1;
                        request_tables(tq[nx & 1], tab + (unsigned)((nx / 4) * 32 + 8 * (nx % 4)) * 4u);
                        wait_lgkm<NTR>();
                    } else {
                        wait_lgkm<0>();
                    }
                    // (the wait is tied to the registers the reads write, not to copies the compiler could make early)
                    tie(tq[idx & 1][2]); tie(tq[idx & 1][3]);
                    const v4i tc = tq[idx & 1][2], td = tq[idx & 1][3];
                    v2s pq[NJ][2];
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int t0 = __mul24(acc[i][j][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                            const int t1 = __mul24(acc[i][j][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                            pq[j][h] = as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u));
                        }
                    if (vlo == 0 && vhi == 255) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][g] = (sat_pk_u8(pq[j][0]) | (sat_pk_u8(pq[j][1]) << 16)) ^ p.out_xor;
                    } else {
                        const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][g] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][1], lo1, hi1)),
                                                                (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][0], lo1, hi1)), 0x06040200u) ^ p.out_xor;
                    }
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        asm volatile("" : "+v"(pk[i][j][g]));
                } else {
                int r[NJ][4];
                // RES: every table of the group is requested at once (LDS answers in order); each phase then waits only
                // for its own, so one LDS latency is paid per group instead of three
                v4i xa, xb, xc, xd, xe, sa, sb, sc, sd, se;
                {
                    // ---- the convolution's own rescale
                    v4i ta = {0, 0, 0, 0}, tb = ta, tc = ta, td = ta, te = ta;
                    if (EPI != EPI_RAW && !RES) {
                        if (idx + 1 < NI * 4) {
                            const int nx = idx + 1;
                            request_tables(tq[nx & 1], tab + (unsigned)((nx / 4) * 32 + 8 * (nx % 4)) * 4u);
                            wait_lgkm<NTR>();
                        } else {
                            wait_lgkm<0>();
                        }
                        tie(tq[idx & 1][0]); tie(tq[idx & 1][1]); tie(tq[idx & 1][2]);
                        if (EPI == EPI_I24) tie(tq[idx & 1][3]);
                        if (EPI != EPI_F32) tie(tq[idx & 1][4]);
                        ta = tq[idx & 1][0]; tb = tq[idx & 1][1]; tc = tq[idx & 1][2];
                        if (EPI == EPI_I24) td = tq[idx & 1][3];
                        if (EPI != EPI_F32) te = tq[idx & 1][4];
                    }
                    if (EPI != EPI_RAW && RES) {
                        lds_read128_nowait<BN * 4>(ta, trow);
                        lds_read128_nowait<2 * BN * 4>(tb, trow);
                        lds_read128_nowait<3 * BN * 4>(tc, trow);
                        if (EPI == EPI_I24) lds_read128_nowait<4 * BN * 4>(td, trow);
                        if (EPI != EPI_F32) lds_read128_nowait<5 * BN * 4>(te, trow);
                        if (RES) {
                            if (q.has_pre) {
                                lds_read128_nowait<11 * BN * 4>(xa, trow);
                                lds_read128_nowait<12 * BN * 4>(xb, trow);
                                lds_read128_nowait<13 * BN * 4>(xc, trow);
                                lds_read128_nowait<14 * BN * 4>(xd, trow);
                                lds_read128_nowait<15 * BN * 4>(xe, trow);
                            }
                            lds_read128_nowait<6 * BN * 4>(sa, trow);
                            lds_read128_nowait<7 * BN * 4>(sb, trow);
                            lds_read128_nowait<8 * BN * 4>(sc, trow);
                            lds_read128_nowait<9 * BN * 4>(sd, trow);
                            lds_read128_nowait<10 * BN * 4>(se, trow);
                            if (q.has_pre) wait_lgkm<10>(); else wait_lgkm<5>();
                        } else {
                            wait_lgkm<0>();
                        }
                        tie(ta); tie(tb); tie(tc); tie(td); tie(te);
                    }
                    if (EPI == EPI_I24 && q.preclamp) {
                        // the pre-clamp keeps the product inside 32 bits; it is skipped when the host has shown that no
                        // accumulator of this layer can overflow it
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
#pragma unroll
                            for (int t = 0; t < 4; ++t)
                                acc[i][j][4 * g + t] = med3_i32(acc[i][j][4 * g + t], ta[t], tb[t]);
                    }
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            const int v = acc[i][j][4 * g + t];
                            if (EPI == EPI_I24) {
                                // (v * c + half) >> e, saturated; the bias is inside `half`
                                r[j][t] = med3_i32((__mul24(v, tc[t]) + td[t]) >> te[t], vlo, vhi);
                            } else if (EPI == EPI_F32) {
                                float f = (float)v;
                                if (q.preclamp) f = fminf(fmaxf(f, as_f32(ta[t])), as_f32(tb[t]));
                                f = round_half_away(f * as_f32(tc[t]));
                                r[j][t] = (int)med3_f32(f, flo, fhi);
                            } else {
                                r[j][t] = epi_apply<EPI>(v, ta[t], tb[t], tc[t], td[t], te[t], p.epi.lo, p.epi.hi, p.epi.relu);
                            }
                        }
                }
                if (RES) {
                    // ---- + the other input of the sum, through its folded ScalingCell if there is one, then the sum's
                    // own rescale (ref: src/Cell/ElemWiseCell_Frame.cpp:116-136 with unit coefficients)
                    int o[NJ][4];
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const unsigned w = resw[RES ? idx : 0][RES ? j : 0] ^ q.res_flip;
                        o[j][0] = (int)(w & 0xffu);
                        o[j][1] = (int)((w >> 8) & 0xffu);
                        o[j][2] = (int)((w >> 16) & 0xffu);
                        o[j][3] = (int)(w >> 24);
                    }
                    if (q.has_pre) {
                        wait_lgkm<5>();
                        tie(xa); tie(xb); tie(xc); tie(xd); tie(xe);
                        if (q.pre_clamp) {
#pragma unroll
                            for (int j = 0; j < NJ; ++j)
#pragma unroll
                                for (int t = 0; t < 4; ++t)
                                    o[j][t] = med3_i32(o[j][t], xa[t], xb[t]);
                        }
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
#pragma unroll
                            for (int t = 0; t < 4; ++t)
                                o[j][t] = med3_i32((__mul24(o[j][t], xc[t]) + xd[t]) >> xe[t], plo, phi);
                    }
                    wait_lgkm<0>();
                    tie(sa); tie(sb); tie(sc); tie(sd); tie(se);
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            r[j][t] += o[j][t];
                    if (q.sum_clamp) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
#pragma unroll
                            for (int t = 0; t < 4; ++t)
                                r[j][t] = med3_i32(r[j][t], sa[t], sb[t]);
                    }
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            r[j][t] = med3_i32((__mul24(r[j][t], sc[t]) + sd[t]) >> se[t], slo, shi);
                }
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    if (out_bytes) {
                        pk[i][j][g] = pack_bytes(r[j][0], r[j][1], r[j][2], r[j][3]) ^ p.out_xor;
                    } else {
                        const int m = m0 + wm * TM + j * 32 + l32;
                        const int ch = n0 + wn * TN + i * 32 + 8 * g + 4 * lh;
                        if (m < p.M && ch < p.out_cs)
                            *(int4*)((int*)p.out + (long long)m * p.out_cs + ch) = int4{r[j][0], r[j][1], r[j][2], r[j][3]};
                    }
                }
                }
            }
        }
        if (!out_bytes)
            return;
        // pk[i][j][g] holds channels 8g + 4*lh .. +3 of tile i.  Swapping g = 2,3 of the lower lane half with g = 0,1 of
        // the upper one leaves every lane with 16 consecutive channels (16*lh ..) of its pixel; a second exchange
        // between the two channel tiles makes that 32 (32*lh ..).
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int m = m0 + wm * TM + j * 32 + l32;
            const int mp = out_pix(m);
            signed char* orow = (signed char*)p.out + (long long)mp * p.out_cs + (n0 + wn * TN);
            unsigned qd[NI][4];
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const auto s02 = __builtin_amdgcn_permlane32_swap(pk[i][j][0], pk[i][j][2], false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(pk[i][j][1], pk[i][j][3], false, false);
                qd[i][0] = s02[0]; qd[i][1] = s02[1]; qd[i][2] = s13[0]; qd[i][3] = s13[1];
            }
            if (NI == 2) {
                v4i first, second;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const auto x = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[NI - 1][e], false, false);
                    first[e] = (int)x[0];
                    second[e] = (int)x[1];
                }
                const int ch = n0 + wn * TN + 32 * lh;
                if (RES) {
                    const unsigned off = m < p.M ? (unsigned)(mp * p.out_cs + ch) : 0x80000000u;
                    __builtin_amdgcn_raw_buffer_store_b128(first, out_rsrc, off, 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(second, out_rsrc, off + 16u, 0, 0);
                } else if (m < p.M) {
                    if (ch < p.out_cs) *(v4i*)(orow + 32 * lh) = first;
                    if (ch + 16 < p.out_cs) *(v4i*)(orow + 32 * lh + 16) = second;
                }
            } else {
                static_assert(NI <= 2, "one or two channel tiles per wave");
                const v4i only = {(int)qd[0][0], (int)qd[0][1], (int)qd[0][2], (int)qd[0][3]};
                const int ch = n0 + wn * TN + 16 * lh;
                if (m < p.M && ch < p.out_cs) *(v4i*)(orow + 16 * lh) = only;
            }
        }
    };

#ifdef N2D2HIP_PROFILE
    pr_t1 = clock64();
#endif
    // ---- per-block constants: bias and rescale tables of the channel tile.  Their loads are issued first and their
    // values stored to LDS behind the ring fill, so that the wait for them (loads return in order) does not include
    // the ring's own loads.
    static_assert(BN <= NT, "one table entry per thread");
    int tv[19];
    const bool tload = tid < BN;
    {
        const int i = tload ? tid : 0;
#pragma unroll
        for (int k = 0; k < 19; ++k) tv[k] = 0;
        if (tload) {
            if (!p16)
                tv[0] = BIAS_REG ? p.bias[n0 + i] : 0;
            if (EPI != EPI_RAW) {
                if (!p16)
                    tv[1] = p.epi.a[n0 + i];
                tv[2] = p.epi.b[n0 + i];
                tv[3] = p.epi.c[n0 + i];
                tv[4] = (EPI == EPI_I24) ? p.epi.d[n0 + i] : 0;
                tv[5] = (EPI != EPI_F32) ? p.epi.e[n0 + i] : 0;
            }
            if (RES) {
                tv[6] = q.sum.a[n0 + i];
                tv[7] = q.sum.b[n0 + i];
                tv[8] = q.sum.c[n0 + i];
                tv[9] = q.sum.d[n0 + i];
                tv[10] = q.sum.e[n0 + i];
                if (p16 && i < BN / 2) {
                    tv[16] = q.sum16[n0 / 2 + i];
                    tv[17] = q.sum16[q.sum16_stride + n0 / 2 + i];
                    tv[18] = q.sum16[2 * q.sum16_stride + n0 / 2 + i];
                }
                if (q.has_pre) {
                    tv[11] = q.pre.a[n0 + i];
                    tv[12] = q.pre.b[n0 + i];
                    tv[13] = q.pre.c[n0 + i];
                    tv[14] = q.pre.d[n0 + i];
                    tv[15] = q.pre.e[n0 + i];
                }
            }
        }
    }
    // ---- fill the ring: the first S steps occupy all S stages
    if (RES)
        issue_res(0);
#pragma unroll
    for (int s = 0; s < S; ++s)
        issue();
    if (tload) {
        int* tabw = (int*)(smem + TAB_OFF);
        const int i = tid;
        if (!p16)
            tabw[i] = tv[0];
        if (EPI != EPI_RAW) {
            if (!p16)
                tabw[BN + i] = tv[1];
            tabw[2 * BN + i] = tv[2];
            tabw[3 * BN + i] = tv[3];
            tabw[4 * BN + i] = tv[4];
            tabw[5 * BN + i] = tv[5];
        }
        if (RES) {
            tabw[6 * BN + i] = tv[6];
            tabw[7 * BN + i] = tv[7];
            tabw[8 * BN + i] = tv[8];
            tabw[9 * BN + i] = tv[9];
            tabw[10 * BN + i] = tv[10];
            if (p16 && i < BN / 2) {
                tabw[i] = tv[16];
                tabw[BN / 2 + i] = tv[17];
                tabw[BN + i] = tv[18];
            }
            if (q.has_pre) {
                tabw[11 * BN + i] = tv[11];
                tabw[12 * BN + i] = tv[12];
                tabw[13 * BN + i] = tv[13];
                tabw[14 * BN + i] = tv[14];
                tabw[15 * BN + i] = tv[15];
            }
        }
    }
    __syncthreads();

    // ---- the bias of this lane's channels (rows 8g + 4*lh + t of each 32-channel tile): C operand of a tile's first
    // MFMAs.  The integer rescale has it folded into its tables instead and starts from zero.
    v16i biasv[BIAS_REG ? NI : 1];
#pragma unroll
    for (int i = 0; i < (BIAS_REG ? NI : 0); ++i) {
        v4i b0, b1, b2, b3;
        const unsigned t = tab + (unsigned)i * 128u;
        lds_read128_nowait<0>(b0, t); lds_read128_nowait<32>(b1, t); lds_read128_nowait<64>(b2, t); lds_read128_nowait<96>(b3, t);
        wait_lgkm<0>();
        tie(b0); tie(b1); tie(b2); tie(b3);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            biasv[i][e] = b0[e]; biasv[i][4 + e] = b1[e]; biasv[i][8 + e] = b2[e]; biasv[i][12 + e] = b3[e];
        }
    }


    if (ntile > 0) {
        wait_loads_and_barrier<LPI*(S - 1)>();         // step 0 has landed
#ifdef N2D2HIP_PROFILE
        pr_t2 = clock64();
#endif
        read_k(std::integral_constant<int, 0>());
        for (int c_tile = 0; c_tile < ntile; ++c_tile) {
            for (int it = 0; it < niter; ++it) {
                // MFMA K step kk of this stage.  Its fragments were requested one K step ago; the next ones are
                // requested before its MFMAs are issued, so that they return while those run.
                auto kstep = [&](auto kkc) {
                    constexpr int kk = decltype(kkc)::value;
                    constexpr int set = kk & 1;
                    wait_lgkm<0>();
                    if (W4) {
#pragma unroll
                        for (int i = 0; i < NI; ++i) {
                            tie(fw4[set][W4 ? i : 0]);
                            const unsigned p0 = (unsigned)fw4[set][W4 ? i : 0][0], p1 = (unsigned)fw4[set][W4 ? i : 0][1];
                            fw[set][i][0] = (int)((p0 << 4) & 0xf0f0f0f0u);
                            fw[set][i][1] = (int)(p0 & 0xf0f0f0f0u);
                            fw[set][i][2] = (int)((p1 << 4) & 0xf0f0f0f0u);
                            fw[set][i][3] = (int)(p1 & 0xf0f0f0f0u);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < NI; ++i) tie(fw[set][i]);
                    }
#pragma unroll
                    for (int j = 0; j < NJ; ++j) tie(fp[set][j]);
                    if (kk == KH - 1) {
                        // Every wave has its last fragments of this stage, so the stage can be refilled; and the next
                        // stage has landed for every wave.
                        wait_loads_and_barrier<LPI*(S - 2)>();
                        issue();
                    }
                    read_k(std::integral_constant<int, (kk + 1) % KH>());      // of this stage, or of the next one
                    if (kk == 0 && it == 0) {
#pragma unroll
                        for (int i = 0; i < NI; ++i)
#pragma unroll
                            for (int j = 0; j < NJ; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[set][i], fp[set][j], BIAS_REG ? biasv[BIAS_REG ? i : 0] : v16i{}, 0, 0, 0);
                    } else {
#pragma unroll
                        for (int i = 0; i < NI; ++i)
#pragma unroll
                            for (int j = 0; j < NJ; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[set][i], fp[set][j], acc[i][j], 0, 0, 0);
                    }
                };
                kstep(std::integral_constant<int, 0>());
                kstep(std::integral_constant<int, 1>());
                if constexpr (KH > 2) {
                    kstep(std::integral_constant<int, 2 % KH>());
                    kstep(std::integral_constant<int, 3 % KH>());
                }
            }
#ifdef N2D2HIP_PROFILE
            const long long e0 = clock64();
            epilogue(c_tile);
            pr_epi += clock64() - e0;
#else
            epilogue(c_tile);
#endif
        }
    }
#ifdef N2D2HIP_PROFILE
    pr_t3 = clock64();
    if (tid == 0 && q.prof) {
        long long* o = q.prof + (long long)blockIdx.x * 16;
        o[0] = pr_t0; o[1] = pr_t1; o[2] = pr_t2; o[3] = pr_t3; o[4] = pr_epi; o[5] = pr_w0; o[6] = wall_clock64(); o[7] = ntile * niter;
    }
#endif
    // no load may still be writing into LDS when the block's LDS is handed to another block
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
}

// 4-bit weights (conv_pipe_w4.hip).  tile: 0 = 128 pixels x 64 channels, 1 = 128 x 128, 2 = 64 x 128; `a.c.w` is the image
// conv_pipe_w4_image() makes; hi16 selects the scaled-up tables.
size_t conv_pipe_w4_image_bytes(int rows, int ktot);
void conv_pipe_w4_image(const signed char* w, int rows, int ktot, signed char* image);
// With a.res set, the residual sum behind the convolution is computed in the epilogue.
int conv_pipe_w4_launch(ConvPipeArgs a, int tile, int valid, bool hi16, int grid, hipStream_t stream);

} // namespace n2d2hip
