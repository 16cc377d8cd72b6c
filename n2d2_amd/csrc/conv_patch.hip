// 3x3 convolution (stride 1, no dilation) on the int8 matrix cores for inputs that carry their padding as a border of
// zeros.
//
// In the flattened index space of such a tensor (image, padded row, padded column) a 3x3 window is nine shifts of one
// run of pixels: out[q] = sum over (ky, kx) of W[ky][kx] . in[q + (ky - 1) * Wp + (kx - 1)].  A block therefore computes
// BM consecutive positions q (border positions included: their results are dropped at the store) from ONE contiguous
// run of BM + 2 * Wp + 2 input pixels, the patch, which it copies to LDS once per 64 input channels and then reads
// nine times at shifted row addresses.  Against a loader that fetches every tap's pixels again, the pixel operand's
// traffic into LDS drops by the kernel size, the loader has no per-tap address arithmetic, and one barrier serves
// 144 matrix instructions per wave.
//
//  * pixels (MFMA B operand): global -> LDS by direct loads (global_load_lds_dwordx4), two patch buffers; the patch of
//    step s + 1 (next 64 channels, or next tile) is requested when step s starts.  Rows are 64 bytes, 16-byte slots
//    XOR-swizzled on the global-address side so that ds_read_b128 of a fragment is conflict-free for any row shift.
//  * weights (MFMA A operand): never pass LDS.  The host stores them in fragment order, so a wave reads one fragment
//    as 64 x 16 consecutive bytes straight into registers; a tap's register set (there are three) is refilled with the
//    weights three taps ahead as soon as its matrix instructions are issued.
//  * a wave owns 128 pixels x 64 channels (4 x 2 tiles of 32 x 32): one weight fragment serves four matrix
//    instructions, one pixel fragment two; fragments of the next K step are requested before the current one's
//    instructions are issued.
//  * the epilogue is the pipelined kernel's: rescale (tables in LDS, bias folded in), saturate, pack, exchange between
//    the lane halves until a lane owns 32 consecutive channels of its pixel, two 16-byte stores; positions on the
//    border, and past the end, are not stored.
//
// Waits are written by hand.  s_waitcnt vmcnt(n) returns when at most n memory operations are outstanding; loads
// return in order, so with n = the number of loads issued after the one needed, that one has landed.  Stores count
// too but only make the wait stricter: n never includes them.
#include <algorithm>
#include <cstdlib>

#include "conv_patch.hpp"
#include "epilogue.hpp"
#include "mfma_util.hpp"

namespace n2d2hip {

template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// WGM x WGN waves (pixels x channels); NPL: 1 KB patch chunks each wave loads per step (the patch buffer holds
// NPL * WGM * WGN * 16 rows); P16: tables scaled up so that the rescaled value is the upper half of the multiply-add.
template <int WGM, int WGN, int NPL, bool P16, int NJ>
__global__ __launch_bounds__(WGM * WGN * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_patch3x3_kernel(ConvPatchArgs q)
{
    constexpr int NW = WGM * WGN;
    constexpr int NI = 2;                              // NJ 32-pixel and NI 32-channel tiles per wave
    static_assert(NJ == 2 || NJ == 4, "tiles of 128 or 256 positions");
    constexpr int BM = 32 * NJ * WGM, BN = 32 * NI * WGN;
    constexpr int PBUF = NPL * NW * 1024;              // bytes of one patch buffer
    constexpr int TAB_OFF = 2 * PBUF;
    constexpr int NTAB = P16 ? 2 : 5;
    constexpr int NWL = NI * 2;                        // weight fragments (loads) per tap and wave
    static_assert(NPL + 2 * NWL < 60, "vmcnt is a 6-bit counter");
    static_assert((NJ - 1) * 2048 < 65536, "ds_read immediate offsets are 16 bits");

    __shared__ __attribute__((aligned(1024))) unsigned char smem[TAB_OFF + NTAB * BN * 4];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int l32 = lane & 31, lh = lane >> 5;

    // ---- tiles of this block: one channel tile, every mlanes-th pixel tile of its XCD's run (blocks 8 apart share an
    // XCD, and with it the rows neighbouring tiles have in common)
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % q.ntiles_n;
    const int mlane = xcd * q.xcd_tiles + slot / q.ntiles_n;
    const int mend = min((xcd + 1) * q.xcd_tiles, q.mtiles);
    const int ntile = (mlane < mend) ? (mend - mlane + q.mlanes - 1) / q.mlanes : 0;
    if (ntile == 0)
        return;
#ifdef N2D2HIP_PROFILE
    long long pr_t0 = clock64(), pr_t1 = 0, pr_t2 = 0, pr_epi = 0, pr_w0 = wall_clock64();
#endif
    const int n0 = tile_n * BN;
    const int nchunk = q.nchunk;
    const int nsteps = ntile * nchunk;

    // ---- patch loader.  Lane l of a wave fills 16-byte slot l of a 1 KB chunk: row l / 4 of the chunk's 16 rows,
    // physical slot l % 4, which holds the logical slot the swizzle maps there.
    const int lrow = lane >> 2;
    const int lq = (lane & 3) ^ ((lane >> 4) & 3);
    const int last_pos = q.total - 1;
    auto issue_patch = [&](int tile, int chunk, int buf) {
        const int qs = tile * BM - (q.Wp + 1);
        unsigned char* dst = smem + buf * PBUF;
        const signed char* src0 = q.in + chunk * 64 + lq * 16;
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const int g = wave + NW * i;
            const int pos = min(max(qs + 16 * g + lrow, 0), last_pos);        // rows before the tensor or past its end: any valid pixel
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src0 + (unsigned)(pos * q.C)), (lds_ptr_t)(dst + g * 1024), 16, 0, 0);
        }
    };

    // ---- weight stream of this wave's two channel tiles: fragments in (chunk, tap, K step) order, 1 KB each
    const unsigned wspan = (unsigned)nchunk * 9u * 2048u;
    const signed char* wlane = q.wfrag + (size_t)(n0 / 32 + wn * NI) * wspan + lane * 16;
    unsigned woff = 0;
    v4i wf[3][NI][2];
    auto issue_w = [&](auto bufc) {
        constexpr int buf = decltype(bufc)::value;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const signed char* p = wlane + (size_t)i * wspan + woff;
            asm volatile("global_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %1, %2, off offset:1024"
                         : "=&v"(wf[buf][i][0]), "=&v"(wf[buf][i][1]) : "v"(p) : "memory");
        }
        woff += 2048u;
        if (woff == wspan) woff = 0;
    };

    // ---- pixel fragments: row of the patch = position in the tile + ky * Wp + kx
    const int r0 = wm * (32 * NJ) + l32;
    v4i fp[2][NJ];
    auto px_addr = [&](unsigned pb, int tapoff) -> unsigned {
        const int r = r0 + tapoff;
        return pb + (unsigned)((r << 6) + ((((r >> 2) ^ lh) & 3) << 4));
    };
    auto read_px = [&](auto setc, unsigned addr) {
        constexpr int set = decltype(setc)::value;
        lds_read128_nowait<0>(fp[set][0], addr);
        lds_read128_nowait<2048>(fp[set][1], addr);
        if constexpr (NJ == 4) {
            lds_read128_nowait<4096>(fp[set][2], addr);
            lds_read128_nowait<6144>(fp[set][3], addr);
        }
    };

    v16i acc[NI][NJ];
    const unsigned tab = lds0 + TAB_OFF + (unsigned)(wn * (32 * NI) + 4 * lh) * 4u;
    const int vlo = q.lo, vhi = q.hi;

    // ---- rescale, pack and store a finished tile
    auto epilogue = [&](int tile) {
        const int q0 = tile * BM;
        unsigned pk[NI][NJ][4];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const unsigned trow = tab + (unsigned)(i * 32 + 8 * g) * 4u;
                if constexpr (P16) {
                    v4i tc, td;
                    lds_read128_nowait<0>(tc, trow);
                    lds_read128_nowait<BN * 4>(td, trow);
                    wait_lgkm<0>();
                    tie(tc); tie(td);
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
                            pk[i][j][g] = (sat_pk_u8(pq[j][0]) | (sat_pk_u8(pq[j][1]) << 16)) ^ q.out_xor;
                    } else {
                        const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            pk[i][j][g] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][1], lo1, hi1)),
                                                                (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[j][0], lo1, hi1)), 0x06040200u) ^ q.out_xor;
                    }
                } else {
                    v4i ta, tb, tc, td, te;
                    lds_read128_nowait<0>(ta, trow);
                    lds_read128_nowait<BN * 4>(tb, trow);
                    lds_read128_nowait<2 * BN * 4>(tc, trow);
                    lds_read128_nowait<3 * BN * 4>(td, trow);
                    lds_read128_nowait<4 * BN * 4>(te, trow);
                    wait_lgkm<0>();
                    tie(ta); tie(tb); tie(tc); tie(td); tie(te);
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        int r[4];
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            int v = acc[i][j][4 * g + t];
                            if (q.preclamp) v = med3_i32(v, ta[t], tb[t]);
                            r[t] = med3_i32((__mul24(v, tc[t]) + td[t]) >> te[t], vlo, vhi);
                        }
                        pk[i][j][g] = pack_bytes(r[0], r[1], r[2], r[3]) ^ q.out_xor;
                    }
                }
                // keeps the groups apart: without it every group's tables would be live at once
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    asm volatile("" : "+v"(pk[i][j][g]));
            }
        }
        // pk[i][j][g] holds channels 8g + 4 * lh .. + 3 of tile i.  Two exchanges between the lane halves leave every lane
        // with 32 consecutive channels (32 * lh ..) of its pixel.
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int pos = q0 + wm * (32 * NJ) + j * 32 + l32;
            const int pc = min(pos, last_pos);
            const int b = div_magic(pc, q.img_mul, q.img_sh);
            const int rem = pc - b * (q.Hp * q.Wp);
            const int yp = div_magic(rem, q.row_mul, q.row_sh);
            const int xp = rem - yp * q.Wp;
            const bool inside = pos <= last_pos && yp >= 1 && yp <= q.Hp - 2 && xp >= 1 && xp <= q.Wp - 2;
            const int opix = (b * q.OHp + yp - 1 + q.out_halo) * q.OWp + xp - 1 + q.out_halo;
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
            if (inside) {
                signed char* orow = (signed char*)q.out + (size_t)opix * q.out_cs + (n0 + wn * (32 * NI) + 32 * lh);
                *(v4i*)orow = first;
                *(v4i*)(orow + 16) = second;
            }
        }
    };

    // ---- fill: the first patch, the weights of the first three taps
#ifdef N2D2HIP_PROFILE
    pr_t1 = clock64();
#endif
    issue_patch(mlane, 0, 0);
    issue_w(std::integral_constant<int, 0>());
    issue_w(std::integral_constant<int, 1>());
    issue_w(std::integral_constant<int, 2>());

    // ---- rescale tables of the channel tile
    if (tid < BN) {
        int* tabw = (int*)(smem + TAB_OFF);
        if (P16) {
            tabw[tid] = q.tc[n0 + tid];
            tabw[BN + tid] = q.td[n0 + tid];
        } else {
            tabw[tid] = q.ta[n0 + tid];
            tabw[BN + tid] = q.tb[n0 + tid];
            tabw[2 * BN + tid] = q.tc[n0 + tid];
            tabw[3 * BN + tid] = q.td[n0 + tid];
            tabw[4 * BN + tid] = q.te[n0 + tid];
        }
    }


    int c_tile = 0, c_chunk = 0;                       // the step being computed
    for (int s = 0; s < nsteps; ++s) {
        // This wave's loads of the step's patch have landed (only three taps' weight requests are younger); behind the
        // barrier everybody's have, and nobody still reads the other buffer.
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" : : "n"(3 * NWL) : "memory");
#ifdef N2D2HIP_PROFILE
        if (s == 0) pr_t2 = clock64();
#endif
        int n_tile = c_tile, n_chunk = c_chunk + 1;
        if (n_chunk == nchunk) { n_chunk = 0; ++n_tile; }
        issue_patch(mlane + n_tile * q.mlanes, n_chunk, (s + 1) & 1);          // past the block's last step: a harmless re-read
        const unsigned pb = lds0 + (unsigned)((s & 1) * PBUF);
        const bool first_chunk = c_chunk == 0;
        read_px(std::integral_constant<int, 0>(), px_addr(pb, 0));

        auto tap = [&](auto tc_) {
            constexpr int T = decltype(tc_)::value;
            constexpr int wb = T % 3;
            // younger than this tap's weights: those of the next two taps and, for the step's first three taps, the patch.
            // (The patch is requested behind the weights of taps 0..2, so that those do not queue up behind it: loads
            // return in order.)
            if (T < 3) wait_vm<NPL + 2 * NWL>(); else wait_vm<2 * NWL>();
#pragma unroll
            for (int i = 0; i < NI; ++i) { tie(wf[wb][i][0]); tie(wf[wb][i][1]); }
            const unsigned a0 = px_addr(pb, (T / 3) * q.Wp + (T % 3));
            // address of the next tap's first K step (unused after the last tap)
            const unsigned an = px_addr(pb, ((T + 1) / 3) * q.Wp + ((T + 1) % 3));
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                wait_lgkm<0>();
                if (kk == 0) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) tie(fp[0][j]);
                    read_px(std::integral_constant<int, 1>(), a0 ^ 32u);
                } else {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) tie(fp[1][j]);
                    if (T < 8) read_px(std::integral_constant<int, 0>(), an);
                }
                if (T == 0 && kk == 0) {
                    if (first_chunk) {
#pragma unroll
                        for (int i = 0; i < NI; ++i)
#pragma unroll
                            for (int j = 0; j < NJ; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[wb][i][kk], fp[kk][j], v16i{}, 0, 0, 0);
                    } else {
#pragma unroll
                        for (int i = 0; i < NI; ++i)
#pragma unroll
                            for (int j = 0; j < NJ; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[wb][i][kk], fp[kk][j], acc[i][j], 0, 0, 0);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NI; ++i)
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[wb][i][kk], fp[kk][j], acc[i][j], 0, 0, 0);
                }
            }
            // this tap's register set takes the weights three taps ahead (the next step's first taps at the end of this one)
            issue_w(std::integral_constant<int, wb>());
        };
        tap(std::integral_constant<int, 0>());
        tap(std::integral_constant<int, 1>());
        tap(std::integral_constant<int, 2>());
        tap(std::integral_constant<int, 3>());
        tap(std::integral_constant<int, 4>());
        tap(std::integral_constant<int, 5>());
        tap(std::integral_constant<int, 6>());
        tap(std::integral_constant<int, 7>());
        tap(std::integral_constant<int, 8>());

#ifdef N2D2HIP_PROFILE
        if (c_chunk == nchunk - 1) {
            const long long e0 = clock64();
            epilogue(mlane + c_tile * q.mlanes);
            pr_epi += clock64() - e0;
        }
#else
        if (c_chunk == nchunk - 1)
            epilogue(mlane + c_tile * q.mlanes);
#endif
        c_tile = n_tile;
        c_chunk = n_chunk;
    }
#ifdef N2D2HIP_PROFILE
    if (tid == 0 && q.prof) {
        long long* o = q.prof + (long long)blockIdx.x * 16;
        o[0] = pr_t0; o[1] = pr_t1; o[2] = pr_t2; o[3] = clock64(); o[4] = pr_epi; o[5] = pr_w0; o[6] = wall_clock64(); o[7] = nsteps;
    }
#endif
    // no load may still be writing into LDS when the block's LDS is handed to another block
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
}

size_t conv_patch_weight_bytes(int C, int O) { return (size_t)O * 9 * C; }

void conv_patch_weight_layout(const signed char* w, int C, int O, signed char* frag)
{
    const int nchunk = C / 64;
    for (int ct = 0; ct < O / 32; ++ct)
        for (int c = 0; c < nchunk; ++c)
            for (int tap = 0; tap < 9; ++tap)
                for (int kk = 0; kk < 2; ++kk)
                    for (int lane = 0; lane < 64; ++lane) {
                        const int o = ct * 32 + (lane & 31), ch = c * 64 + kk * 32 + (lane >> 5) * 16;
                        const signed char* src = w + ((size_t)o * 9 + tap) * C + ch;
                        signed char* dst = frag + (((((size_t)ct * nchunk + c) * 9 + tap) * 2 + kk) * 64 + lane) * 16;
                        memcpy(dst, src, 16);
                    }
}

bool conv_patch_eligible(int C, int O, int Wp)
{
    // the patch of a 256-position tile, BM + 2 * Wp + 2 rows, must fit the largest buffer built below (384 rows)
    return C > 0 && C % 64 == 0 && O > 0 && O % 64 == 0 && Wp >= 3 && 256 + 2 * Wp + 2 <= 384;
}

template <int WGM, int WGN, int NPL, int NJ>
static void launch(const ConvPatchArgs& a, bool hi16, int grid, hipStream_t stream)
{
    if (hi16)
        N2D2HIP_LAUNCH_T(conv_patch3x3_kernel, (WGM, WGN, NPL, true, NJ), dim3(grid), dim3(WGM * WGN * 64), 0, stream, a);
    else
        N2D2HIP_LAUNCH_T(conv_patch3x3_kernel, (WGM, WGN, NPL, false, NJ), dim3(grid), dim3(WGM * WGN * 64), 0, stream, a);
}

int conv_patch_launch(ConvPatchArgs a, bool hi16, int num_cus, int tile_m, hipStream_t stream)
{
    N2D2HIP_REQUIRE(conv_patch_eligible(a.C, a.O, a.Wp), N2D2HIP_ERR_INVALID, "conv_patch: shape not served");
    N2D2HIP_REQUIRE((long long)a.total * a.C < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED, "conv_patch: tensor too large");
    N2D2HIP_REQUIRE(tile_m == 0 || tile_m == 64 || tile_m == 128 || tile_m == 256, N2D2HIP_ERR_INVALID, "conv_patch: tile choice %d", tile_m);
    const bool wide = a.O % 128 == 0;                 // 128 channels per block (2 x 2 waves); else 64 channels
    const int BN = wide ? 128 : 64;
    a.nchunk = a.C / 64;
    a.ntiles_n = a.O / BN;
    // The forms of the kernel.  Tiles of 256 positions, a wave on 128 of them, re-read less of their neighbours' rows and
    // stream the weights half as often (20.2 against 21.4 us for 256 -> 256 channels on 14x14 at batch 128, one block per
    // CU either way).  Tiles of 128 positions, a wave on 64, where the larger ones would leave CUs without a block (12.4
    // against 16.8 us for the same layer at batch 64).  With 64 input channels a tile is one channel step and the waves of
    // 64 positions win (64 -> 64 channels on 56x56: 15.0 against 18.9 us at batch 64); four of them on a tile of 256 share
    // more of the patch than two on a tile of 128 (23.0 against 26.6 us at batch 128).
    enum Form { M256, M128, M256_WAVES4 };
    const bool few = (a.total + 255) / 256 * a.ntiles_n < num_cus;
    Form form = few ? M128 : (a.C < 128 ? (wide ? M128 : M256_WAVES4) : M256);
    if (tile_m == 256) form = M256;
    if (tile_m == 128) form = M128;
    if (tile_m == 64) form = wide ? M128 : M256_WAVES4;
    const int BM = form == M128 ? 128 : 256;
    const int NW = (wide || form == M256_WAVES4) ? 4 : 2;
    const int chunks = (BM + 2 * a.Wp + 2 + 15) / 16;
    const int npl = (chunks + NW - 1) / NW;
    // blocks per CU: two of four waves, three of two (LDS: at most 49 KB + tables per block)
    const int slots = (NW == 4 ? 2 : 3) * num_cus;
    a.mtiles = (a.total + BM - 1) / BM;
    const int per_xcd = std::max(1, std::min((a.mtiles + 7) / 8, slots / (8 * a.ntiles_n)));
    a.mlanes = per_xcd;
    a.xcd_tiles = (a.mtiles + 7) / 8;
    const int grid = 8 * a.ntiles_n * per_xcd;
#ifdef N2D2HIP_PROFILE
    a.prof = nullptr;      // probe builds: launch_kernel() points it at this launch's records
#endif
    // patch rows: at most 384 (tiles of 256) or 256 (tiles of 128) wherever the kernel is eligible
    if (form == M256_WAVES4) {
        launch<4, 1, 6, 2>(a, hi16, grid, stream);
    } else if (form == M256) {
        if (wide) {
            if (npl <= 5) launch<2, 2, 5, 4>(a, hi16, grid, stream);
            else launch<2, 2, 6, 4>(a, hi16, grid, stream);
        } else {
            if (npl <= 10) launch<2, 1, 10, 4>(a, hi16, grid, stream);
            else launch<2, 1, 12, 4>(a, hi16, grid, stream);
        }
    } else {
        if (wide) {
            if (npl <= 3) launch<2, 2, 3, 2>(a, hi16, grid, stream);
            else launch<2, 2, 4, 2>(a, hi16, grid, stream);
        } else {
            if (npl <= 6) launch<2, 1, 6, 2>(a, hi16, grid, stream);
            else launch<2, 1, 8, 2>(a, hi16, grid, stream);
        }
    }
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // namespace n2d2hip
