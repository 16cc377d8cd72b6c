// First-layer convolution: at most 4 input channels stored as one dword per
// pixel, horizontal stride 2, no dilation (the 7x7 / 3x3 stride-2 stems).
//
// Such a layer has almost no arithmetic per byte it writes (K = 7*7*3 against
// 64 output channels), so the kernel is built around moving data once:
//  * a tile is 128 consecutive output pixels of one output row; the KH input
//    rows it needs (2*128 + 6 pixels each) are copied global -> LDS by 4-byte
//    direct loads, one pixel per lane, so that padding is decided per pixel
//    (a lane outside the image fetches the input's zero instead) and every
//    window of the tile is then read from LDS;
//  * one MFMA K step is one kernel row: 8 taps x 4 channel slots = 32; the tap
//    past the kernel's width and the channel slots past C meet zero weights.
//    A lane's 16-byte pixel operand is 4 consecutive pixels of the row, at
//    8 bytes * pixel + 16 bytes * lane half: two ds_read_b64;
//  * the weights (64 channels x KH x 32 bytes) stay in registers for the
//    block's whole life;
//  * three LDS stages: the rows of the next two tiles are in flight while this
//    one is multiplied and rescaled; one barrier per tile.  Two tiles ahead,
//    not one, because the wait is a count of outstanding operations and the
//    epilogue's stores count too: with NLOAD younger loads allowed, the wait
//    is over when this tile's rows have landed (loads return in order) without
//    having to see the previous tile's stores acknowledged;
//  * the epilogue is the pipelined kernel's: rescale, pack to bytes, exchange
//    between lane halves until a lane owns 32 consecutive channels, store.
//    H16 (integer rescale, byte output, tables scaled up by the host so that
//    the result is the upper half of the multiply-add): a lane's 32 channels
//    never change, so their multipliers and addends live in registers and the
//    epilogue reads no table at all.
#pragma once

namespace n2d2hip {

struct ConvStemArgs {
    ConvArgs c;
    const signed char* wk;       // [channel][KH * 32]: kernel row, tap (8 slots), channel (4 slots)
    const signed char* fill16;   // the input's logical zero
    int ntiles;                  // pixel tiles: B * OH * tiles_per_row
    int tiles_per_row;
    int nlanes;                  // blocks of one XCD that share its run of pixel tiles
    int xcd_tiles;               // consecutive pixel tiles given to one XCD
    unsigned oh_mul, oh_sh;      // division by OH
    unsigned tpr_mul, tpr_sh;    // division by tiles_per_row
    int preclamp;
    // POOL kernels: the 3x3 stride-2 max pooling that follows the convolution is computed in the same launch.  A block
    // takes strips of pool_rows pooled rows of one image: the 2 * pool_rows + 1 convolution rows a strip needs go to a ring
    // of four rows in LDS as bytes, and each pooled row is written as soon as its third convolution row is there.  `ntiles`
    // then counts strips, `out` is the pooled tensor and the convolution's own output is never stored.
    int pool_rows, pool_pad, strips_per_image;
    int POH, POW;                // pooled rows / columns
    int pool_halo, POHp, POWp;   // border of the pooled tensor and its rows / columns with it
};

// NBLK: 32-channel blocks of outputs a work-group computes: 2, or 1 for a layer of at most 32 output channels (half the
// matrix instructions and half the rescale).
template <int KH, int EPI, bool H16 = false, bool POOL = false, int NBLK = 2>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 3))) void conv_stem_kernel(ConvStemArgs q)
{
    static_assert(NBLK == 2 || (NBLK == 1 && !POOL), "the pooled variant works on 64 channels");
    static_assert(!H16 || EPI == EPI_I24, "scaled-up tables belong to the integer rescale");
    static_assert(!POOL || H16, "the pooled variant is written for byte outputs of the integer rescale");
    const ConvArgs& p = q.c;
    constexpr int TW = 128;                    // output pixels per tile
    constexpr int PITCH = 1280;                // bytes per patch row in LDS: 5 loads of 64 pixels
    constexpr int NCHUNK = KH * 5;             // 256-byte chunks per stage
    constexpr int NLOAD = (NCHUNK + 3) / 4;    // per wave (chunks past the end land in the spare row)
    constexpr int STAGE = (KH + 1) * PITCH;
    constexpr int BN = 32 * NBLK;
    constexpr int TAB_OFF = 3 * STAGE;
    constexpr bool BIAS_ADD = EPI != EPI_I24;  // the integer rescale carries the bias in its tables
    constexpr int ROWS_OFF = TAB_OFF + 6 * BN * 4;             // POOL: four convolution rows of TW pixels x 64 bytes
    __shared__ __attribute__((aligned(16))) unsigned char smem[ROWS_OFF + (POOL ? 4 * TW * BN : 0)];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;      // blocks 8 apart run on the same XCD
    const int tile_n = slot % p.ntiles_n;
    const int n0 = tile_n * BN;
    // An XCD gets a run of consecutive tiles (consecutive output rows share most of their input rows through that XCD's
    // L2) and its blocks take them in turn.
    const int first = xcd * q.xcd_tiles + slot / p.ntiles_n;
    const int last = min((xcd + 1) * q.xcd_tiles, q.ntiles);
    // POOL: the units dealt to blocks are strips; a block's tiles are the convolution rows of its strips, one after the other
    const int nunit = (first < last) ? (last - first + q.nlanes - 1) / q.nlanes : 0;
    const int rows_per_strip = 2 * q.pool_rows + 1;
    const int ntile = POOL ? nunit * rows_per_strip : nunit;
    // Position of a walk over the block's tiles: strip k of the block, row j of the strip, the strip's image and the
    // convolution row of j = 0.  The loader walks two tiles ahead of the consumer; a division only where a strip begins.
    struct StripWalk { int k, j, b, oy0; };
    auto set_strip = [&](StripWalk& w) {
        const int sid = first + (w.k < nunit ? w.k : 0) * q.nlanes;
        w.b = sid / q.strips_per_image;
        w.oy0 = 2 * (sid - w.b * q.strips_per_image) * q.pool_rows - q.pool_pad;
    };
    auto walk_next = [&](StripWalk& w) {
        if (++w.j == rows_per_strip) { w.j = 0; ++w.k; set_strip(w); }
    };
    auto row_live = [&](const StripWalk& w) -> bool {
        const int oy = w.oy0 + w.j;
        return w.k < nunit && oy >= 0 && oy < p.OH;
    };
    StripWalk lw = {0, 0, 0, 0}, cw = {0, 0, 0, 0};
    if (POOL) { set_strip(lw); cw = lw; }

    // ---- loader: chunk c = wave + 4*j is 64 pixels (part c%5) of patch row c/5.  Which row and part a wave's j-th
    // load fetches never changes, so that is worked out once; the scalar unit is shared by every wave of the CU and
    // the per-tile part of this arithmetic is what the kernel spends most of its issue slots on.
    int ld_row[NLOAD], ld_x[NLOAD], ld_lds[NLOAD];
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) {
        const int c = wave + 4 * j;
        const int r = c / 5, part = c - r * 5;
        ld_row[j] = c < NCHUNK ? r : -(1 << 20);        // a chunk past the end reads a row that is never inside
        ld_x[j] = part * 64;
        ld_lds[j] = r * PITCH + part * 256;
    }
    const unsigned row_bytes = (unsigned)p.W * 4u;
    auto issue = [&](int t, int stage) {
        const int id = first + t * q.nlanes;
        bool live = t < ntile;
        int b, oy, txi = 0;
        if (POOL) {
            live = row_live(lw);
            b = live ? lw.b : 0;
            oy = live ? lw.oy0 + lw.j : 0;
            walk_next(lw);
        } else {
            const int rowid = div_magic(live ? id : 0, q.tpr_mul, q.tpr_sh);          // b * OH + oy
            txi = (live ? id : 0) - rowid * q.tiles_per_row;
            b = div_magic(rowid, q.oh_mul, q.oh_sh);
            oy = rowid - b * p.OH;
        }
        const int x0 = txi * TW * p.strideX - p.padL + lane;
        const int y0 = live ? oy * p.strideY - p.padT : -(1 << 21);
        unsigned char* sbase = smem + stage * STAGE;
        const signed char* img = p.in + (long long)b * p.H * row_bytes;
#pragma unroll
        for (int j = 0; j < NLOAD; ++j) {
            const int iy = y0 + ld_row[j];
            // everything about the row is block-uniform; a row outside the image sends every lane to the zero
            const bool row_ok = (unsigned)iy < (unsigned)p.H;
            const signed char* rowp = img + (row_ok ? (unsigned)iy : 0u) * row_bytes;
            const int ix = x0 + ld_x[j];
            const signed char* src = (row_ok & ((unsigned)ix < (unsigned)p.W)) ? rowp + (unsigned)ix * 4u : q.fill16;
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)(sbase + ld_lds[j]), 4, 0, 0);
        }
    };
    issue(0, 0);
    issue(1, 1);

    // ---- weights of this lane's channels: A operand of kernel row ky is 16 bytes at ky*32 + 16*lh
    v4i wf[NBLK][KH];
#pragma unroll
    for (int i = 0; i < NBLK; ++i)
#pragma unroll
        for (int ky = 0; ky < KH; ++ky)
            wf[i][ky] = *(const v4i*)(q.wk + (long long)(n0 + i * 32 + l32) * (KH * 32) + ky * 32 + 16 * lh);

    // ---- rescale tables of the channel tile
    {
        int* tabw = (int*)(smem + TAB_OFF);
        for (int i = tid; i < BN; i += 256) {
            tabw[i] = BIAS_ADD ? p.bias[n0 + i] : 0;
            if (EPI != EPI_RAW) {
                tabw[BN + i] = p.epi.a[n0 + i];
                tabw[2 * BN + i] = p.epi.b[n0 + i];
                tabw[3 * BN + i] = p.epi.c[n0 + i];
                tabw[4 * BN + i] = (EPI == EPI_I24) ? p.epi.d[n0 + i] : 0;
                tabw[5 * BN + i] = (EPI != EPI_F32) ? p.epi.e[n0 + i] : 0;
            }
        }
    }
    __syncthreads();
    v4i rc[H16 ? NBLK : 1][H16 ? 4 : 1], rd[H16 ? NBLK : 1][H16 ? 4 : 1];
    if (H16) {
#pragma unroll
        for (int i = 0; i < NBLK; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                rc[H16 ? i : 0][H16 ? g : 0] = *(const v4i*)(p.epi.c + n0 + i * 32 + 8 * g + 4 * lh);
                rd[H16 ? i : 0][H16 ? g : 0] = *(const v4i*)(p.epi.d + n0 + i * 32 + 8 * g + 4 * lh);
            }
    }
    const unsigned tab = lds0 + TAB_OFF + (unsigned)(4 * lh) * 4u;
    const bool out_bytes = p.out_dtype != N2D2HIP_I32;
    const int vlo = p.epi.lo, vhi = p.epi.hi;
    const float flo = (float)p.epi.lo, fhi = (float)p.epi.hi;
    // this lane's window origin inside a patch row: pixel 2 * (32*wave + l32), tap slot 4*lh
    const unsigned frag = lds0 + (unsigned)((p.strideX * (32 * wave + l32) + 4 * lh) * 4);

    for (int t = 0; t < ntile; ++t) {
        const int stage = t % 3;
        // this tile's rows have landed for every wave, and every wave is done with the stage of the previous tile
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(NLOAD) : "memory");
        issue(t + 2, (t + 2) % 3);

        v16i acc[NBLK];
        {
            typedef int v2i __attribute__((ext_vector_type(2)));
            v2i lo[KH], hi[KH];
            const unsigned fa = frag + (unsigned)(stage * STAGE);
#pragma unroll
            for (int ky = 0; ky < KH; ++ky)
                asm volatile("ds_read_b64 %0, %2 offset:%3\n\tds_read_b64 %1, %2 offset:%4"
                             : "=&v"(lo[ky]), "=&v"(hi[ky]) : "v"(fa), "n"(ky * PITCH), "n"(ky * PITCH + 8) : "memory");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int ky = 0; ky < KH; ++ky) {
                asm volatile("" : "+v"(lo[ky]), "+v"(hi[ky]));
                const v4i pf = {lo[ky][0], lo[ky][1], hi[ky][0], hi[ky][1]};
#pragma unroll
                for (int i = 0; i < NBLK; ++i)
                    acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i][ky], pf, ky == 0 ? v16i{} : acc[i], 0, 0, 0);
            }
        }

        // ---- epilogue: this lane holds channels 8g + 4*lh .. +3 of both 32-channel tiles for output pixel ox
        const int id = first + t * q.nlanes;
        const int rowid = POOL ? 0 : div_magic(id, q.tpr_mul, q.tpr_sh);
        const int ox = POOL ? 32 * wave + l32 : (id - rowid * q.tiles_per_row) * TW + 32 * wave + l32;
        const long long m = (long long)rowid * p.OW + ox;
        const bool pix_ok = ox < p.OW;
        unsigned pk[NBLK][4];
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if constexpr (H16) {
                    const v4i tc = rc[H16 ? i : 0][H16 ? g : 0], td = rd[H16 ? i : 0][H16 ? g : 0];
                    v2s pq[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int t0 = __mul24(acc[i][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                        const int t1 = __mul24(acc[i][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                        pq[h] = as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u));
                    }
                    if (vlo == 0 && vhi == 255) {
                        pk[i][g] = (sat_pk_u8(pq[0]) | (sat_pk_u8(pq[1]) << 16)) ^ p.out_xor;
                    } else {
                        const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
                        pk[i][g] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[1], lo1, hi1)),
                                                         (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[0], lo1, hi1)), 0x06040200u) ^ p.out_xor;
                    }
                    continue;
                }
                const unsigned trow = tab + (unsigned)(i * 32 + 8 * g) * 4u;
                v4i tbias = {0, 0, 0, 0}, ta = tbias, tb = tbias, tc = tbias, td = tbias, te = tbias;
                if (BIAS_ADD) lds_read128_nowait<0>(tbias, trow);
                if (EPI != EPI_RAW) {
                    lds_read128_nowait<BN * 4>(ta, trow);
                    lds_read128_nowait<2 * BN * 4>(tb, trow);
                    lds_read128_nowait<3 * BN * 4>(tc, trow);
                    if (EPI == EPI_I24) lds_read128_nowait<4 * BN * 4>(td, trow);
                    if (EPI != EPI_F32) lds_read128_nowait<5 * BN * 4>(te, trow);
                }
                wait_lgkm<0>();
                tie(tbias); tie(ta); tie(tb); tie(tc); tie(td); tie(te);
                int r[4];
                if (EPI == EPI_I24 && q.preclamp) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i][4 * g + e] = med3_i32(acc[i][4 * g + e], ta[e], tb[e]);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    int v = acc[i][4 * g + e];
                    if (BIAS_ADD) v += tbias[e];
                    if (EPI == EPI_I24) {
                        r[e] = med3_i32((__mul24(v, tc[e]) + td[e]) >> te[e], vlo, vhi);
                    } else if (EPI == EPI_F32) {
                        float f = (float)v;
                        if (q.preclamp) f = fminf(fmaxf(f, as_f32(ta[e])), as_f32(tb[e]));
                        f = round_half_away(f * as_f32(tc[e]));
                        r[e] = (int)med3_f32(f, flo, fhi);
                    } else {
                        r[e] = epi_apply<EPI>(v, ta[e], tb[e], tc[e], td[e], te[e], p.epi.lo, p.epi.hi, p.epi.relu);
                    }
                }
                if (out_bytes) {
                    pk[i][g] = pack_bytes(r[0], r[1], r[2], r[3]) ^ p.out_xor;
                } else {
                    const int ch = n0 + i * 32 + 8 * g + 4 * lh;
                    if (pix_ok && ch < p.out_cs)
                        *(int4*)((int*)p.out + m * p.out_cs + ch) = int4{r[0], r[1], r[2], r[3]};
                }
            }
        }
        if (out_bytes) {
            unsigned qd[NBLK][4];
#pragma unroll
            for (int i = 0; i < NBLK; ++i) {
                const auto s02 = __builtin_amdgcn_permlane32_swap(pk[i][0], pk[i][2], false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(pk[i][1], pk[i][3], false, false);
                qd[i][0] = s02[0]; qd[i][1] = s02[1]; qd[i][2] = s13[0]; qd[i][3] = s13[1];
            }
            v4i first, second;
            if constexpr (NBLK == 2) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const auto x = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[NBLK - 1][e], false, false);
                    first[e] = (int)x[0];
                    second[e] = (int)x[1];
                }
            } else {
                // one block: the lower lane half holds channels 0..15 of its pixel, the upper half channels 16..31
                first = v4i{(int)qd[0][0], (int)qd[0][1], (int)qd[0][2], (int)qd[0][3]};
                second = first;
            }
            if constexpr (POOL) {
                // the row goes to the ring in LDS (a row that does not exist: the smallest byte, which no maximum picks);
                // once the third row of a pooled row is there, that pooled row is computed and stored
                const int pb = cw.b, poy = cw.oy0 + cw.j, pj = cw.j;
                const bool live_row = row_live(cw);
                walk_next(cw);
                if (!live_row) {
                    const int lowest = (int)0x80808080u;     // -128 in every byte: bytes are compared as stored, i.e. signed
                    first = v4i{lowest, lowest, lowest, lowest};
                    second = first;
                }
                unsigned char* rowp = smem + ROWS_OFF + ((pj & 3) * TW + ox) * BN + 32 * lh;
                *(v4i*)rowp = first;
                *(v4i*)(rowp + 16) = second;
                const int py = ((poy + q.pool_pad) >> 1) - 1;      // the pooled row whose last convolution row this is
                if (pj >= 2 && !(pj & 1)) {
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    const int px = tid >> 2, cg = tid & 3;
                    if (px < q.POW && py < q.POH) {
                        v2s me[4], mo[4];
#pragma unroll
                        for (int sy = 0; sy < 3; ++sy) {
                            const unsigned char* rp = smem + ROWS_OFF + (((pj - 2 + sy) & 3) * TW) * BN + cg * 16;
#pragma unroll
                            for (int sx = 0; sx < 3; ++sx) {
                                const int col = min(max(2 * px - q.pool_pad + sx, 0), p.OW - 1);
                                const v4i v = *(const v4i*)(rp + col * BN);
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const unsigned w = (unsigned)v[e];
                                    const unsigned ev = (w << 8) & 0xFF00FF00u, od = w & 0xFF00FF00u;
                                    const v2s ee = as_v2s((int)ev), oo = as_v2s((int)od);
                                    if (sy == 0 && sx == 0) { me[e] = ee; mo[e] = oo; }
                                    else { me[e] = __builtin_elementwise_max(me[e], ee); mo[e] = __builtin_elementwise_max(mo[e], oo); }
                                }
                            }
                        }
                        v4i res;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned ue = (unsigned)__builtin_bit_cast(int, me[e]), uo = (unsigned)__builtin_bit_cast(int, mo[e]);
                            res[e] = (int)(((ue >> 8) & 0x00FF00FFu) | (uo & 0xFF00FF00u));
                        }
                        const long long opix = ((long long)pb * q.POHp + py + q.pool_halo) * q.POWp + px + q.pool_halo;
                        *(v4i*)((signed char*)p.out + opix * p.out_cs + cg * 16) = res;
                    }
                }
            } else {
            if constexpr (NBLK == 2) {
                signed char* orow = (signed char*)p.out + m * p.out_cs + n0 + 32 * lh;
                const int ch = n0 + 32 * lh;
                if (pix_ok) {
                    if (ch < p.out_cs) *(v4i*)orow = first;
                    if (ch + 16 < p.out_cs) *(v4i*)(orow + 16) = second;
                }
            } else {
                const int ch = n0 + 16 * lh;
                if (pix_ok && ch < p.out_cs)
                    *(v4i*)((signed char*)p.out + m * p.out_cs + ch) = first;
            }
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

} // namespace n2d2hip
