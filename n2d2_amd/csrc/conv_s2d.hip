// First-layer convolution on a space-to-depth input (see conv_s2d.hpp), with the 3x3 stride-2 max pooling that follows
// ResNet's first layer optionally computed in the same launch.
//
// Reference semantics: ConvCell_Frame_Kernels::forward (src/Cell/ConvCell_Frame_Kernels.cpp:26-149) skips the taps
// that fall outside the input; a tap on a stored zero adds the same nothing, so reading the border is exact.
// PoolCell_Frame_Kernels::forwardMax (src/Cell/PoolCell_Frame_Kernels.cpp:102-197) takes the maximum over the part of
// the window inside its input; clamping a tap to the nearest row / column inside repeats a value of that part.
//
// How the kernel is organised:
//  * Positions.  The bordered input of the whole batch is one array of 16-byte pixels; output (oy, ox) of image b has
//    its window origin at position ((b * Hp + oy + ty) * Wp + ox + tx) and reads positions p + ky' * Wp + kx'.  A
//    work-group walks a strip of consecutive convolution rows as one stream of positions: a tile is TR rows = TR * Wp
//    consecutive positions (the few positions of a row past the last output are computed and dropped).
//  * Input ring.  The stream is copied global -> LDS by 16-byte direct loads in aligned chunks of 64 positions into a
//    ring of 2048 positions; every wave issues one chunk per tile, two tiles ahead of its use.  The only wait for
//    memory in a tile is `vmcnt(1)` behind the tile's matrix instructions: loads return in order, so with at most one
//    operation in flight the chunk issued one tile earlier has landed (stores of the previous tile had the matrix
//    phase to drain and are not waited for by design, only by coincidence).
//  * One MFMA K step (32 bytes) = two neighbouring pixels of one window row: lane half h supplies pixel 2 * half + h.
//    The 64 x (KS * 32) weights live in registers for the work-group's whole life.  A wave owns 32-position tiles
//    wave, wave + 4 of the tile.
//  * Rescale on scaled-up tables (the result is the upper half of the multiply-add), kept as pairs of 16-bit values.
//    POOL: a wave's two 32-position tiles are not consecutive positions but, lane by lane, the first and the second
//    column of a pooled column's window, so that the maximum along the row is taken between a lane's own registers
//    and its neighbour's (one wave shift); only the row of maxima goes to LDS, a ring of three rows (16-byte chunks
//    XOR-swizzled by the column, so that writes and reads of consecutive columns meet no bank conflict).  Tiles are
//    aligned so that a pooled row's third convolution row is a tile's second, which makes one pooled row ready per
//    tile with three rows alive.  The maximum down the column is taken from LDS by one thread per pooled pixel and 16
//    channels, which saturates and packs only the pooled values (saturation commutes with the maximum).
#include "conv_s2d.hpp"
#include "mfma_util.hpp"

namespace n2d2hip {

template <int NY, int NXH, bool H16, bool POOL, int NBLK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 4))) void conv_s2d_kernel(ConvS2dArgs q)
{
    static_assert(!POOL || (H16 && NBLK == 2), "the pooled variant: 64 channels, scaled-up tables");
    constexpr int KS = NY * NXH;
    constexpr int RING = 2048, RINGB = RING * 16;
    constexpr int BN = 32 * NBLK;
    constexpr int TAB_OFF = RINGB;
    constexpr int TAB_BYTES = H16 ? 0 : 5 * BN * 4;
    constexpr int ROWS_OFF = TAB_OFF + TAB_BYTES;
    constexpr int ROWB = 62 * 128;             // POOL: a row of at most 62 pooled columns, 64 channels as 16-bit values
    constexpr int SPARE_OFF = ROWS_OFF + (POOL ? 3 * ROWB : 0);       // POOL: where lanes without an output write (8 bytes each)
    __shared__ __attribute__((aligned(16))) unsigned char smem[SPARE_OFF + (POOL ? 512 : 0)];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int Wp = q.Wp, T = q.T, NT = q.NT;
    const int n0 = (int)blockIdx.y * BN;          // this work-group's channel tile
#ifdef N2D2HIP_PROFILE
    long long pr_t0 = clock64(), pr_t1 = 0, pr_t2 = 0, pr_w0 = wall_clock64();
    long long pr_ph[6] = {0, 0, 0, 0, 0, 0}, pr_last = 0;
    int pr_units = 0;
#define S2D_MARK(k) do { const long long now__ = clock64(); pr_ph[k] += now__ - pr_last; pr_last = now__; } while (0)
#else
#define S2D_MARK(k) do { } while (0)
#endif

    // ---- weights of this lane's channels: A operand of K step s is 16 bytes at s * 32 + 16 * lh
    v4i wf[NBLK][KS];
#pragma unroll
    for (int i = 0; i < NBLK; ++i)
#pragma unroll
        for (int s = 0; s < KS; ++s)
            wf[i][s] = *(const v4i*)(q.wk + (size_t)(n0 + i * 32 + l32) * (KS * 32) + s * 32 + 16 * lh);
    // ---- rescale: scaled-up multiplier and addend of this lane's channels (rows 8g + 4 * lh + e of each block) in
    // registers, or the five tables of the general integer rescale in LDS
    v4i rc[H16 ? NBLK : 1][H16 ? 4 : 1], rd[H16 ? NBLK : 1][H16 ? 4 : 1];
    if (H16) {
#pragma unroll
        for (int i = 0; i < NBLK; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                rc[H16 ? i : 0][H16 ? g : 0] = *(const v4i*)(q.tc + n0 + i * 32 + 8 * g + 4 * lh);
                rd[H16 ? i : 0][H16 ? g : 0] = *(const v4i*)(q.td + n0 + i * 32 + 8 * g + 4 * lh);
            }
    } else {
        int* tabw = (int*)(smem + TAB_OFF);
        for (int i = tid; i < BN; i += 256) {
            tabw[i] = q.ta[n0 + i];
            tabw[BN + i] = q.tb[n0 + i];
            tabw[2 * BN + i] = q.tc[n0 + i];
            tabw[3 * BN + i] = q.td[n0 + i];
            tabw[4 * BN + i] = q.te[n0 + i];
        }
    }
    const unsigned tab = lds0 + TAB_OFF + (unsigned)(4 * lh) * 4u;
    const int vlo = q.lo, vhi = q.hi;

    // ---- this lane's two positions inside a tile: row of the tile, output column, byte offset of the position (+ lane half)
    // from the tile's first position.
    // Plain convolution: the tile's positions in order, 32-position tiles wave and wave + 4.
    // POOL: a wave owns one of the tile's two convolution rows (wave & 1) and a run of 31 pooled columns (wave >> 1); lane l of
    // its first tile computes the first column of pooled column p_col's window (2 * p_col - pad), of its second tile the
    // second (columns off the row's ends clamped to the nearest inside, which repeats a value of the window), and the
    // window's third column is the first of lane l + 1: the maximum along the row is taken between registers.
    int t_row[2], t_ox[2];
    unsigned t_addr[2];
    const int p_col = POOL ? (wave >> 1) * 31 + l32 : 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (POOL) {
            const int col = min(max(2 * p_col - q.pool_pad + j, 0), q.OW - 1);
            t_row[j] = wave & 1;
            t_ox[j] = col;
            t_addr[j] = (unsigned)((wave & 1) * Wp + q.tx + col + lh) * 16u;
        } else {
            const int pos = (wave + 4 * j) * 32 + l32;
            const int r = div_magic(pos, q.wp_mul, q.wp_sh);
            t_row[j] = r;
            t_ox[j] = pos - r * Wp - q.tx;
            t_addr[j] = (unsigned)(pos + lh) * 16u;
        }
    }
    // byte offset of K step s inside the window: row ky' = s / NXH, pixels 2 * (s % NXH) (+ lane half)
    unsigned koff[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s)
        koff[s] = (unsigned)((s / NXH) * Wp + 2 * (s % NXH)) * 16u;

    // the output through a buffer descriptor: a lane without an output stores past its end, which drops the store
    __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(q.out, 0, POOL ? 0 : q.out_bytes, 0x00020000);
    const int last_pos = q.total - 1;
    const int pf_chunks = q.PF >> 6;
    // chunk `c` (64 positions) of the stream that starts at global position g0 -> its place in the ring
    auto load_chunk = [&](int g0, int c) {
        const int pos = min(max(g0 + (c << 6) + lane, 0), last_pos);        // rows before the first / past the last image: any pixel
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)(q.in + (size_t)pos * 16u), (lds_ptr_t)(smem + ((c << 6) & (RING - 1)) * 16), 16, 0, 0);
    };

    for (int strip = blockIdx.x; strip < q.nstrips; strip += gridDim.x) {
        const int b = strip / q.strips_per_image;
        const int sj = strip - b * q.strips_per_image;
        // rows of the strip: [row0, row0 + ntile * TR) convolution rows; POOL: pooled rows [py0, py1), tiles aligned so that
        // pooled row py0 + k - 1 is complete behind tile k
        int row0, ntile, py0 = 0, py1 = 0, pbase = 0;
        if (POOL) {
            py0 = sj * q.rows_per_strip;
            py1 = min(py0 + q.rows_per_strip, q.POH);
            row0 = 2 * py0 - q.pool_pad - 1;
            ntile = py1 - py0 + 1;
            pbase = py0 - 1;                                      // pooled row behind tile t: pbase + t (none behind tile 0)
            if (row0 + 1 < 0) { row0 += 2; --ntile; ++pbase; }    // a first tile wholly above the image is skipped
        } else {
            row0 = sj * q.rows_per_strip;
            ntile = (min(row0 + q.rows_per_strip, q.OH) - row0 + q.TR - 1) / q.TR;
        }
        const int g0 = (b * q.Hp + row0 + q.ty) * Wp;

        // (the barriers of this kernel are bare s_barrier instructions with the waits they need written out: __syncthreads()
        // would wait for every outstanding load, the chunks requested for later tiles included)
        // ---- fill: the first PF positions of the stream, a chunk per wave in turn
        for (int c = wave; c < pf_chunks; c += 4)
            load_chunk(g0, c);
        asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#ifdef N2D2HIP_PROFILE
        if (pr_t1 == 0) pr_t1 = clock64();
#endif

        for (int t = 0; t < ntile; ++t) {
            // ---- request the chunks that complete tile t + 2's window: [PF + t * T, PF + (t + 1) * T), aligned chunks, one per
            // wave (a wave with nothing new left reloads the last one)
            {
                const int c_lo = (q.PF + t * T + 63) >> 6, c_hi = (q.PF + (t + 1) * T + 63) >> 6;
                load_chunk(g0, min(c_lo + wave, max(c_hi - 1, c_lo)));
            }
#ifdef N2D2HIP_PROFILE
            pr_last = clock64();
#endif
            const unsigned tbase = (unsigned)(t * T) * 16u;
            v16i acc[2][NBLK];
            v4i pf[2][KS];
            v2i hq[POOL ? 2 : 1][POOL ? 4 * NBLK : 1];          // POOL: the two tiles' rescaled values as 16-bit pairs
            // Requests the window of 32-position tile j: K step s = two pixels of window row s / NXH
            auto request = [&](int j) {
                const unsigned a0 = tbase + t_addr[j];
#pragma unroll
                for (int s = 0; s < KS; ++s)
                    lds_read128_nowait<0>(pf[j][s], lds0 + ((a0 + koff[s]) & (unsigned)(RINGB - 1)));
            };
            auto multiply = [&](int j) {
#pragma unroll
                for (int s = 0; s < KS; ++s)
#pragma unroll
                    for (int i = 0; i < NBLK; ++i)
                        acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i][s], pf[j][s], s == 0 ? v16i{} : acc[j][i], 0, 0, 0);
            };
            // Rescales tile j (a wave's second tile past the end of a short row tile computes positions that are dropped).
            // No branch: a lane whose position is no output writes to a spare slot / past the end of the buffer descriptor, so
            // that this code and the matrix instructions of the other tile can be interleaved by the scheduler.
            auto rescale = [&](int j) {
                const int crow = row0 + t * q.TR + t_row[j];                  // convolution row of this lane's position
                const bool ok = t_row[j] < q.TR && (unsigned)t_ox[j] < (unsigned)q.OW && (unsigned)crow < (unsigned)q.OH;
                if constexpr (POOL) {
                    // 16-bit pairs of this tile (one window column per lane), kept for the maximum along the row
#pragma unroll
                    for (int i = 0; i < NBLK; ++i) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const v4i tc = rc[H16 ? i : 0][H16 ? g : 0], td = rd[H16 ? i : 0][H16 ? g : 0];
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                const int t0 = __mul24(acc[j][i][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                                const int t1 = __mul24(acc[j][i][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                                hq[j][i * 4 + g][h] = (int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u);
                            }
                        }
                    }
                    (void)ok;
                } else {
                    unsigned pk[NBLK][4];
                    v4i tq[2][5];
                    auto request_tables = [&](v4i* t5, unsigned trow) {
                        lds_read128_nowait<0>(t5[0], trow);
                        lds_read128_nowait<BN * 4>(t5[1], trow);
                        lds_read128_nowait<2 * BN * 4>(t5[2], trow);
                        lds_read128_nowait<3 * BN * 4>(t5[3], trow);
                        lds_read128_nowait<4 * BN * 4>(t5[4], trow);
                    };
#pragma unroll
                    for (int i = 0; i < NBLK; ++i) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            if constexpr (H16) {
                                const v4i tc = rc[H16 ? i : 0][H16 ? g : 0], td = rd[H16 ? i : 0][H16 ? g : 0];
                                v2s pq[2];
#pragma unroll
                                for (int h = 0; h < 2; ++h) {
                                    const int t0 = __mul24(acc[j][i][4 * g + 2 * h], tc[2 * h]) + td[2 * h];
                                    const int t1 = __mul24(acc[j][i][4 * g + 2 * h + 1], tc[2 * h + 1]) + td[2 * h + 1];
                                    pq[h] = as_v2s((int)__builtin_amdgcn_perm((unsigned)t1, (unsigned)t0, 0x07060302u));
                                }
                                if (vlo == 0 && vhi == 255) {
                                    pk[i][g] = (sat_pk_u8(pq[0]) | (sat_pk_u8(pq[1]) << 16)) ^ q.out_xor;
                                } else {
                                    const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
                                    pk[i][g] = __builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(pq[1], lo1, hi1)),
                                                                     (unsigned)__builtin_bit_cast(int, clamp_v2s(pq[0], lo1, hi1)), 0x06040200u) ^ q.out_xor;
                                }
                            } else {
                                // the tables of the next channel group are requested before this one is rescaled
                                const int u = i * 4 + g;
                                if (u == 0)
                                    request_tables(tq[0], tab);
                                if (u + 1 < 4 * NBLK) {
                                    request_tables(tq[(u + 1) & 1], tab + (unsigned)(((u + 1) / 4) * 32 + 8 * ((u + 1) % 4)) * 4u);
                                    wait_lgkm<5>();
                                } else {
                                    wait_lgkm<0>();
                                }
                                v4i* t5 = tq[u & 1];
                                tie(t5[0]); tie(t5[1]); tie(t5[2]); tie(t5[3]); tie(t5[4]);
                                int r[4];
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    int v = acc[j][i][4 * g + e];
                                    if (q.preclamp) v = med3_i32(v, t5[0][e], t5[1][e]);
                                    r[e] = med3_i32((__mul24(v, t5[2][e]) + t5[3][e]) >> t5[4][e], vlo, vhi);
                                }
                                pk[i][g] = pack_bytes(r[0], r[1], r[2], r[3]) ^ q.out_xor;
                            }
                        }
                    }
                    // pk[i][g] holds channels 8g + 4 * lh .. + 3 of block i: exchanges between the lane halves leave a lane with
                    // 16 consecutive channels of its pixel (one block) or 32 (two blocks)
                    unsigned qd[NBLK][4];
#pragma unroll
                    for (int i = 0; i < NBLK; ++i) {
                        const auto s02 = __builtin_amdgcn_permlane32_swap(pk[i][0], pk[i][2], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(pk[i][1], pk[i][3], false, false);
                        qd[i][0] = s02[0]; qd[i][1] = s02[1]; qd[i][2] = s13[0]; qd[i][3] = s13[1];
                    }
                    const int m = (b * q.OH + crow) * q.OW + t_ox[j];
                    if constexpr (NBLK == 2) {
                        v4i first, second;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const auto x = __builtin_amdgcn_permlane32_swap(qd[0][e], qd[NBLK - 1][e], false, false);
                            first[e] = (int)x[0];
                            second[e] = (int)x[1];
                        }
                        const int ch = n0 + 32 * lh;
                        const unsigned off = (unsigned)(m * q.out_cs + ch);
                        __builtin_amdgcn_raw_buffer_store_b128(first, out_rsrc, (ok && ch < q.out_cs) ? off : 0x80000000u, 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b128(second, out_rsrc, (ok && ch + 16 < q.out_cs) ? off + 16u : 0x80000000u, 0, 0);
                    } else {
                        const v4i only = {(int)qd[0][0], (int)qd[0][1], (int)qd[0][2], (int)qd[0][3]};
                        const int ch = n0 + 16 * lh;
                        __builtin_amdgcn_raw_buffer_store_b128(only, out_rsrc, (ok && ch < q.out_cs) ? (unsigned)(m * q.out_cs + ch) : 0x80000000u, 0, 0);
                    }
                }
            };

            // ---- the tile: the first 32-position tile's products, then the second's while the first is rescaled
            request(0);
            request(1);
            wait_lgkm<KS>();           // the LDS answers in order: the first tile's reads have arrived
#pragma unroll
            for (int s = 0; s < KS; ++s) tie(pf[0][s]);
            multiply(0);
            S2D_MARK(0);
            if (POOL)
                asm volatile("s_barrier" ::: "memory");          // the pooling of the previous tile has read the rows this tile overwrites
            S2D_MARK(1);
            wait_lgkm<0>();
#pragma unroll
            for (int s = 0; s < KS; ++s) tie(pf[1][s]);
            multiply(1);
            S2D_MARK(2);
            rescale(0);
            rescale(1);
            if constexpr (POOL) {
                // ---- maximum along the row: window columns 2p - pad, + 1 (this lane's two tiles) and + 2 (the first tile of the
                // next lane, fetched by a shift of the wave by one lane; lane 31 of a half has no such neighbour and its pooled
                // column belongs to the next run).  The row of pooled columns goes to the ring of three rows in LDS: a lane's
                // four channels 32 * i + 8 * g + 4 * lh .. + 3 are one half (lh) of the pixel's 16-byte chunk 4 * i + g.
                const int crow = row0 + 2 * t + (wave & 1);
                const bool ok = l32 < 31 && p_col < q.POW && (unsigned)crow < (unsigned)q.OH;
                const unsigned pix = lds0 + ROWS_OFF + (unsigned)((crow + 3) % 3) * ROWB + (unsigned)p_col * 128u + 8u * (unsigned)lh;
                const unsigned sw = (unsigned)(p_col & 7);
#pragma unroll
                for (int u = 0; u < 4 * NBLK; ++u) {
                    v2i hm;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int next = __builtin_amdgcn_update_dpp(0, hq[0][u][h], 0x130, 0xf, 0xf, false);       // wave_shl:1
                        const v2s m = __builtin_elementwise_max(__builtin_elementwise_max(as_v2s(hq[0][u][h]), as_v2s(hq[POOL ? 1 : 0][u][h])), as_v2s(next));
                        hm[h] = __builtin_bit_cast(int, m);
                    }
                    const unsigned at = ok ? pix + ((sw ^ (unsigned)u) << 4) : lds0 + SPARE_OFF + (unsigned)lane * 8u;
                    *(__attribute__((address_space(3))) v2i*)(unsigned long)at = hm;
                }
            }
            S2D_MARK(3);
            // Order asked of the scheduler: the first tile's matrix instructions back to back, then each of the second tile's
            // followed by a few of the first tile's rescale instructions, which run while the matrix core is busy.
#pragma unroll
            for (int k = 0; k < KS * NBLK; ++k)
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
            for (int k = 0; k < KS * NBLK; ++k) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, POOL ? 5 : 6, 0);
            }
            // the chunk requested one tile ago has landed (see the head of this file); behind the next barrier every
            // wave's has
            asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
#ifdef N2D2HIP_PROFILE
            if (pr_t2 == 0) pr_t2 = clock64();
            ++pr_units;
#endif

            if constexpr (POOL) {
                // ---- pooled row py = pbase + t: rows 2 * py - pad .. + 2, the last of which this tile has just written
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                S2D_MARK(4);
                const int py = pbase + t;
                const int px = lane, cg = wave;
                if (py >= py0 && py < py1 && px < q.POW) {
                    // rows 2 * py - pad .. + 2 of the row maxima, clamped to the rows that exist: 16 channels (chunks 2 * cg, + 1)
                    v2s m[8];
                    v4i v[3][2];
#pragma unroll
                    for (int sy = 0; sy < 3; ++sy) {
                        const int r = min(max(2 * py - q.pool_pad + sy, 0), q.OH - 1);
                        const unsigned pix = lds0 + ROWS_OFF + (unsigned)(r % 3) * ROWB + (unsigned)px * 128u;
                        const unsigned sw = (unsigned)(px & 7);
                        lds_read128_nowait<0>(v[sy][0], pix + ((sw ^ (unsigned)(2 * cg)) << 4));
                        lds_read128_nowait<0>(v[sy][1], pix + ((sw ^ (unsigned)(2 * cg + 1)) << 4));
                    }
                    wait_lgkm<0>();
#pragma unroll
                    for (int sy = 0; sy < 3; ++sy) {
                        tie(v[sy][0]); tie(v[sy][1]);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const v2s x = as_v2s(v[sy][e >> 2][e & 3]);
                            m[e] = sy == 0 ? x : __builtin_elementwise_max(m[e], x);
                        }
                    }
                    v4i res;
                    if (vlo == 0 && vhi == 255) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            res[e] = (int)((sat_pk_u8(m[2 * e]) | (sat_pk_u8(m[2 * e + 1]) << 16)) ^ q.out_xor);
                    } else {
                        const v2s lo1 = splat_v2s(vlo), hi1 = splat_v2s(vhi);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            res[e] = (int)(__builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, clamp_v2s(m[2 * e + 1], lo1, hi1)),
                                                                 (unsigned)__builtin_bit_cast(int, clamp_v2s(m[2 * e], lo1, hi1)), 0x06040200u) ^ q.out_xor);
                    }
                    const long long opix = ((long long)b * q.POHp + py + q.pool_halo) * q.POWp + px + q.pool_halo;
                    *(v4i*)((signed char*)q.out + opix * q.out_cs + cg * 16) = res;
                }
                S2D_MARK(5);
            } else {
                // every wave is done with this tile's window before the chunks of later tiles overwrite part of it
                asm volatile("s_barrier" ::: "memory");
                S2D_MARK(4);
            }
        }
        // every wave is done reading the ring, and nothing requested for this strip is still on its way into it, before the
        // next strip refills it
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    }
#ifdef N2D2HIP_PROFILE
    if (tid == 0 && q.prof) {
        long long* o = q.prof + (long long)blockIdx.x * 16;
        o[0] = pr_t0; o[1] = pr_t1; o[2] = pr_t2; o[3] = clock64(); o[4] = 0; o[5] = pr_w0; o[6] = wall_clock64(); o[7] = pr_units;
        for (int k = 0; k < 6; ++k) o[8 + k] = pr_ph[k];
    }
#endif
    // no load may still be writing into LDS when the block's LDS is handed to another block
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
}

// ----------------------------------------------------------------------------------------------------------- host

static void geometry(int k, int pad, int* qn, int* f)
{
    *qn = (pad + 1) / 2;          // border pixels in front
    *f = 2 * *qn - pad;           // zero taps in front (0 or 1)
}

size_t conv_s2d_weight_bytes(int O, int k, int pad)
{
    (void)pad;
    const int ny = (k + 1) / 2, nxh = (ny + 1) / 2;
    return (size_t)round_up(O, 64) * ny * nxh * 32;
}

void conv_s2d_weight_layout(const signed char* w, int C, int O, int k, int padT, int padL, signed char* out)
{
    const int ny = (k + 1) / 2, nxh = (ny + 1) / 2, ks = ny * nxh;
    int qy, fy, qx, fx;
    geometry(k, padT, &qy, &fy);
    geometry(k, padL, &qx, &fx);
    memset(out, 0, conv_s2d_weight_bytes(O, k, padT));
    for (int o = 0; o < O; ++o)
        for (int kyp = 0; kyp < ny; ++kyp)
            for (int kxp = 0; kxp < 2 * nxh; ++kxp)
                for (int dy = 0; dy < 2; ++dy)
                    for (int dx = 0; dx < 2; ++dx) {
                        const int ky = 2 * kyp + dy - fy, kx = 2 * kxp + dx - fx;
                        if (ky < 0 || ky >= k || kx < 0 || kx >= k)
                            continue;
                        const int s = kyp * nxh + kxp / 2;
                        for (int ch = 0; ch < C; ++ch)
                            out[((size_t)o * ks + s) * 32 + (kxp & 1) * 16 + (dy * 2 + dx) * 4 + ch] = w[(((size_t)o * C + ch) * k + ky) * k + kx];
                    }
}

int conv_s2d_halo(int k, int padT, int padL, int padB, int padR, int H, int W)
{
    if ((k != 3 && k != 5 && k != 7) || padT < 0 || padL < 0 || padB < 0 || padR < 0 || H < 2 || W < 2)
        return -1;
    const int ny = (k + 1) / 2, nxh = (ny + 1) / 2;
    int qy, fy, qx, fx;
    geometry(k, padT, &qy, &fy);
    geometry(k, padL, &qx, &fx);
    const int OH = (H + padT + padB - k) / 2 + 1, OW = (W + padL + padR - k) / 2 + 1;
    const int Hs = (H + 1) / 2, Ws = (W + 1) / 2;
    // the last window's last row / pixel pair must lie inside the bordered image
    int halo = std::max(std::max(qy, qx), 0);
    halo = std::max(halo, OH - qy + ny - 1 - Hs);
    halo = std::max(halo, OW - qx + 2 * nxh - 1 - Ws);
    // an even border keeps the pixel pairs of a stored row aligned with those of the input's rows: the conversion then
    // moves whole dwords (a larger border than needed is as good to the kernel)
    return (halo + 1) & ~1;
}

int conv_s2d_launch(ConvS2dArgs a, int k, bool hi16, bool pool, int nblk, int blocks, int channel_tiles, hipStream_t stream)
{
    const dim3 grid(blocks, channel_tiles);
#define N2D2HIP_S2D(NY, NXH)                                                                                              \
    do {                                                                                                                  \
        if (pool) N2D2HIP_LAUNCH_T(conv_s2d_kernel, (NY, NXH, true, true, 2), grid, dim3(256), 0, stream, a);     \
        else if (nblk == 2 && hi16) N2D2HIP_LAUNCH_T(conv_s2d_kernel, (NY, NXH, true, false, 2), grid, dim3(256), 0, stream, a);  \
        else if (nblk == 2) N2D2HIP_LAUNCH_T(conv_s2d_kernel, (NY, NXH, false, false, 2), grid, dim3(256), 0, stream, a);         \
        else if (hi16) N2D2HIP_LAUNCH_T(conv_s2d_kernel, (NY, NXH, true, false, 1), grid, dim3(256), 0, stream, a);               \
        else N2D2HIP_LAUNCH_T(conv_s2d_kernel, (NY, NXH, false, false, 1), grid, dim3(256), 0, stream, a);                        \
    } while (0)
    if (k == 3) N2D2HIP_S2D(2, 1);
    else if (k == 5) N2D2HIP_S2D(3, 2);
    else N2D2HIP_S2D(4, 2);
#undef N2D2HIP_S2D
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // namespace n2d2hip
