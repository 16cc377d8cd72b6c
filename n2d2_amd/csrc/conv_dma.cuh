// Persistent implicit-GEMM convolution with a multi-stage LDS ring filled by
// direct global->LDS loads (global_load_lds_dwordx4), for int8 weights and
// activations with a channel stride that is a multiple of 16.
//
// One K step of a 128x128 tile is only 256 matrix-core cycles per wavefront,
// while a global load takes a few thousand cycles to return and every vector
// ALU instruction costs 4 cycles of the same SIMD.  So:
//  * S-1 K steps are always in flight per block; the loads land in LDS by
//    themselves (no staging registers, no LDS store instructions);
//  * the ring runs across tile boundaries: a block walks a list of pixel tiles
//    for one channel tile, the loads of the next tile are in flight while the
//    current one is rescaled and stored;
//  * the steady state is stripped of address arithmetic: the step loop is
//    unrolled over the ring so that stage offsets are instruction immediates,
//    fragment addresses are four loop-invariant registers, tap offsets come
//    precomputed from an LDS table, rows are 32-bit offsets, the bias is the
//    accumulators' initial value.
//
// Because the loads complete asynchronously, every LDS access of this kernel is
// explicit: waits are written by hand (s_waitcnt vmcnt(n) counts the loads that
// may still be outstanding), LDS reads and writes are inline ds_* instructions.
//   step w:  wait until the loads of step w have landed (all but the youngest
//            S-2 steps' loads complete), barrier, issue the loads of step w+S-1
//            into the stage freed by step w-1, run the MFMAs of step w.
// A thread issues the same number of loads at every step (steps past the end
// of its work fetch a constant 16-byte block), so the count is uniform.  Global
// stores of the epilogue also count in vmcnt and may retire out of order with
// the loads; that can only make a wait longer, never shorter: n counts younger
// LOADS, which return in order.
#pragma once

namespace n2d2hip {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

template <int OFF>
__device__ __forceinline__ void lds_read128_nowait(v4i& v, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
}
__device__ __forceinline__ void lds_write32(unsigned addr, unsigned value)
{
    asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(value) : "memory");
}
// Makes the data of earlier asynchronous LDS reads usable: ties the registers to the wait.
__device__ __forceinline__ void lds_wait(v4i& a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a) : : "memory"); }
__device__ __forceinline__ void lds_wait(v4i& a, v4i& b) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b) : : "memory"); }
__device__ __forceinline__ void lds_wait(v4i& a, v4i& b, v4i& c) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c) : : "memory"); }
__device__ __forceinline__ void lds_wait(v4i& a, v4i& b, v4i& c, v4i& d)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : : "memory");
}
__device__ __forceinline__ void lds_wait(v4i& a, v4i& b, v4i& c, v4i& d, v4i& e)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : : "memory");
}
__device__ __forceinline__ void lds_wait(v4i& a, v4i& b, v4i& c, v4i& d, v4i& e, v4i& f)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f) : : "memory");
}

struct ConvDmaArgs {
    ConvArgs c;
    const signed char* fill16;   // 16 bytes of the input's logical zero (device)
    int mtiles, mlanes;          // pixel tiles, and how many block "lanes" walk them
    int all_valid;               // 1x1 kernel without padding: every tap of an existing pixel is inside the input
};

template <int N>
__device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(N) : "memory");
}

// 4 saturated values -> one dword of bytes
__device__ __forceinline__ unsigned pack_bytes(int r0, int r1, int r2, int r3)
{
    const unsigned t01 = __builtin_amdgcn_perm((unsigned)r1, (unsigned)r0, 0x0c0c0400u);
    const unsigned t23 = __builtin_amdgcn_perm((unsigned)r3, (unsigned)r2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(t23, t01, 0x05040100u);
}

template <int BM, int BN, int WGM, int EPI, int S>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_dma_kernel(ConvDmaArgs q)
{
    const ConvArgs& p = q.c;
    constexpr int WGN = 4 / WGM;
    constexpr int TM = BM / WGM, TN = BN / WGN;
    constexpr int NI = TN / 32, NJ = TM / 32;
    constexpr int A_J = BM / 64, B_J = BN / 64;        // 1 KB chunks (16 rows) each thread's wave loads per step
    constexpr int LPI = A_J + B_J;                     // loads per thread and step
    constexpr int STAGE = (BM + BN) * 64;
    constexpr int MAX_SUB = 512;                       // sub-chunk table entries held in LDS
    constexpr int TAB_OFF = S * STAGE;                 // 6 int arrays of BN entries: bias, a, b, c, d, e
    constexpr int SUB_OFF = TAB_OFF + 6 * BN * 4;
    static_assert(BM * BN <= STAGE, "the output tile is staged in one ring stage");
    static_assert(LPI * (S - 1) < 60, "vmcnt is a 6-bit counter");
    static_assert((S - 1) * STAGE + 2048 < 65536 && 6 * BN * 4 + 256 < 65536, "ds_read immediate offsets are 16 bits");
    static_assert(NI <= 2 && NJ <= 2, "wave tile is at most 2x2 MFMA tiles");

    __shared__ __attribute__((aligned(16))) unsigned char smem[SUB_OFF + MAX_SUB * 16];
    const unsigned lds0 = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int l32 = lane & 31, lh = lane >> 5;

    // ---- which tiles this block walks: one channel tile, every mlanes-th pixel tile.
    // Blocks 8 apart run on the same XCD; they take the same pixel tiles for neighbouring channel tiles.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % p.ntiles_n;
    const int mlane = (slot / p.ntiles_n) * 8 + xcd;
    const int n0 = tile_n * BN;
    const int ntile = (mlane < q.mtiles) ? (q.mtiles - mlane + q.mlanes - 1) / q.mlanes : 0;
    const int niter = p.niter;
    const int nsteps = ntile * niter;

    // ---- per-block constants into LDS: rescale tables + bias of the channel tile, and the sub-chunk table
    // with the byte offset of each tap already multiplied out: {ky, kx, offset, valid<<30 | dx<<15 | dy}
    {
        int* tab = (int*)(smem + TAB_OFF);
        for (int i = tid; i < BN; i += 256) {
            tab[i] = p.bias[n0 + i];
            if (EPI != EPI_RAW) {
                tab[BN + i] = p.epi.a[n0 + i];
                tab[2 * BN + i] = p.epi.b[n0 + i];
                tab[3 * BN + i] = p.epi.c[n0 + i];
                tab[4 * BN + i] = (EPI == EPI_I24) ? p.epi.d[n0 + i] : 0;
                tab[5 * BN + i] = (EPI != EPI_F32) ? p.epi.e[n0 + i] : 0;
            }
        }
        int4* sub = (int4*)(smem + SUB_OFF);
        for (int i = tid; i < niter * 4; i += 256) {
            int4 e = p.sub[i];
            const int dy = e.x * p.dilY, dx = e.y * p.dilX;
            e.z = (dy * p.W + dx) * p.in_cs + e.z;
            e.w = (e.w ? (1 << 30) : 0) | (dx << 15) | dy;
            sub[i] = e;
        }
    }
    __syncthreads();

    // ---- loader state.  Lane l of a wave fills 16-byte slot l of a 1 KB chunk: row l/4 of the chunk,
    // physical sub-chunk l%4, which holds logical sub-chunk (l%4) ^ ((row/4)%4) of that row.
    const int lrow = lane >> 2;
    const int lq = (lane & 3) ^ ((lane >> 4) & 3);
    const unsigned sub_addr = lds0 + SUB_OFF + (unsigned)lq * 16u;
    unsigned woff[B_J];            // byte offset into the prepared weights, advanced by 64 per step
#pragma unroll
    for (int j = 0; j < B_J; ++j)
        woff[j] = (unsigned)((n0 + (wave + 4 * j) * 16 + lrow) * p.ktot + lq * 16);
    int rowoff[A_J];               // byte offset of the window origin of this thread's pixel rows
    int ymin[A_J], ylim[A_J], xmin[A_J], xlim[A_J];
    int l_tile = 0, l_it = 0;
    const int ohw = p.OH * p.OW;
    auto loader_new_tile = [&]() {
        const int m0 = (mlane + l_tile * q.mlanes) * BM;
#pragma unroll
        for (int j = 0; j < A_J; ++j) {
            const int m = m0 + (wave + 4 * j) * 16 + lrow;
            if (l_tile < ntile && m < p.M) {
                const int b = m / ohw;
                const int rem = m - b * ohw;
                const int oy = rem / p.OW;
                const int ox = rem - oy * p.OW;
                const int by = oy * p.strideY - p.padT, bx = ox * p.strideX - p.padL;
                ymin[j] = -by; ylim[j] = p.H - by;
                xmin[j] = -bx; xlim[j] = p.W - bx;
                rowoff[j] = ((b * p.H + by) * p.W + bx) * p.in_cs;
            } else {
                ymin[j] = 1 << 28; ylim[j] = 0; xmin[j] = 1 << 28; xlim[j] = 0;       // no tap is valid
                rowoff[j] = 0;
            }
        }
    };
    loader_new_tile();

    // Issues the LPI loads of the loader's current step into ring stage STG, then advances the loader.
    auto issue = [&](auto stg) {
        constexpr int STG = decltype(stg)::value;
        unsigned char* sbase = smem + STG * STAGE;
        if (l_tile < ntile) {
            v4i s;
            asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(s) : "v"(sub_addr + (unsigned)l_it * 64u) : "memory");
            const int dy = s[3] & 0x7fff, dx = (s[3] >> 15) & 0x7fff;
#pragma unroll
            for (int j = 0; j < A_J; ++j) {
                // branch-free: tap index >= max(pad - o*stride, 0) and dilated offset inside the input
                // (ref: src/Cell/ConvCell_Frame_Kernels.cpp:72-83)
                const int okv = (s[3] >> 30) & (int)(s[0] >= ymin[j]) & (int)(dy < ylim[j]) & (int)(s[1] >= xmin[j]) & (int)(dx < xlim[j]);
                const bool ok = q.all_valid ? (ylim[j] != 0) : (okv != 0);
                const signed char* src = ok ? p.in + (rowoff[j] + s[2]) : q.fill16;
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)(sbase + (wave + 4 * j) * 1024), 16, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < B_J; ++j) {
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)(p.w + woff[j]), (lds_ptr_t)(sbase + BM * 64 + (wave + 4 * j) * 1024), 16, 0, 0);
                woff[j] += 64;
            }
            if (++l_it == niter) {
                l_it = 0;
                ++l_tile;
#pragma unroll
                for (int j = 0; j < B_J; ++j)
                    woff[j] -= (unsigned)niter * 64u;
                loader_new_tile();
            }
        } else {
            // past the end: keep the per-step load count uniform
#pragma unroll
            for (int j = 0; j < LPI; ++j)
                __builtin_amdgcn_global_load_lds((gbl_ptr_t)q.fill16, (lds_ptr_t)(sbase + (wave + 4 * j) * 1024), 16, 0, 0);
        }
    };

    // ---- loop-invariant fragment addresses: (operand, k half) -> one register; tiles and stages are immediates
    const unsigned p_addr0 = lds0 + swz(wm * TM + l32, lh), p_addr1 = lds0 + swz(wm * TM + l32, 2 + lh);
    const unsigned w_addr0 = lds0 + BM * 64 + swz(wn * TN + l32, lh), w_addr1 = lds0 + BM * 64 + swz(wn * TN + l32, 2 + lh);
    const unsigned tab = lds0 + TAB_OFF + (unsigned)(wn * TN + 4 * lh) * 4u;      // this lane's first channel in the tables

    v16i acc[NI][NJ];
    auto init_acc = [&]() {
        // the accumulators start from the bias: channel rows 8g + 4*lh + t of each 32-channel tile
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            v4i b0, b1, b2, b3;
            if (i == 0) {
                lds_read128_nowait<0>(b0, tab); lds_read128_nowait<32>(b1, tab); lds_read128_nowait<64>(b2, tab); lds_read128_nowait<96>(b3, tab);
            } else {
                lds_read128_nowait<128>(b0, tab); lds_read128_nowait<160>(b1, tab); lds_read128_nowait<192>(b2, tab); lds_read128_nowait<224>(b3, tab);
            }
            lds_wait(b0, b1, b2, b3);
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    acc[i][j][t] = b0[t];
                    acc[i][j][4 + t] = b1[t];
                    acc[i][j][8 + t] = b2[t];
                    acc[i][j][12 + t] = b3[t];
                }
        }
    };
    init_acc();

    int c_tile = 0, c_it = 0;

    // One K step on ring stage STG: returns after the epilogue when the step finishes a tile.
    auto step = [&](auto stg) {
        constexpr int STG = decltype(stg)::value;
        constexpr int SOFF = STG * STAGE;
        wait_loads_and_barrier<LPI*(S - 2)>();
        issue(std::integral_constant<int, (STG + S - 1) % S>());       // into the stage step w-1 used
        {
            v4i wf0, wf1, pf0, pf1;
            lds_read128_nowait<SOFF>(wf0, w_addr0);
            if (NI == 2) lds_read128_nowait<SOFF + 2048>(wf1, w_addr0);
            lds_read128_nowait<SOFF>(pf0, p_addr0);
            if (NJ == 2) lds_read128_nowait<SOFF + 2048>(pf1, p_addr0);
            v4i wg0, wg1, pg0, pg1;
            lds_read128_nowait<SOFF>(wg0, w_addr1);
            if (NI == 2) lds_read128_nowait<SOFF + 2048>(wg1, w_addr1);
            lds_read128_nowait<SOFF>(pg0, p_addr1);
            if (NJ == 2) lds_read128_nowait<SOFF + 2048>(pg1, p_addr1);
            if (NI == 2 && NJ == 2) lds_wait(wf0, wf1, pf0, pf1);
            else if (NI == 1 && NJ == 2) lds_wait(wf0, pf0, pf1);
            else if (NI == 2 && NJ == 1) lds_wait(wf0, wf1, pf0);
            else lds_wait(wf0, pf0);
            acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf0, pf0, acc[0][0], 0, 0, 0);
            if (NJ == 2) acc[0][NJ - 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf0, pf1, acc[0][NJ - 1], 0, 0, 0);
            if (NI == 2) acc[NI - 1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf1, pf0, acc[NI - 1][0], 0, 0, 0);
            if (NI == 2 && NJ == 2) acc[NI - 1][NJ - 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf1, pf1, acc[NI - 1][NJ - 1], 0, 0, 0);
            if (NI == 2 && NJ == 2) lds_wait(wg0, wg1, pg0, pg1);
            else if (NI == 1 && NJ == 2) lds_wait(wg0, pg0, pg1);
            else if (NI == 2 && NJ == 1) lds_wait(wg0, wg1, pg0);
            else lds_wait(wg0, pg0);
            acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wg0, pg0, acc[0][0], 0, 0, 0);
            if (NJ == 2) acc[0][NJ - 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wg0, pg1, acc[0][NJ - 1], 0, 0, 0);
            if (NI == 2) acc[NI - 1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wg1, pg0, acc[NI - 1][0], 0, 0, 0);
            if (NI == 2 && NJ == 2) acc[NI - 1][NJ - 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wg1, pg1, acc[NI - 1][NJ - 1], 0, 0, 0);
        }
        if (++c_it != niter)
            return;

        // ---- epilogue of the finished tile.  The stage just consumed becomes the output staging area
        // ([pixel][BN bytes], 16-byte slots XOR-swizzled by the pixel); the next step's loads go elsewhere.
        const int m0 = (mlane + c_tile * q.mlanes) * BM;
        const bool out_bytes = p.out_dtype != N2D2HIP_I32;
        const unsigned tp = lds0 + SOFF;
        if (out_bytes)
            asm volatile("s_barrier" ::: "memory");      // every wave is done reading this stage
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ch_local = wn * TN + i * 32 + 8 * g + 4 * lh;
                const unsigned trow = tab + (unsigned)(i * 32 + 8 * g) * 4u;
                v4i ta = {0, 0, 0, 0}, tb = ta, tc = ta, td = ta, te = ta;
                if (EPI != EPI_RAW) {
                    lds_read128_nowait<BN * 4>(ta, trow);
                    lds_read128_nowait<2 * BN * 4>(tb, trow);
                    lds_read128_nowait<3 * BN * 4>(tc, trow);
                    if (EPI == EPI_I24) lds_read128_nowait<4 * BN * 4>(td, trow);
                    if (EPI != EPI_F32) lds_read128_nowait<5 * BN * 4>(te, trow);
                    lds_wait(ta, tb, tc, td, te);
                }
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int pix_local = wm * TM + j * 32 + l32;
                    const int r0 = epi_apply<EPI>(acc[i][j][4 * g + 0], ta[0], tb[0], tc[0], td[0], te[0], p.epi.lo, p.epi.hi, p.epi.relu);
                    const int r1 = epi_apply<EPI>(acc[i][j][4 * g + 1], ta[1], tb[1], tc[1], td[1], te[1], p.epi.lo, p.epi.hi, p.epi.relu);
                    const int r2 = epi_apply<EPI>(acc[i][j][4 * g + 2], ta[2], tb[2], tc[2], td[2], te[2], p.epi.lo, p.epi.hi, p.epi.relu);
                    const int r3 = epi_apply<EPI>(acc[i][j][4 * g + 3], ta[3], tb[3], tc[3], td[3], te[3], p.epi.lo, p.epi.hi, p.epi.relu);
                    if (out_bytes) {
                        const unsigned packed = pack_bytes(r0, r1, r2, r3) ^ p.out_xor;
                        const int slot16 = (ch_local >> 4) ^ (pix_local & (BN / 16 - 1));
                        lds_write32(tp + pix_local * BN + slot16 * 16 + (ch_local & 15), packed);
                    } else {
                        const int m = m0 + pix_local;
                        const int ch = n0 + ch_local;
                        if (m < p.M && ch < p.out_cs)
                            *(int4*)((int*)p.out + (long long)m * p.out_cs + ch) = int4{r0, r1, r2, r3};
                    }
                }
            }
        }
        init_acc();
        if (out_bytes) {
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // staging complete
            constexpr int CHUNKS = BN / 16;
#pragma unroll
            for (int id = tid; id < BM * CHUNKS; id += 256) {
                const int row = id / CHUNKS;
                const int cq = id - row * CHUNKS;
                const int m = m0 + row;
                const int ch = n0 + cq * 16;
                v4i v;
                lds_read128_nowait<0>(v, tp + row * BN + ((cq ^ (row & (CHUNKS - 1))) << 4));
                lds_wait(v);
                if (m < p.M && ch < p.out_cs)
                    *(v4i*)((signed char*)p.out + (long long)m * p.out_cs + ch) = v;
            }
        }
        c_it = 0;
        ++c_tile;
    };

    // ---- fill the ring, then run: the step loop is unrolled over the ring so that stages are compile-time
    if (S > 1) issue(std::integral_constant<int, 0>());
    if (S > 2) issue(std::integral_constant<int, 1 % S>());
    if (S > 3) issue(std::integral_constant<int, 2 % S>());
    if (S > 4) issue(std::integral_constant<int, 3 % S>());
    static_assert(S >= 2 && S <= 5, "ring depth");
    for (int w = 0; w < nsteps; w += S) {
        step(std::integral_constant<int, 0>());
        if (w + 1 < nsteps) step(std::integral_constant<int, 1 % S>());
        if (S > 2 && w + 2 < nsteps) step(std::integral_constant<int, 2 % S>());
        if (S > 3 && w + 3 < nsteps) step(std::integral_constant<int, 3 % S>());
        if (S > 4 && w + 4 < nsteps) step(std::integral_constant<int, 4 % S>());
    }
    // no load may still be writing into LDS when the block's LDS is handed to another block
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

} // namespace n2d2hip
