// Prefill product y[M,N] = x[M,K] * dequant(W)[N,K]^T for large M (compute-bound).
//
// Replaces xe_linear.forward_new at large M
// (python/llm/src/ipex_llm/transformers/low_bit_linear.py:660-668).
//
// Workgroup tile: 128 rows of x (M) by 256 weight rows (N), 4 waves side by side along N,
// so that every weight is dequantized by exactly one wave.  Per 128-column step of K:
//   weights: each lane loads its 16/32 bytes of four tiles straight from HBM into registers -
//            the tiled layout already is the MFMA operand layout - and turns them into scaled
//            fp16 / bf16 values in registers (no LDS for weights);
//   x:       the workgroup copies the 128 x 128 block of x into LDS in operand order
//            (double buffered), and every wave reads it from there;
//   8 v_mfma_f32_32x32x16 per 16 columns and wave, weights as the A operand (rows = n) and x
//   as the B operand (columns = m), so a lane ends up with groups of 4 consecutive n for one m
//   and stores 8 contiguous bytes of y at a time.
// FLOP per launch: 2*M*N*K; MFMA-bound (fp16 / bf16 dense peak).
#include "lowbit_gemm.h"

namespace lowbit {

int launch_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                int waves, hipStream_t st);

constexpr int GM = 128;          // rows of x per workgroup (the tall form below takes 256)
constexpr int GN_WAVE = 64;      // weight rows per wave
constexpr int GN = 256;          // weight rows per workgroup (4 waves)

constexpr int MB32 = GM / 32;        // 32-row blocks of x per workgroup
constexpr int NB32 = GN_WAVE / 32;   // 32-row blocks of W per wave (two tiles each)
constexpr int GM_TALL = 256, MB32_TALL = GM_TALL / 32;

// Operand layout of v_mfma_f32_32x32x16: lane l = 32*kg + i holds 8 consecutive k (8*kg .. +7 of
// the 16-column step) of row/column i.  A 32-row weight block is two tiles (rows 0-15, 16-31);
// in a tile, lane slot 16*c + r holds columns 8*c .. +7 of each 32-column sub-block, so lane
// (kg, i) takes slot 16*kg + i%16 of tile i/16 for the first 16 columns of every sub-block
// ("lo" registers) and slot 16*(kg+2) + i%16 for the second 16 columns ("hi" registers).
//
// MB = 32-row blocks of x per workgroup: 4 (128 rows) or, for the tall form, 8 (256 rows, DMA form only).  The
// tall form dequantizes every weight once per 256 rows of x: half the VALU work, half the weight loads and
// half the barriers per MFMA; its 16 accumulator blocks take all 256 accumulation registers, so a CU holds
// one workgroup.  tn0 / tn_cnt: the launch covers the column tiles tn0 .. tn0 + tn_cnt - 1 of y.
template <int QT, typename AT, bool DMA, int MB>
__global__ __launch_bounds__(256, (DMA && MB == 4) ? 2 : 1) void gemm_mfma_kernel(const AT *__restrict__ x, const uint8_t *__restrict__ w,
                                                        AT *__restrict__ y, int M, int N, int K, int xcd_m,
                                                        const int32_t *__restrict__ group_offsets,
                                                        const uint8_t *const *__restrict__ group_weights,
                                                        int n_groups, int max_mtiles, int k_steps,
                                                        float *__restrict__ ws, int tn0, int tn_cnt) {
    using F = Fmt<QT>;
    using V8 = typename Vec8<AT>::type;
    static_assert(MB == 4 || (MB == 8 && DMA), "row tiles of 128 rows, or 256 rows in the DMA form");
    constexpr int MB32 = MB, GM = 32 * MB;            // shadow the 128-row constants of the file
    // x block of a K step: 8 * MB32 pieces of 1 KiB (layout below), double buffered
    __shared__ __attribute__((aligned(16))) uint8_t xs0[8 * MB32 * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t xs1[8 * MB32 * 1024];
    __shared__ float lut[16];
    if constexpr (QT == QT_NF4) {
        if (threadIdx.x < 16) lut[threadIdx.x] = NF4_CODEBOOK[threadIdx.x];
    }

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: scalar address arithmetic
    const int G = K / TILE_COLS;
    const int n_tiles = N / TILE_ROWS;

    // Workgroups are handed to the 8 XCDs round-robin (id % 8) and each XCD has its own L2.  The
    // output tiles are therefore dealt out so that one XCD owns a block of band_m row-tiles by
    // band_n column-tiles: its L2 then only has to hold that band of x (re-read by every
    // column-tile) and sees each weight tile from all its row-tiles at about the same time.
    int m0, tile_n;
    if (group_offsets == nullptr) {
        const int tiles_m = (M + GM - 1) / GM, tiles_n = tn_cnt;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int band_m = (tiles_m + xcd_m - 1) / xcd_m;
        const int xcd_n = 8 / xcd_m;
        const int band_n = (tiles_n + xcd_n - 1) / xcd_n;
        const int tile_m = (xcd % xcd_m) * band_m + slot % band_m;
        tile_n = (xcd / xcd_m) * band_n + slot / band_m;
        if (slot >= band_m * band_n || tile_m >= tiles_m || tile_n >= tiles_n) return;   // whole workgroup leaves
        tile_n += tn0;
        m0 = tile_m * GM;
    } else {
        // Grouped mode (mixture-of-experts): rows group_offsets[e] .. group_offsets[e+1]-1 of x use
        // weight group_weights[e].  The grid is sized on the host from an upper bound of row tiles;
        // every workgroup finds its group by walking the offsets (a handful of scalar loads).
        // Whole row tiles first, then the groups' last, partly filled ones: the short tiles fill the
        // gaps at the end of the launch instead of delaying whole tiles queued behind them.
        int full = 0, part = 0;
        for (int e = 0; e < n_groups; e++) {
            const int rows = group_offsets[e + 1] - group_offsets[e];
            full += rows / GM;
            part += (rows % GM) != 0;
        }
        const int tiles_n = tn_cnt;
        int idx;
        bool want_full = true;
        if ((int)blockIdx.x < full * tiles_n) {
            idx = blockIdx.x % full;
            tile_n = blockIdx.x / full;
        } else {
            const int b = blockIdx.x - full * tiles_n;
            if (b >= part * tiles_n) return;                                        // whole workgroup leaves
            want_full = false;
            idx = b % part;
            tile_n = b / part;
        }
        int e = 0, r0 = 0, r1 = 0;
        for (; e < n_groups; e++) {
            r0 = group_offsets[e];
            r1 = group_offsets[e + 1];
            const int f = (r1 - r0) / GM;
            if (want_full) {
                if (idx < f) break;
                idx -= f;
            } else if ((r1 - r0) % GM) {
                if (idx == 0) { idx = f; break; }
                idx--;
            }
        }
        if (e == n_groups) return;
        m0 = r0 + idx * GM;
        M = r1;                                     // rows past the group's end are clamped / not stored
        w = group_weights[e];
    }
    const int n0 = tile_n * GN + wave * GN_WAVE;

    // weight tiles of this lane: block nb covers rows n0 + 32*nb .. +31 (clamped: a tile row past N
    // is computed and never stored)
    const int kg = lane >> 5, i32 = lane & 31, r16 = lane & 15;
    const int slot_lo = kg * 16 + r16, slot_hi = (kg + 2) * 16 + r16;
    gbytes wt[NB32];
#pragma unroll
    for (int nb = 0; nb < NB32; nb++) {
        int trow = n0 / TILE_ROWS + nb * 2 + (i32 >> 4);
        trow = trow < n_tiles ? trow : n_tiles - 1;
        wt[nb] = (gbytes)w + (int64_t)trow * G * F::TILE_BYTES;
    }

    // The x block of a K step (128 rows x 256 bytes) sits in LDS as 32 pieces of 1 KiB: piece h * 16 + t
    // holds rows 8t .. 8t+7 of the half row h (64 columns = 128 bytes), the 16 bytes of (row r, 16-byte
    // chunk c) at (c * 8 + r % 8) * 16.  Lane (kg, i) of the MFMA reads, for 16-column step ks and row
    // block mb, piece (ks/4) * 16 + 4*mb + i/8 at ((ks%4 * 2 + kg) * 8 + i%8) * 16: eight consecutive
    // lanes read 128 contiguous bytes.  The layout is chosen for the DMA form below.
    //
    // Register-staged form: x goes global -> registers -> LDS; a wave-wide load covers 16 rows x 64
    // bytes: chunk = 4*wave + lane/16 (16 bytes each), row = 16*i + lane%16 for i = 0..7.
    const int chunk = wave * 4 + (lane >> 4);
    uint32_t xoff[DMA ? 1 : 8];
    int xl[DMA ? 1 : 8];
    // DMA form: x goes global -> LDS without passing through registers.  One wave-wide instruction
    // fills one piece: lane 8*c + i fetches the 16 bytes at row 8t + i, byte 16c of the half row - whole
    // 128-byte lines, 8 per instruction - and the hardware writes the lanes to LDS in lane order.  Wave
    // w fills pieces 8w .. 8w+7: half row w/2, rows 64*(w%2) + 8j + i.  Rows past M are clamped (the
    // offsets are formed with 24-bit multiplies: the launcher keeps M and 2K below 2^24).
    uint32_t xrow0 = 0, xcol = 0;
    if constexpr (!DMA) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int row_in = i * 16 + r16;
            int row = m0 + row_in;
            row = row < M ? row : M - 1;
            xoff[i] = (uint32_t)(((int64_t)row * K + chunk * 8) * (int64_t)sizeof(AT));
            xl[i] = (((chunk >> 3) * (4 * MB32) + (row_in >> 3)) * 64 + (chunk & 7) * 8 + (row_in & 7)) * 16;
        }
    } else {
        xrow0 = m0 + (GM / 2) * (wave & 1) + (lane & 7);
        xcol = (wave >> 1) * 128 + (lane >> 3) * 16;
    }
    constexpr int PW = 2 * MB32;                     // pieces of 1 KiB (8 rows of a half row) a wave fetches per K step
    // Split-K: with a workspace the grid has a second dimension, workgroup (t, s) walks the K steps
    // s * k_steps .. and leaves its fp32 partial tile in ws[s]; a second kernel sums the splits.  It
    // fills the machine when the output alone has too few tiles (small M, narrow N).
    const int kt0 = ws ? blockIdx.y * k_steps : 0;
    const int Gs = ws ? (k_steps < G - kt0 ? k_steps : G - kt0) : G;
    const int last = Gs - 1;
    // the same loads one at a time, for spreading them over a step: a burst of 8 + 6 loads per wave,
    // from eight waves at once, queues up at the CU's address unit and the waves stand still meanwhile
    // (measured with cycle counters: 41 % of a K step at M = 2048)
    auto dma_x_one = [&](int kt, uint8_t *buf, int j) {
        kt = kt0 + (kt < last ? kt : last);
        // Issued from inline assembly: the compiler's wait-count pass treats an LDS-DMA as aliasing
        // every later LDS access and would wait for it immediately.  Completion is awaited by the
        // explicit vmcnt(0) ahead of the workgroup barrier that publishes the buffer.
        const uint8_t *xk = (const uint8_t *)x + (int64_t)kt * TILE_COLS * sizeof(AT);
        const uint32_t lbase = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)buf + wave * PW * 1024);
        uint32_t row = xrow0 + 8 * j;
        row = row < (uint32_t)M ? row : (uint32_t)M - 1;
        const uint8_t *src = xk + (__umul24(row, (uint32_t)K * (uint32_t)sizeof(AT)) + xcol);
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :: "v"(src), "s"(lbase + j * 1024) : "memory", "m0");
    };
    // Tall form (whole 256-row tiles only, so no row is clamped): the per-lane part of the address is a
    // constant 32-bit offset and everything that changes from load to load is scalar arithmetic.
    const uint32_t xlane_off = (uint32_t)(lane & 7) * (uint32_t)K * (uint32_t)sizeof(AT) + (uint32_t)(lane >> 3) * 16u;
    const uint64_t xwave_base = (uint64_t)(uintptr_t)x +
        ((uint64_t)(m0 + (GM / 2) * (wave & 1)) * (uint64_t)K + (uint64_t)(wave >> 1) * 64u) * sizeof(AT);
    auto dma_x_scalar = [&](int kt, uint8_t *buf, int j) {
        kt = kt0 + (kt < last ? kt : last);
        const uint64_t src = xwave_base + (uint64_t)kt * (TILE_COLS * sizeof(AT)) + (uint64_t)j * 8u * (uint64_t)K * sizeof(AT);
        const uint32_t lbase = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)buf + (wave * PW + j) * 1024);
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(xlane_off), "s"(src), "s"(lbase) : "memory", "m0");
    };
    auto dma_x = [&](int kt, uint8_t *buf) {
#pragma unroll
        for (int j = 0; j < PW; j++) {
            if constexpr (MB32 == 8) dma_x_scalar(kt, buf, j);
            else dma_x_one(kt, buf, j);
        }
    };
    auto load_x = [&](int kt, u32x4 (&xr)[8]) {
        kt = kt0 + (kt < last ? kt : last);              // past the end: a harmless re-read, never used
        const uint8_t *xk = (const uint8_t *)x + (int64_t)kt * TILE_COLS * sizeof(AT);
#pragma unroll
        for (int i = 0; i < 8; i++) xr[i] = *(const u32x4 *)(xk + xoff[i]);
    };
    auto load_x_one = [&](int kt, u32x4 (&xr)[8], int i) {
        kt = kt0 + (kt < last ? kt : last);
        xr[i] = *(const u32x4 *)((const uint8_t *)x + (int64_t)kt * TILE_COLS * sizeof(AT) + xoff[DMA ? 0 : i]);
    };
    auto store_x = [&](uint8_t *buf, const u32x4 (&xr)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) *(u32x4 *)(buf + xl[i]) = xr[i];
    };
    struct WRegs {
        TileRegs<QT> lo[NB32], hi[NB32];
    };
    auto load_w = [&](int kt, WRegs &t) {
        kt = kt0 + (kt < last ? kt : last);
#pragma unroll
        for (int nb = 0; nb < NB32; nb++) {
            const gbytes tile = wt[nb] + (int64_t)kt * F::TILE_BYTES;
            load_tile<QT>(tile, slot_lo, r16, t.lo[nb]);
            t.hi[nb].q0 = ld<u32x4>(tile + slot_hi * 16);
            if constexpr (F::BITS == 8) t.hi[nb].q1 = ld<u32x4>(tile + 1024 + slot_hi * 16);
        }
    };

    auto load_w_nb = [&](int kt, WRegs &t, int nb) {
        kt = kt0 + (kt < last ? kt : last);
        const gbytes tile = wt[nb] + (int64_t)kt * F::TILE_BYTES;
        load_tile<QT>(tile, slot_lo, r16, t.lo[nb]);
        t.hi[nb].q0 = ld<u32x4>(tile + slot_hi * 16);
        if constexpr (F::BITS == 8) t.hi[nb].q1 = ld<u32x4>(tile + 1024 + slot_hi * 16);
    };

    // The loads of the next K step, as NB32 + PW units (the weight registers of a 32-row block; one piece of x),
    // dealt out over the first five eighths of the step's MFMA groups, so that the data has the rest of the
    // step to arrive and no group carries more than a load or two: a burst stalls the waves at the CU's
    // address unit (41 % of a K step at M = 2048 when all loads of a step went out together), and with one or
    // two waves per SIMD every cycle a wave stands at a memory instruction is a cycle its MFMA pipe idles.
    // `point` = index of the MFMA group (16-column step * row blocks + row block) the call follows.
    auto fetch_units = [&](int kt, uint8_t *buf, WRegs &t, const int point, const int points) {
        constexpr int UNITS = NB32 + PW;
        const int spread = points * 5 / 8 > 0 ? points * 5 / 8 : 1;
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            if (u < point * UNITS / spread || u >= (point + 1) * UNITS / spread || point >= spread) continue;
            if (u < NB32) load_w_nb(kt, t, u);
            else if constexpr (MB32 == 8) dma_x_scalar(kt, buf, u - NB32);
            else dma_x_one(kt, buf, u - NB32);
        }
    };

    f32x16 acc[MB32][NB32];
#pragma unroll
    for (int mb = 0; mb < MB32; mb++)
#pragma unroll
        for (int nb = 0; nb < NB32; nb++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mb][nb][i] = 0.0f;

    const DqCtx ctx = {lut, dq_magic<QT, AT>()};
    // weights of 16-column step ks for block nb: sub-block ks/2, lo or hi registers
    auto dequant_pair = [&](const WRegs &t, int ks, int nb, int p) -> uint32_t {
        if (ks & 1) {
            TileRegs<QT> h = t.hi[nb];
            h.h = t.lo[nb].h;
            return Dequant<QT, AT>::pair(h, ks >> 1, p, ctx);
        }
        return Dequant<QT, AT>::pair(t.lo[nb], ks >> 1, p, ctx);
    };

    // 8 steps of 16 columns, written in the order the hardware should issue them: after the MFMAs
    // of an m-block its x operand for the NEXT step is requested from LDS, and register pairs of
    // the next step's weights are dequantized after every MFMA, so that LDS latency and the VALU
    // work run in the shadow of the MFMA pipe.  MBC = number of 32-row blocks of x that take part
    // (a compile-time constant: a branch around each MFMA would cut the schedule into pieces).
    auto x_piece = [](int ks, int mb) { return ((ks / 4) * 4 * MB32 + 4 * mb) * 1024 + (ks % 4) * 256; };
    const int xlane = (i32 >> 3) * 1024 + kg * 128 + (i32 & 7) * 16;
    auto compute = [&](const uint8_t *cur, const WRegs &t, auto mbc_, auto &&between) {
        constexpr int MBC = decltype(mbc_)::value;
        constexpr int SLOTS = MBC * NB32, PAIRS = 4 * NB32;   // MFMAs per 16-column step; register pairs to dequantize meanwhile
        V8 xv[MBC];
        u32x4 wv[NB32];
#pragma unroll
        for (int mb = 0; mb < MBC; mb++) xv[mb] = *(const V8 *)(cur + xlane + x_piece(0, mb));
#pragma unroll
        for (int nb = 0; nb < NB32; nb++)
#pragma unroll
            for (int p = 0; p < 4; p++) wv[nb][p] = dequant_pair(t, 0, nb, p);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            u32x4 wn[NB32];
#pragma unroll
            for (int mb = 0; mb < MBC; mb++) {
#pragma unroll
                for (int nb = 0; nb < NB32; nb++) {
                    mfma_acc(acc[mb][nb], __builtin_bit_cast(V8, wv[nb]), xv[mb]);
                    if (ks < 7) {
                        // pairs [slot * PAIRS / SLOTS, (slot + 1) * PAIRS / SLOTS): spread evenly over the MFMA slots
                        const int slot_i = mb * NB32 + nb;
#pragma unroll
                        for (int idx = 0; idx < PAIRS; idx++) {
                            if (idx < slot_i * PAIRS / SLOTS || idx >= (slot_i + 1) * PAIRS / SLOTS) continue;
                            wn[idx >> 2][idx & 3] = dequant_pair(t, ks + 1, idx >> 2, idx & 3);   // (weight block, pair)
                        }
                    }
                }
                if (ks < 7) xv[mb] = *(const V8 *)(cur + xlane + x_piece(ks + 1, mb));
                // keep this order: the scheduler does not know how long an MFMA takes and would
                // sink the LDS read down to its first use, exposing the LDS latency every time
                __builtin_amdgcn_sched_barrier(0);
                between(ks * MBC + mb, 8 * MBC);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (ks < 7) {
#pragma unroll
                for (int nb = 0; nb < NB32; nb++) wv[nb] = wn[nb];
            }
        }
    };
    typedef std::integral_constant<int, MB32> full_t;
    auto nothing = [](int, int) {};

    auto epilogue = [&](auto mbc_) {
        constexpr int MBC = decltype(mbc_)::value;
    // The MFMAs above are opaque to the compiler's hazard tracking: give the last results time to
    // land before the accumulation registers are read back (a 16-pass MFMA needs 18 wait states
    // before its result may be read; 64 are spent).  The accumulators are operands of the statement,
    // so that no read of them can be scheduled ahead of it.
#pragma unroll
    for (int mb = 0; mb < MBC; mb++)
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7"
                     : "+a"(acc[mb][0]), "+a"(acc[mb][1]));
    // C layout of the 32x32 block: lane = 32*g + col (col = x row within the block), register i =
    // weight row 8*(i/4) + 4*g + i%4: four consecutive n per group of registers
#pragma unroll
    for (int mb = 0; mb < MBC; mb++) {
        const int m = m0 + mb * 32 + i32;
        if (m < M) {
#pragma unroll
            for (int nb = 0; nb < NB32; nb++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int n = n0 + nb * 32 + q * 8 + kg * 4;
                    if (n < N) {
                        if (ws) {
                            // partial sums keep the register layout (split, tile, wave, register group,
                            // lane): every store is 1 KiB contiguous; the reduction kernel undoes it
                            const f32x4 o = {acc[mb][nb][q * 4], acc[mb][nb][q * 4 + 1], acc[mb][nb][q * 4 + 2],
                                             acc[mb][nb][q * 4 + 3]};
                            const int64_t tile_id = (int64_t)(m0 / GM) * ((N + GN - 1) / GN) + tile_n;
                            const int64_t n_tiles_all = (int64_t)((M + GM - 1) / GM) * ((N + GN - 1) / GN);
                            const int64_t slot = (((int64_t)blockIdx.y * n_tiles_all + tile_id) * 4 + wave) * (MB32 * NB32 * 4) +
                                                 (mb * NB32 + nb) * 4 + q;
                            *(f32x4 *)(ws + (slot * 64 + lane) * 4) = o;
                        } else {
                            typedef AT at4 __attribute__((ext_vector_type(4)));
                            at4 o;
#pragma unroll
                            for (int i = 0; i < 4; i++) o[i] = to_at<AT>(acc[mb][nb][q * 4 + i]);
                            *(at4 *)(y + (int64_t)m * N + n) = o;
                        }
                    }
                }
                // one 32x32 block at a time: moving all 128 accumulators to vector registers at
                // once would set the register footprint of the whole kernel
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    };

    if constexpr (DMA) {
        // One K step ahead: while step kt is computed the x block of step kt+1 streams into the
        // other LDS buffer and its weight tiles into the second register set.  The waits this
        // leaves exposed are covered by the second workgroup that the smaller register footprint
        // lets a CU hold.
        auto run = [&](auto mbc) {
            WRegs w0, w1;
            dma_x(0, xs0);
            load_w(0, w0);
            wait_all_loads();
            __syncthreads();
            for (int kt = 0; kt + 1 < Gs; kt += 2) {
                compute(xs0, w0, mbc, [&](const int point, const int points) {
                    fetch_units(kt + 1, xs1, w1, point, points);
                });
                wait_all_loads();
                __syncthreads();
                compute(xs1, w1, mbc, [&](const int point, const int points) {   // past the end: clamped, unused re-reads
                    fetch_units(kt + 2, xs0, w0, point, points);
                });
                wait_all_loads();
                __syncthreads();
            }
            if (Gs & 1) compute(xs0, w0, mbc, nothing);
        };
        // tail tiles and small expert groups: 32-row blocks without rows of x skip their MFMAs
        const int mb_cnt = (M - m0 + 31) / 32;
        if constexpr (MB32 == 8) {
            // the launcher hands the tall form whole 256-row tiles only
            run(full_t());
            epilogue(full_t());
        } else if (mb_cnt <= 1) {
            run(std::integral_constant<int, 1>());
            epilogue(std::integral_constant<int, 1>());
        } else if (mb_cnt <= 2) {
            run(std::integral_constant<int, 2>());
            epilogue(std::integral_constant<int, 2>());
        } else {
            run(full_t());
            epilogue(full_t());
        }
    } else {
    // Software pipeline, two K steps deep: while step kt is computed, the data of step kt+1 is
    // already in registers (it moves to LDS at the end of step kt) and the loads of step kt+2
    // are issued.  x rotates through two register sets, the weight tiles through three, hence
    // the period of six.
    u32x4 xa[8], xb[8];
    WRegs w0, w1, w2;
    load_x(0, xa);
    load_w(0, w0);
    load_x(1, xb);
    load_w(1, w1);
    store_x(xs0, xa);
    __syncthreads();

#define LOWBIT_GEMM_STEP(i, cur, nxt, xst, xld, wc, wl)                        \
    if (kt + (i) < Gs) {                                                       \
        compute(cur, wc, full_t(), [&](const int point, const int points) {    \
            if (point % MB32 == MB32 - 1) {                                    \
                const int ks = point / MB32;                                   \
                if (ks < 2) load_w_nb(kt + (i) + 2, wl, ks);                   \
                load_x_one(kt + (i) + 2, xld, ks);                             \
            }                                                                  \
        });                                                                    \
        store_x(nxt, xst);                                                     \
        __syncthreads();                                                       \
    }
    for (int kt = 0; kt < Gs; kt += 6) {
        LOWBIT_GEMM_STEP(0, xs0, xs1, xb, xa, w0, w2)
        LOWBIT_GEMM_STEP(1, xs1, xs0, xa, xb, w1, w0)
        LOWBIT_GEMM_STEP(2, xs0, xs1, xb, xa, w2, w1)
        LOWBIT_GEMM_STEP(3, xs1, xs0, xa, xb, w0, w2)
        LOWBIT_GEMM_STEP(4, xs0, xs1, xb, xa, w1, w0)
        LOWBIT_GEMM_STEP(5, xs1, xs0, xa, xb, w2, w1)
    }
#undef LOWBIT_GEMM_STEP
    epilogue(full_t());
    }
}


// Sums the fp32 partial tiles of the splits (stored in the GEMM's register layout: split, tile, wave,
// register group, lane) and writes y, rounded once.  One thread per group of 4 consecutive n.
template <typename AT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ ws, AT *__restrict__ y, int M,
                                                            int N, int splits) {
    const int tiles_n = (N + GN - 1) / GN;
    const int64_t n_tiles_all = (int64_t)((M + GM - 1) / GM) * tiles_n;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;       // (tile, wave, group, lane)
    if (t >= n_tiles_all * 4 * (MB32 * NB32 * 4) * 64) return;
    const int lane = (int)(t & 63);
    const int grp = (int)((t >> 6) % (MB32 * NB32 * 4));
    const int wave = (int)((t >> 6) / (MB32 * NB32 * 4) % 4);
    const int64_t tile_id = (t >> 6) / (MB32 * NB32 * 4) / 4;
    const int mb = grp / (NB32 * 4), nb = grp / 4 % NB32, q = grp % 4;
    const int m = (int)(tile_id / tiles_n) * GM + mb * 32 + (lane & 31);
    const int n = (int)(tile_id % tiles_n) * GN + wave * GN_WAVE + nb * 32 + q * 8 + (lane >> 5) * 4;
    if (m >= M || n >= N) return;
    const int64_t per_split = n_tiles_all * 4 * (MB32 * NB32 * 4) * 64 * 4;     // floats
    f32x4 a = *(const f32x4 *)(ws + t * 4);
    for (int s = 1; s < splits; s++) a += *(const f32x4 *)(ws + (int64_t)s * per_split + t * 4);
    typedef AT at4 __attribute__((ext_vector_type(4)));
    at4 o;
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = to_at<AT>(a[k]);
    *(at4 *)(y + (int64_t)m * N + n) = o;
}

// Estimated run time in microseconds of the GEMM with K split `splits` ways (1 = no split), from
// measurements on MI355X: a workgroup takes about 1.9 us per 128-column step on an otherwise idle
// machine, 2.7 us when every CU holds one workgroup and 5.0 us when every CU holds two (the clock
// drops and the memory system fills as more CUs work); the partial sums of a split are written and
// read back at about 4 TB/s.
double gemm_time_us(int M, int N, int K, int splits) {
    const double tiles = (double)((M + GM - 1) / GM) * (double)((N + GN - 1) / GN);
    const int G = K / TILE_COLS;
    const int k_steps = (G + splits - 1) / splits;
    const int ny = (G + k_steps - 1) / k_steps;
    const double wgs = tiles * ny;
    const double live = wgs < 512.0 ? wgs : 512.0;
    // row tiles that are partly empty skip MFMAs and write fewer partial sums: the load-dependent
    // part of a step and the reduction traffic shrink with the fill, the latency floor does not
    const double fill = (double)M / ((double)((M + GM - 1) / GM) * GM);
    const double load = live <= 256.0 ? 0.8 * live / 256.0 : 0.8 + 2.3 * (live - 256.0) / 256.0;
    const double step = 1.9 + load * (0.4 + 0.6 * fill);
    double t = (double)k_steps * step * (wgs > 512.0 ? wgs / 512.0 : 1.0);
    if (ny > 1) t += (double)ny * tiles * (GM * GN * 8.0) * fill / 4.0e6 + 3.0;
    return t;
}

// Number of K splits to use for this shape given `ws_bytes` of workspace (1 = none): the fastest by
// the estimate above among 1 .. 8 splits of at least two K steps that fit the workspace.
int gemm_splits(int M, int N, int K, size_t ws_bytes) {
    const size_t tiles = (size_t)((M + GM - 1) / GM) * (size_t)((N + GN - 1) / GN);
    const size_t per_split = tiles * GM * GN * sizeof(float);     // whole tiles: partial sums keep the tile layout
    const int G = K / TILE_COLS;
    int best = 1;
    double best_t = gemm_time_us(M, N, K, 1);
    for (int s = 2; s <= 8 && s * 2 <= G; s++) {
        if ((size_t)s * per_split > ws_bytes) break;
        const double t = gemm_time_us(M, N, K, s);
        if (t < 0.9 * best_t) {                                   // a split must pay clearly
            best = s;
            best_t = t;
        }
    }
    return best;
}

// How many column tiles (256 weight rows each) the tall form takes, from the left: whole rounds of one
// 256 x 256 tile per CU, so that no CU sits idle while another still works on a second tall tile; the 128-row
// form covers the columns that are left.  0 = the tall form is not used: M not a multiple of 256, too few
// tiles to fill the machine once, K too long for 24-bit row offsets - or columns left over that would not
// fill the machine themselves.  Measured on MI355X: a machine full of tall tiles runs 4-7 % (sym_int4) to
// 10 % (nf4) faster than the 128-row form with two workgroups per CU, which the idle CUs of a thin remainder
// eat up again ([11008 x 4096] at M = 2048: 32 tall columns + 11 left over, no faster than 688 small tiles).
static int tall_columns(int M, int N, int K, int n_cus) {
    if (M < 2 * GM_TALL || M % GM_TALL || M >= (1 << 24) || K >= (1 << 23)) return 0;
    const int tiles_m = M / GM_TALL, tiles_n = (N + GN - 1) / GN;
    const int rounds = tiles_m * tiles_n / n_cus;
    if (rounds < 1) return 0;
    int cols = rounds * n_cus / tiles_m;
    if (cols >= tiles_n) return tiles_n;
    const int left = (tiles_n - cols) * (M / GM);        // 128-row tiles of the remainder
    return 2 * left >= 3 * n_cus ? cols : 0;
}

template <int QT, typename AT>
static int launch_gemm_t(const void *x, const void *w, void *y, int M, int N, int K, float *ws, int splits,
                         hipStream_t st) {
    if (splits <= 1) ws = nullptr;
    const int G = K / TILE_COLS;
    const int tiles_n_all = (N + GN - 1) / GN;
    static const int n_cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            n = 256;
        return n > 0 ? n : 256;
    }();
    // tall form on the left columns, 128-row form on the rest (both in the same stream, the second starts when
    // the tall tiles, which all take the same time, are done)
    const int tall = ws ? 0 : tall_columns(M, N, K, n_cus);
    if (tall > 0) {
        const int tiles_m = M / GM_TALL;
        int xcd_m = 1;
        while (xcd_m * 2 <= 8 && xcd_m * 2 <= tiles_m) xcd_m *= 2;
        const int xcd_n = 8 / xcd_m;
        const int band_m = (tiles_m + xcd_m - 1) / xcd_m, band_n = (tall + xcd_n - 1) / xcd_n;
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL>), dim3(8 * band_m * band_n), dim3(256), 0, st,
                           (const AT *)x, (const uint8_t *)w, (AT *)y, M, N, K, xcd_m, (const int32_t *)nullptr,
                           (const uint8_t *const *)nullptr, 0, 0, G, (float *)nullptr, 0, tall);
        if (tall == tiles_n_all) return 0;
    }
    const int tn0 = tall, tiles_n = tiles_n_all - tall;
    const int tiles_m = (M + GM - 1) / GM;
    int xcd_m = 1;                                       // XCDs along M: power of two <= min(8, tiles_m)
    while (xcd_m * 2 <= 8 && xcd_m * 2 <= tiles_m) xcd_m *= 2;
    const int xcd_n = 8 / xcd_m;
    const int band_m = (tiles_m + xcd_m - 1) / xcd_m, band_n = (tiles_n + xcd_n - 1) / xcd_n;
    const int k_steps = ws ? (G + splits - 1) / splits : G;
    const int ny = ws ? (G + k_steps - 1) / k_steps : 1;             // splits that actually hold steps
    dim3 grid(8 * band_m * band_n, ny);
    // Two forms of the kernel.  The DMA form (x straight into LDS, one K step of prefetch, 128
    // vector registers) lets a CU hold two workgroups that cover each other's waits; it wins as
    // soon as there are more workgroups than CUs.  With at most one per CU the register-staged
    // form with its deeper prefetch is faster.
    const bool dma = tiles_m * tiles_n * ny > 256 && M < (1 << 24) && K < (1 << 23);   // 24-bit row offsets
    if (dma)
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32>), grid, dim3(256), 0, st, (const AT *)x, (const uint8_t *)w,
                           (AT *)y, M, N, K, xcd_m, (const int32_t *)nullptr, (const uint8_t *const *)nullptr, 0, 0,
                           k_steps, ws, tn0, tiles_n);
    else
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, false, MB32>), grid, dim3(256), 0, st, (const AT *)x, (const uint8_t *)w,
                           (AT *)y, M, N, K, xcd_m, (const int32_t *)nullptr, (const uint8_t *const *)nullptr, 0, 0,
                           k_steps, ws, tn0, tiles_n);
    if (ws) {
        const int64_t threads = (int64_t)tiles_m * tiles_n * (GM * GN / 4);
        hipLaunchKernelGGL((splitk_reduce_kernel<AT>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, ws,
                           (AT *)y, M, N, ny);
    }
    return 0;
}

template <int QT, typename AT>
static int launch_grouped_t(const void *x, const void *const *w, void *y, const int32_t *offsets, int n_groups,
                            int total_rows, int N, int K, hipStream_t st) {
    const int max_mtiles = (total_rows + GM - 1) / GM + n_groups;    // every group adds at most one partial tile
    const int tiles_n = (N + GN - 1) / GN;
    hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32>), dim3(tiles_n * max_mtiles), dim3(256), 0, st, (const AT *)x,
                       (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, offsets, (const uint8_t *const *)w, n_groups,
                       max_mtiles, 0, (float *)nullptr, 0, tiles_n);
    return 0;
}

template <int QT>
static int launch_grouped_q(const void *x, const void *const *w, void *y, const int32_t *offsets, int n_groups,
                            int total_rows, int dt, int N, int K, hipStream_t st) {
    if (dt == DT_F16) return launch_grouped_t<QT, _Float16>(x, w, y, offsets, n_groups, total_rows, N, K, st);
    if (dt == DT_BF16) return launch_grouped_t<QT, __bf16>(x, w, y, offsets, n_groups, total_rows, N, K, st);
    return -4;
}

// Grouped product for mixture-of-experts layers: one launch for all experts.
int launch_grouped_gemm(const void *x, const void *const *w, void *y, const int32_t *offsets, int n_groups,
                        int total_rows, int qtype, int act_dtype, int N, int K, hipStream_t st) {
    if (total_rows == 0 || N == 0 || n_groups == 0) return 0;
    if (total_rows >= (1 << 24) || K >= (1 << 23)) return -3;        // 24-bit row offsets in the kernel
    switch (qtype) {
    case QT_SYM_INT4: return launch_grouped_q<QT_SYM_INT4>(x, w, y, offsets, n_groups, total_rows, act_dtype, N, K, st);
    case QT_ASYM_INT4: return launch_grouped_q<QT_ASYM_INT4>(x, w, y, offsets, n_groups, total_rows, act_dtype, N, K, st);
    case QT_SYM_INT8: return launch_grouped_q<QT_SYM_INT8>(x, w, y, offsets, n_groups, total_rows, act_dtype, N, K, st);
    case QT_NF4: return launch_grouped_q<QT_NF4>(x, w, y, offsets, n_groups, total_rows, act_dtype, N, K, st);
    case QT_FP8_E4M3: return launch_grouped_q<QT_FP8_E4M3>(x, w, y, offsets, n_groups, total_rows, act_dtype, N, K, st);
    default: return -2;
    }
}

template <int QT>
static int launch_gemm_q(const void *x, const void *w, void *y, int dt, int M, int N, int K, float *ws, int splits,
                         hipStream_t st) {
    if (dt == DT_F16) return launch_gemm_t<QT, _Float16>(x, w, y, M, N, K, ws, splits, st);
    if (dt == DT_BF16) return launch_gemm_t<QT, __bf16>(x, w, y, M, N, K, ws, splits, st);
    return -4;
}

// splits: 0 = chosen here from the workspace size, otherwise as given (the caller has checked that it fits)
int launch_gemm(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                void *workspace, size_t workspace_bytes, int want_splits, hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    // the MFMA GEMM reads the tiled layout and stores 8-byte groups of y (N % 4 == 0 is implied
    // by N % 16 == 0); anything else goes through the streaming kernel in 16-row slices
    if (layout != LAYOUT_TILED || (N % TILE_ROWS) || (K % TILE_COLS) || (((uintptr_t)y) & 7))
        return launch_gemv(x, w, y, qtype, layout, act_dtype, M, N, K, 0, st);
    float *ws = (float *)workspace;
    const int splits = !ws ? 1 : want_splits > 0 ? want_splits : gemm_splits(M, N, K, workspace_bytes);
    switch (qtype) {
    case QT_SYM_INT4: return launch_gemm_q<QT_SYM_INT4>(x, w, y, act_dtype, M, N, K, ws, splits, st);
    case QT_ASYM_INT4: return launch_gemm_q<QT_ASYM_INT4>(x, w, y, act_dtype, M, N, K, ws, splits, st);
    case QT_SYM_INT8: return launch_gemm_q<QT_SYM_INT8>(x, w, y, act_dtype, M, N, K, ws, splits, st);
    case QT_NF4: return launch_gemm_q<QT_NF4>(x, w, y, act_dtype, M, N, K, ws, splits, st);
    case QT_FP8_E4M3: return launch_gemm_q<QT_FP8_E4M3>(x, w, y, act_dtype, M, N, K, ws, splits, st);
    default: return -2;
    }
}

}  // namespace lowbit
