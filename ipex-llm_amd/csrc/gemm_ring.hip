// y[M,N] = x[M,K] * dequant(W)[N,K]^T for M of a few dozen to a few hundred rows: a batch of decode
// tokens or a short prompt.
//
// Replaces xe_batch.batch_forward / xe_linear.forward_new at these M
// (python/llm/src/ipex_llm/transformers/low_bit_linear.py:657-668).
//
// At these M the product is bound by streaming the weights once, like the GEMV, but x no longer fits
// a wave's share of LDS, so the work is cut like a GEMM: a workgroup of 8 waves owns 32, 64 or 128
// rows of x by 256 weight rows (32 per wave).  N / 256 tiles are far fewer than CUs, so K is cut
// as well: the list of (tile, 128-column step) units is dealt out in equal contiguous runs, one per
// workgroup, whatever the shape; a run that covers only part of a tile's K leaves an fp32 partial
// tile in a workspace and a second kernel adds the parts.
//
// Both operands of a step - the block of x and the RAW quantized tiles - travel HBM -> LDS by
// LDS-DMA into a ring of stages, ahead of their use.  A wave fetches the weight tiles it consumes
// itself (no barrier needed for them), the block of x is shared (one barrier per step).  The loads
// of a stage are counted, and the wait before a step leaves the loads of the younger stages in
// flight (s_waitcnt vmcnt(n) retires loads in order).
//
// Bytes per launch: N*K*TS/QK of weights + x once per 256 weight rows (from L2) + partial sums.
#include "lowbit_gemm.h"

namespace lowbit {

constexpr int RING_WAVES = 8;  // waves per workgroup; each owns 32 * RNB weight rows (RNB = 1 or 2)

template <int QT> constexpr int ring_hdr_bytes() { return Fmt<QT>::TILE_BYTES - Fmt<QT>::TILE_CODE_BYTES; }
// one stage: the x block as 8 * MB pieces of 1 KiB (see the kernel), the code part of the workgroup's
// 16 tiles, then their header parts
template <int QT> constexpr int ring_stage_bytes(int mb, int rnb) { return mb * 8 * 1024 + 16 * rnb * Fmt<QT>::TILE_BYTES; }
// 32 weight rows per wave (256 per workgroup).  64 rows per wave would let an x operand read from LDS
// feed two MFMAs, but measured 15-60 % slower at every M (sym_int4: [65536 x 4096] at M = 32 / 64 / 128
// 49 / 62 / 109 us against 42 / 54 / 85), with register spills at 128 rows of x.
template <int QT> constexpr int ring_rnb(int mb) { return 1; }
// number of stages: 3, or 2 where 3 do not fit.  A deeper ring measured no faster.
template <int QT> constexpr int ring_stages(int mb) {
    const int fit = (160 * 1024 - 64) / ring_stage_bytes<QT>(mb, ring_rnb<QT>(mb));
    return fit > 3 ? 3 : fit;
}

// s_waitcnt that waits for the vector-memory counter only: vmcnt = n (6 bits, split over the
// immediate), the export and LDS counters left at "no wait"
template <int N> __device__ inline void wait_vm() {
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
    asm volatile("" ::: "memory");
}

// The work of a launch is the list of units u = tile * G + kt (tile = (tile_n, tile_m) pair, kt = 128-
// column step, G = K / 128), dealt out in equal contiguous runs: workgroup b of B takes units
// b*U/B .. (b+1)*U/B - 1.  A run may cross from one tile into the next; each piece of a tile
// ("segment") that does not cover all of K leaves an fp32 partial tile in the workspace, in slot
// b * seg_slots + (tile - first tile of b).
// With q = U / B and r = U % B the first r workgroups take q + 1 units, the others q: no division on the
// device beyond 32-bit ones.
__host__ __device__ inline int ring_first_unit(int b, int q, int r) { return b * q + (b < r ? b : r); }
__host__ __device__ inline int ring_owner(int u, int q, int r) {
    const int big = r * (q + 1);                     // units held by the workgroups with q + 1
    return u < big ? u / (q + 1) : r + (u - big) / q;
}

// MB = 32-row blocks of x per workgroup, RNB = 32-row weight blocks per wave, S = ring stages
template <int QT, typename AT, int MB, int RNB, int S>
__global__ __launch_bounds__(64 * RING_WAVES, 1) void gemm_ring_kernel(const AT *__restrict__ x, const uint8_t *__restrict__ w,
                                                                  AT *__restrict__ y, int M, int N, int K, int seg_slots,
                                                                  int run_q, int run_r, float *__restrict__ ws) {
    using F = Fmt<QT>;
    using V8 = typename Vec8<AT>::type;
    constexpr int WAVES = RING_WAVES, NT = 2 * RNB * WAVES, RN = 16 * NT;   // tiles and weight rows per workgroup
    constexpr int XB = MB * 8 * 1024, CODE = F::TILE_CODE_BYTES, HDR = ring_hdr_bytes<QT>();
    constexpr int STAGE = ring_stage_bytes<QT>(MB, RNB);
    constexpr int CPT = CODE / 1024;                 // 1 KiB code loads per tile
    constexpr int TPI = 256 / HDR;                   // tiles whose headers one 256-byte load covers
    static_assert(TPI >= 1 && TPI <= 4, "header load shape");
    constexpr int TPW = NT / WAVES;                  // tiles per wave
    constexpr int XL = 8 * MB / WAVES;               // loads per stage and wave: x blocks,
    constexpr int CL = TPW * CPT;                    //   code KiBs,
    constexpr int HL = TPW / TPI > 0 ? TPW / TPI : 1;   // header loads (a wave with fewer tiles than a load covers repeats its neighbour's)
    constexpr int L = XL + CL + HL;
    static_assert((S - 2) * L < 64, "too many loads in flight for vmcnt");
    static_assert(S >= 2 && S <= 6, "ring depth");
    extern __shared__ __attribute__((aligned(16))) uint8_t ring[];
    float *lut = (float *)(ring + S * STAGE);        // nf4 code book, behind the ring
    if constexpr (QT == QT_NF4) {
        if (threadIdx.x < 16) lut[threadIdx.x] = NF4_CODEBOOK[threadIdx.x];
        __syncthreads();
    }

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: LDS-DMA targets are scalars
    const int G = K / TILE_COLS;
    const int n_tiles = N / TILE_ROWS;
    const int tiles_m = (M + 32 * MB - 1) / (32 * MB);
    const int kg = lane >> 5, i32 = lane & 31, r16 = lane & 15;
    const int slot_lo = kg * 16 + r16, slot_hi = (kg + 2) * 16 + r16;

    const int u0 = ring_first_unit(blockIdx.x, run_q, run_r), u1 = ring_first_unit(blockIdx.x + 1, run_q, run_r);
    const int n_units = u1 - u0;
    const int first_tile = u0 / G;

    // ---- sources of this lane's share of a stage, for the tile being fetched
    // x: one load moves 8 rows x 128 bytes (64 columns) - whole cache lines - into one 1 KiB piece of
    // LDS, lane l at byte 16 l of it.  Eight consecutive lanes fetch the eight 16-byte chunks of one row (one
    // cache line; with the lanes running across rows the loads are 3.6 times slower): lane l = 8*s + c'
    // fetches row 8*t + (s ^ t%2), chunk c' ^ (s ^ t%2) of the half row h.  Piece q = h * 4*MB + t; wave v
    // fills pieces v*XL .. .  The 16 bytes that lane (kg, i) of the MFMA wants for 16-column step ks and row i
    // of a 32-row block sit in piece (ks/4) * 4*MB + 4*mb + i/8 at ((i%8 ^ i/8 % 2) * 8 + ((ks%4 * 2 + kg) ^ i%8)) * 16:
    // the two xors spread the eight rows of a piece, 128 bytes apart, and the pieces, 1 KiB apart, over the LDS
    // banks, so that every 16 lanes of a wave-wide read cover all banks once.
    // weights: wave v owns tiles v*TPW .. of the workgroup's NT (tile rows past N are clamped: they are
    // computed and never stored).  Codes: lane l fetches bytes 16l .. of the tile (and of its second
    // KiB for 8-bit codes).  Headers: one 4-byte load per lane, 256 bytes per instruction, which is
    // the header part of TPI tiles.
    gbytes xsrc[XL], csrc[TPW], hsrc[HL];
    constexpr int HFIRST_NUM = NT / TPI;             // header loads per stage and workgroup
    const int hfirst = wave * HFIRST_NUM / WAVES;    // index of this wave's first header load
    auto set_tile = [&](int tile) {
        const int tile_m = tile % tiles_m, tile_n = tile / tiles_m;
#pragma unroll
        for (int j = 0; j < XL; j++) {
            const int q = wave * XL + j, h = q / (4 * MB), t = q % (4 * MB);
            const int r = (lane >> 3) ^ (t & 1);
            int row = tile_m * 32 * MB + t * 8 + r;
            row = row < M ? row : M - 1;
            xsrc[j] = (gbytes)x + ((int64_t)row * K + h * 64 + ((lane & 7) ^ r) * 8) * (int64_t)sizeof(AT);
        }
#pragma unroll
        for (int i = 0; i < TPW; i++) {
            int trow = tile_n * NT + wave * TPW + i;
            trow = trow < n_tiles ? trow : n_tiles - 1;
            csrc[i] = (gbytes)w + (int64_t)trow * G * F::TILE_BYTES + lane * 16;
        }
#pragma unroll
        for (int i = 0; i < HL; i++) {
            constexpr int LPT = 64 / TPI;            // lanes per tile
            int trow = tile_n * NT + (hfirst + i) * TPI + lane / LPT;
            trow = trow < n_tiles ? trow : n_tiles - 1;
            hsrc[i] = (gbytes)w + (int64_t)trow * G * F::TILE_BYTES + CODE + (lane % LPT) * 4;
        }
    };
    const uint32_t ring_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)ring;

    // Issued from inline assembly: the compiler neither counts these loads nor orders LDS accesses
    // against them; completion is awaited by the explicit vmcnt waits below.
    auto dma16 = [&](gbytes src, uint32_t lds) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
    };
    auto dma4 = [&](gbytes src, uint32_t lds) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
    };
    // load j of the L loads of a stage (x blocks first, then code KiBs, then headers); `first` .. `last`
    // selects a part of them, so that the loads of a stage can be spread over a step
    auto issue_part = [&](int kt, int slot, const int FIRST, const int LAST) {   // constants once unrolled
        const uint32_t base = __builtin_amdgcn_readfirstlane(ring_base + slot * STAGE);
        const int64_t xk = (int64_t)kt * TILE_COLS * sizeof(AT), wk = (int64_t)kt * F::TILE_BYTES;
#pragma unroll
        for (int j = 0; j < XL; j++) {
            if (j < FIRST || j >= LAST) continue;
            dma16(xsrc[j] + xk, base + (wave * XL + j) * 1024);
        }
#pragma unroll
        for (int i = 0; i < TPW; i++)
#pragma unroll
            for (int c = 0; c < CPT; c++) {
                if (XL + i * CPT + c < FIRST || XL + i * CPT + c >= LAST) continue;
                dma16(csrc[i] + wk + c * 1024, base + XB + (wave * TPW + i) * CODE + c * 1024);
            }
#pragma unroll
        for (int i = 0; i < HL; i++) {
            if (XL + CL + i < FIRST || XL + CL + i >= LAST) continue;
            dma4(hsrc[i] + wk, base + XB + NT * CODE + (hfirst + i) * 256);
        }
    };
    auto issue = [&](int kt, int slot) {             // exactly L loads
        issue_part(kt, slot, 0, L);
    };

    struct WRegs {
        TileRegs<QT> lo[RNB], hi[RNB];
    };
    // this lane's registers of a stage: block nb = tiles TPW*v + 2nb (rows 0-15) and TPW*v + 2nb + 1
    auto read_w = [&](int slot, WRegs &t) {
        const uint8_t *st = ring + slot * STAGE + XB;
#pragma unroll
        for (int nb = 0; nb < RNB; nb++) {
            const int ti = wave * TPW + nb * 2 + (i32 >> 4);
            const uint8_t *codes = st + ti * CODE;
            const uint8_t *hdr = st + NT * CODE + ti * HDR;
            t.lo[nb].q0 = *(const u32x4 *)(codes + slot_lo * 16);
            t.hi[nb].q0 = *(const u32x4 *)(codes + slot_hi * 16);
            if constexpr (F::BITS == 8) {
                t.lo[nb].q1 = *(const u32x4 *)(codes + 1024 + slot_lo * 16);
                t.hi[nb].q1 = *(const u32x4 *)(codes + 1024 + slot_hi * 16);
            }
            if constexpr (QT == QT_SYM_INT4 || QT == QT_SYM_INT8) {
                const u32x2 h = *(const u32x2 *)(hdr + r16 * 8);
                t.lo[nb].h[0] = h[0]; t.lo[nb].h[1] = h[1];
            } else if constexpr (QT == QT_ASYM_INT4) {
                t.lo[nb].h = *(const u32x4 *)(hdr + r16 * 16);
            } else {
                t.lo[nb].h[0] = *(const uint32_t *)(hdr + r16 * 4);
            }
        }
    };

    f32x16 acc[MB][RNB];
    auto clear_acc = [&]() {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int nb = 0; nb < RNB; nb++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[mb][nb][i] = 0.0f;
    };
    clear_acc();

    const DqCtx ctx = {lut, dq_magic<QT, AT>()};
    auto dequant_pair = [&](const WRegs &t, int ks, int nb, int p) -> uint32_t {
        if (ks & 1) {
            TileRegs<QT> h = t.hi[nb];
            h.h = t.lo[nb].h;
            return Dequant<QT, AT>::pair(h, ks >> 1, p, ctx);
        }
        return Dequant<QT, AT>::pair(t.lo[nb], ks >> 1, p, ctx);
    };

    // 8 steps of 16 columns in issue order: the x operand of the next step is requested from LDS
    // right after the MFMAs that used the current one, and the next step's weights are dequantized
    // pair by pair between the MFMAs.
    // The MFMAs are opaque to the compiler: should it ever copy accumulators between registers around
    // a step, the copies must not run into an MFMA still in flight (an 8-pass MFMA needs 11 wait
    // states before its result may be read).  All accumulators are operands, so that such copies
    // cannot be scheduled across the statement.
    auto acc_guard = [&]() {
        if constexpr (MB * RNB == 1) asm volatile("s_nop 7\n\ts_nop 4" : "+a"(acc[0][0]));
        else if constexpr (MB * RNB == 2) asm volatile("s_nop 7\n\ts_nop 4" : "+a"(acc[0][0]), "+a"(acc[MB - 1][RNB - 1]));
        else if constexpr (MB * RNB == 4)
            asm volatile("s_nop 7\n\ts_nop 4" : "+a"(acc[0][0]), "+a"(acc[(1 / RNB) % MB][1 % RNB]), "+a"(acc[2 / RNB][2 % RNB]),
                         "+a"(acc[3 / RNB][3 % RNB]));
        else
            asm volatile("s_nop 7\n\ts_nop 4" : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[1][0]), "+a"(acc[1][1]),
                         "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[3][0]), "+a"(acc[3][1]));
    };
    // where the x operand of (16-column step ks, row block mb) starts, and this lane's place in it
    auto x_piece = [](int ks, int mb) { return ((ks / 4) * 4 * MB + 4 * mb) * 1024; };
    int xlane[4];                                    // by ks % 4
#pragma unroll
    for (int t = 0; t < 4; t++)
        xlane[t] = (i32 >> 3) * 1024 + (((i32 & 7) ^ ((i32 >> 3) & 1)) * 8 + ((2 * t + kg) ^ (i32 & 7))) * 16;
    auto compute = [&](const uint8_t *cur, const WRegs &t, bool fetch, int f_slot, int f_kt_now) {
        constexpr int PER = 4 / MB;                  // dequantized pairs per MFMA slot
        V8 xv[2][MB];                                // x operands of this 16-column step and the next
        u32x4 wv[RNB];
#pragma unroll
        for (int k = 0; k < 2; k++)
#pragma unroll
            for (int mb = 0; mb < MB; mb++) xv[k][mb] = *(const V8 *)(cur + xlane[k] + x_piece(k, mb));
#pragma unroll
        for (int nb = 0; nb < RNB; nb++)
#pragma unroll
            for (int p = 0; p < 4; p++) wv[nb][p] = dequant_pair(t, 0, nb, p);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            u32x4 wn[RNB];
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
#pragma unroll
                for (int nb = 0; nb < RNB; nb++) {
                    mfma_acc(acc[mb][nb], __builtin_bit_cast(V8, wv[nb]), xv[ks & 1][mb]);
                    if (ks < 7) {
#pragma unroll
                        for (int q = 0; q < PER; q++) {
                            const int idx = (mb * RNB + nb) * PER + q;
                            wn[idx >> 2][idx & 3] = dequant_pair(t, ks + 1, idx >> 2, idx & 3);
                        }
                    }
                }
                // two steps ahead: one MFMA slot is shorter than the LDS latency when MB is small
                if (ks < 6) xv[ks & 1][mb] = *(const V8 *)(cur + xlane[(ks + 2) % 4] + x_piece(ks + 2, mb));
                __builtin_amdgcn_sched_barrier(0);
            }
            if (ks < 7) {
#pragma unroll
                for (int nb = 0; nb < RNB; nb++) wv[nb] = wn[nb];
            }
            // The loads of the stage S - 1 steps ahead go out a few at a time between the 16-column
            // steps: issued in one burst after the barrier, the eight waves queue up at the address
            // unit and stand still for about a third of the step.
            if (fetch) {
                if ((ks * L) / 8 != ((ks + 1) * L) / 8) issue_part(f_kt_now, f_slot, (ks * L) / 8, ((ks + 1) * L) / 8);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        acc_guard();
    };

    // Writes the finished segment of `tile`: straight to y when it covers all of K, else as a partial
    // tile.  C layout of a 32x32 block: lane = 32*g + column (= row of x), register i = weight row
    // 8*(i/4) + 4*g + i%4.
    auto store_segment = [&](int tile, bool whole) {
        // The MFMAs are opaque to the compiler's hazard tracking: the accumulators are operands of
        // the wait statement so that no read of them can be scheduled ahead of it.
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int nb = 0; nb < RNB; nb++)
                asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7" : "+a"(acc[mb][nb]));
        const int m0 = (tile % tiles_m) * 32 * MB, n0 = (tile / tiles_m) * RN + wave * (32 * RNB);
        // partial sums keep the register layout (slot, wave, register group, lane): every store
        // instruction writes 1 KiB contiguous
        float *part = ws + ((int64_t)blockIdx.x * seg_slots + (tile - first_tile)) * (32 * MB * RN);
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            const int m = m0 + mb * 32 + i32;
            if (m < M) {
#pragma unroll
                for (int nb = 0; nb < RNB; nb++) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int n = n0 + nb * 32 + q * 8 + kg * 4;
                        if (n < N) {
                            if (!whole) {
                                const f32x4 o = {acc[mb][nb][q * 4], acc[mb][nb][q * 4 + 1], acc[mb][nb][q * 4 + 2],
                                                 acc[mb][nb][q * 4 + 3]};
                                const int grp = (mb * RNB + nb) * 4 + q;
                                *(f32x4 *)(part + ((wave * (MB * RNB * 4) + grp) * 64 + lane) * 4) = o;
                            } else {
                                typedef AT at4 __attribute__((ext_vector_type(4)));
                                at4 o;
#pragma unroll
                                for (int i = 0; i < 4; i++) o[i] = to_at<AT>(acc[mb][nb][q * 4 + i]);
                                *(at4 *)(y + (int64_t)m * N + n) = o;
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    // ---- the ring.  The i-th unit of this workgroup lives in slot i % S.  Before unit i is used, the
    // units i+1 .. min(n, i+S-1)-1 may still be in flight; everything older has to have landed.
    auto wait_for = [&](int younger) {              // number of whole stages that may stay in flight
        switch (younger) {
        case 0: wait_vm<0>(); break;
        case 1: wait_vm<(S > 2 ? 1 : 0) * L>(); break;
        case 2: wait_vm<(S > 3 ? 2 : 0) * L>(); break;
        case 3: wait_vm<(S > 4 ? 3 : 0) * L>(); break;
        default: wait_vm<(S > 5 ? 4 : 0) * L>(); break;
        }
    };
    int f_tile = first_tile, f_kt = u0 - first_tile * G;      // fetch position
    set_tile(f_tile);
    auto fetched = [&]() {                           // the fetch position moves on by one unit
        if (++f_kt == G) {
            f_kt = 0;
            f_tile++;
            set_tile(f_tile);                        // one tile past the end at worst: clamped, never fetched
        }
    };
#pragma unroll
    for (int s = 0; s < S - 1; s++)
        if (s < n_units) {
            issue(f_kt, s);
            fetched();
        }
    int slot = 0, fill = S - 1;                      // slot of the current unit / of the next one to fill
    int c_tile = first_tile, c_kt = u0 - first_tile * G;
    WRegs wr;
    // one pass of the outer loop per segment, so that the accumulators are loop-carried by the inner
    // loop only and stay where the MFMAs want them
    for (int i = 0; i < n_units;) {
        const int seg_len = n_units - i < G - c_kt ? n_units - i : G - c_kt;
        const int seg_end = i + seg_len;
        clear_acc();
        for (; i < seg_end; i++) {
            const int issued = n_units < i + S - 1 ? n_units : i + S - 1;
            wait_for(issued - i - 1);
            // every wave's part of x for this stage has landed, and every wave is done with the
            // previous stage, whose slot is the one refilled next
            __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0): this wave's LDS reads of the previous stage are done
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const bool fetch = i + S - 1 < n_units;
            read_w(slot, wr);
            compute(ring + slot * STAGE, wr, fetch, fill, f_kt);
            if (fetch) fetched();
            slot = slot + 1 == S ? 0 : slot + 1;
            fill = fill + 1 == S ? 0 : fill + 1;
        }
        store_segment(c_tile, seg_len == G);
        c_tile++;
        c_kt = 0;
    }
}

// Sums the partial tiles of every output tile that was cut into segments and writes y, rounded once.
// Grid (tiles, pieces of 256 threads): the tile, and with it the list of workgroups that hold a part of
// it, is the same for a whole workgroup (scalar arithmetic).  One thread per group of 4 consecutive n,
// in the order the partial sums were stored.
template <typename AT, int MB, int RNB>
__global__ __launch_bounds__(256) void ring_reduce_kernel(const float *__restrict__ ws, AT *__restrict__ y, int M, int N,
                                                          int G, int run_q, int run_r, int seg_slots) {
    constexpr int WAVES = RING_WAVES, GRP = MB * RNB * 4, RN = 32 * RNB * WAVES;
    const int tile = blockIdx.x;
    const int b0 = ring_owner(tile * G, run_q, run_r), b1 = ring_owner((tile + 1) * G - 1, run_q, run_r);
    if (b0 == b1) return;                            // one segment covered all of K and wrote y itself
    const int t = blockIdx.y * 256 + threadIdx.x;    // (wave, group, lane)
    const int lane = t & 63;
    const int grp = (t >> 6) % GRP;
    const int wave = (t >> 6) / GRP;
    const int tiles_m = (M + 32 * MB - 1) / (32 * MB);
    const int mb = grp / (RNB * 4), nb = grp / 4 % RNB, q = grp % 4;
    const int m = (tile % tiles_m) * 32 * MB + mb * 32 + (lane & 31);
    const int n = (tile / tiles_m) * RN + wave * (32 * RNB) + nb * 32 + q * 8 + (lane >> 5) * 4;
    if (m >= M || n >= N) return;
    // eight parts in flight at a time (a thread that waited for each part in turn would spend a memory
    // latency per part); they are added in workgroup order whatever their number
    f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = b0; c <= b1; c += 8) {
        f32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int b = c + j <= b1 ? c + j : b1;
            const int seg = tile - ring_first_unit(b, run_q, run_r) / G;
            const float *part = ws + ((int64_t)b * seg_slots + seg) * (32 * MB * RN);
            v[j] = *(const f32x4 *)(part + (int64_t)t * 4);
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (c + j <= b1) a += v[j];
    }
    typedef AT at4 __attribute__((ext_vector_type(4)));
    at4 o;
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = to_at<AT>(a[k]);
    *(at4 *)(y + (int64_t)m * N + n) = o;
}

struct RingPlan {
    int mb, rnb, tiles, B, seg_slots;
    size_t ws_bytes;
};

static int ring_rnb_of(int qtype, int mb) {
    switch (qtype) {
    case QT_SYM_INT4: return ring_rnb<QT_SYM_INT4>(mb);
    case QT_ASYM_INT4: return ring_rnb<QT_ASYM_INT4>(mb);
    case QT_SYM_INT8: return ring_rnb<QT_SYM_INT8>(mb);
    case QT_NF4: return ring_rnb<QT_NF4>(mb);
    default: return ring_rnb<QT_FP8_E4M3>(mb);
    }
}

// wgs = number of workgroups to deal the units to; 0 = one per CU, but at least four units each (the
// fixed cost of a workgroup and its partial tile are not worth less).  Without a workspace every
// workgroup takes whole tiles.
static RingPlan ring_plan(int M, int N, int K, int rnb, int wgs, bool have_ws) {
    RingPlan p;
    p.mb = M <= 32 ? 1 : M <= 64 ? 2 : 4;
    p.rnb = rnb;
    const int rn = 32 * rnb * RING_WAVES;
    p.tiles = ((M + 32 * p.mb - 1) / (32 * p.mb)) * ((N + rn - 1) / rn);
    const int G = K / TILE_COLS;
    const int64_t U = (int64_t)p.tiles * G;
    int64_t B = wgs > 0 ? wgs : (U / 4 < 256 ? U / 4 : 256);
    if (B > U) B = U;
    if (B < 1) B = 1;
    if (!have_ws) B = p.tiles;
    p.B = (int)B;
    // a run of ceil(U/B) units touches at most this many tiles
    const int64_t run = (U + B - 1) / B;
    p.seg_slots = (int)((run + G - 2) / G) + 1;
    p.ws_bytes = (U % B == 0 && (U / B) % G == 0) ? 0 : (size_t)B * p.seg_slots * (32 * p.mb) * rn * sizeof(float);
    return p;
}

// Estimated run time in microseconds, fitted to measurements on MI355X (40 weight shapes in all five formats,
// M = 17 .. 256, nf4 to 768; 7.5 % rms): a fixed part (launch, first loads, partial tiles and their reduction) plus
// the steps of the longest run; 8-bit codes and nf4 take 15 - 30 % longer per step, and steps are shorter on a
// machine that is not full.  The whole is scaled by 0.95: against the estimates of the other kernels that picks
// the fastest one most often.
double ring_time_us(int M, int N, int K, int qtype, bool have_ws) {
    const int mb = M <= 32 ? 1 : M <= 64 ? 2 : 4;
    const RingPlan p = ring_plan(M, N, K, ring_rnb_of(qtype, mb), 0, have_ws);
    static const double fixed[3] = {9.2, 11.8, 16.4}, step[3] = {1.22, 1.45, 1.99};
    const int i = p.mb == 1 ? 0 : p.mb == 2 ? 1 : 2;
    const int64_t U = (int64_t)p.tiles * (K / TILE_COLS);
    const double run = (double)((U + p.B - 1) / p.B) * p.rnb;          // in steps of 256 weight rows
    const double format = qtype == QT_SYM_INT8 ? 1.30 : qtype == QT_FP8_E4M3 ? 1.15 : qtype == QT_NF4 ? 1.26 : 1.0;
    const double busy = p.B >= 256 ? 1.0 : 0.13 + 0.87 * p.B / 256.0;
    return 0.95 * (fixed[i] - (p.ws_bytes ? 0.0 : 4.5) + run * step[i] * format * busy);
}

// every format runs 32 weight rows per wave (ring_rnb), so one plan covers them all
size_t ring_workspace_bytes(int M, int N, int K, int wgs) {
    return ring_plan(M, N, K, 1, wgs, true).ws_bytes;
}

template <int QT, typename AT, int MB, int RNB>
static int launch_ring_m(const void *x, const void *w, void *y, int M, int N, int K, float *ws, const RingPlan &p,
                         hipStream_t st) {
    constexpr int S = ring_stages<QT>(MB);
    constexpr int LDS = S * ring_stage_bytes<QT>(MB, RNB) + 64;
    auto kern = gemm_ring_kernel<QT, AT, MB, RNB, S>;
    // the default limit of dynamic LDS is 64 KB; raised once per process (thread-safe static), on the one GPU
    // this library drives
    static const hipError_t raised =
        hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (raised != hipSuccess) return -6;
    const int64_t U = (int64_t)p.tiles * (K / TILE_COLS);
    if (U >= (int64_t)1 << 31) return -3;
    const int run_q = (int)(U / p.B), run_r = (int)(U % p.B);
    hipLaunchKernelGGL(kern, dim3(p.B), dim3(64 * RING_WAVES), LDS, st, (const AT *)x, (const uint8_t *)w, (AT *)y, M, N, K,
                       p.seg_slots, run_q, run_r, ws);
    if (p.ws_bytes) {
        constexpr int per_tile = (32 * MB) * (32 * RNB * RING_WAVES) / 4;     // threads: a multiple of 256
        hipLaunchKernelGGL((ring_reduce_kernel<AT, MB, RNB>), dim3(p.tiles, per_tile / 256), dim3(256), 0, st, ws, (AT *)y,
                           M, N, K / TILE_COLS, run_q, run_r, p.seg_slots);
    }
    return 0;
}

template <int QT, typename AT>
static int launch_ring_t(const void *x, const void *w, void *y, int M, int N, int K, float *ws, const RingPlan &p,
                         hipStream_t st) {
    if (p.mb == 1) return launch_ring_m<QT, AT, 1, ring_rnb<QT>(1)>(x, w, y, M, N, K, ws, p, st);
    if (p.mb == 2) return launch_ring_m<QT, AT, 2, ring_rnb<QT>(2)>(x, w, y, M, N, K, ws, p, st);
    return launch_ring_m<QT, AT, 4, ring_rnb<QT>(4)>(x, w, y, M, N, K, ws, p, st);
}

template <int QT>
static int launch_ring_q(const void *x, const void *w, void *y, int dt, int M, int N, int K, float *ws, const RingPlan &p,
                         hipStream_t st) {
    if (dt == DT_F16) return launch_ring_t<QT, _Float16>(x, w, y, M, N, K, ws, p, st);
    if (dt == DT_BF16) return launch_ring_t<QT, __bf16>(x, w, y, M, N, K, ws, p, st);
    return -4;
}

// Tiled layout only; the caller has checked the shape and the alignment of y (8 bytes).  A workspace
// smaller than ring_workspace_bytes() for the same `wgs` is not used: the tiles are then not cut.
int launch_gemm_ring(const void *x, const void *w, void *y, int qtype, int act_dtype, int M, int N, int K,
                     void *workspace, size_t workspace_bytes, int wgs, hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    const int rnb = ring_rnb_of(qtype, M <= 32 ? 1 : M <= 64 ? 2 : 4);
    RingPlan p = ring_plan(M, N, K, rnb, wgs, workspace != nullptr);
    if (p.ws_bytes > workspace_bytes) p = ring_plan(M, N, K, rnb, wgs, false);
    float *ws = (float *)workspace;
    switch (qtype) {
    case QT_SYM_INT4: return launch_ring_q<QT_SYM_INT4>(x, w, y, act_dtype, M, N, K, ws, p, st);
    case QT_ASYM_INT4: return launch_ring_q<QT_ASYM_INT4>(x, w, y, act_dtype, M, N, K, ws, p, st);
    case QT_SYM_INT8: return launch_ring_q<QT_SYM_INT8>(x, w, y, act_dtype, M, N, K, ws, p, st);
    case QT_NF4: return launch_ring_q<QT_NF4>(x, w, y, act_dtype, M, N, K, ws, p, st);
    case QT_FP8_E4M3: return launch_ring_q<QT_FP8_E4M3>(x, w, y, act_dtype, M, N, K, ws, p, st);
    default: return -2;
    }
}

}  // namespace lowbit
