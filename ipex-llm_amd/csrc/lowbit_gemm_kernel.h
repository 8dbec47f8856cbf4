// The tiled MFMA GEMM kernel, shared by the dense launchers (gemm.hip) and the grouped ones for
// mixture-of-experts layers (gemm_grouped.hip).
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
#pragma once
#include "lowbit_gemm.h"
#include "lowbit_grouped_plan.h"

namespace lowbit {

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
// WAVES = 8 (tall form only): the same tile with eight waves of 32 weight rows, two per SIMD, 128
// accumulation registers each; every x operand read from LDS then feeds one MFMA instead of two.  The two waves
// of a SIMD cover each other's dequantization, LDS reads and barrier waits, which a partly filled grouped tile
// (a few 32-row blocks of x: few MFMAs per weight) cannot cover with its own MFMAs.
// Grouped mode (mixture-of-experts): rows offsets[e] .. offsets[e+1]-1 of x use the weight w[e]
// (and w_up[e] in the fused gate/up form); all pointers are device memory.
// The fused gate/up form also runs a dense gated MLP - one group that holds all M rows - without any table in
// device memory: offsets == nullptr, the gate weight is the kernel's own `w` argument, the up weight w_up_one.
struct GroupArgs {
    const int32_t *offsets;
    const uint8_t *const *w;
    const uint8_t *const *w_up;
    int n_groups;
    int act;                      // activation of the gate branch in the fused form: 0 = SiLU, 1 = tanh-GELU
    int split_tail;               // dense 128-row DMA form: the last split_tail tiles of every XCD's share go out as two
                                  // half tiles of 64 rows each, to one workgroup apiece
    int chunk;                    // grouped: column tiles per cell of the tile order (see grouped_tile)
    const uint8_t *w_up_one;      // fused form without tables (offsets == nullptr): the up weight
};

// Which row tile of which group, and which column tile, workgroup `b` of a grouped launch works on.
//
// The row tiles of all groups form one list: whole row tiles first, then the groups' last, partly filled ones
// (short tiles then fill the end of the launch instead of delaying whole tiles queued behind them).  Each row tile
// times `chunk` consecutive column tiles is a cell; the cells, row tile by row tile, are dealt to the 8 XCDs in turn
// (workgroups go to the XCDs round-robin: XCD = b % 8), and an XCD walks its cells in order, so that
//   - the workgroups an XCD runs at the same time belong to few row tiles: their rows of x stay in that XCD's L2
//     (with the column tiles of a row tile spread over all XCDs instead, every XCD read all of x over and over:
//     the fused gate/up launch of eight groups of 128 rows fetched 1.43 times its weights, and a K step waited
//     for x to arrive from beyond L2);
//   - with chunk = ceil(tiles_n / 8) every XCD gets one cell of every row tile: equal shares however uneven the
//     groups are (a group per XCD was 9-12 % slower with 10 to 300 rows per group);
//   - with chunk = tiles_n a row tile is one cell: all its column tiles on one XCD, for launches of a single round,
//     where shares do not matter.
// Workgroups beyond an XCD's last cell leave at once; they are the last of that XCD's sequence (workgroups go to
// the compute units of an XCD in turn: idle ones between working ones leave units idle).
struct GroupTile {
    int group, m0, m_end, tile_n;
};
// The walk over the cells, shared by both ways of finding the row tile: which cell of which row tile workgroup b has,
// as (index of the row tile in the list, column tile); false when the XCD has no cell left for it.
__device__ inline bool grouped_cell(int row_tiles, int tiles_n, int chunk, int b, int &idx, int &tile_n) {
    const int cells_per_row_tile = (tiles_n + chunk - 1) / chunk, cells = row_tiles * cells_per_row_tile;
    int i = b >> 3, ci = b & 7, q = 0;
    for (;; ci += 8) {                                   // this XCD's cells, in order
        if (ci >= cells) return false;
        q = ci % cells_per_row_tile;
        const int size = tiles_n - q * chunk < chunk ? tiles_n - q * chunk : chunk;
        if (i < size) break;
        i -= size;
    }
    tile_n = q * chunk + i;
    idx = ci / cells_per_row_tile;
    return true;
}
// Up to 64 groups: lane e of the wave holds group e's offsets (two loads per lane, all in flight at once), the
// counts come from a prefix sum over the lanes and the group from a ballot.  Walking the offsets one scalar load
// after the other, twice, makes every load wait for the one before, at the head of every workgroup: the fused
// gate/up launch of 64 groups x [1408 x 2048] with 6144 rows took 158 us that way and takes 125 us this way
// (60 groups, 2048 rows: 114 -> 87; 8 groups: no difference).  Every wave of the workgroup calls this with all
// lanes active.
template <int ROWS>
__device__ inline bool grouped_tile_lanes(const int32_t *__restrict__ offsets, int n_groups, int tiles_n, int chunk, int b,
                                          GroupTile &t) {
    const int lane = threadIdx.x & 63;
    const bool on = lane < n_groups;
    const int r0 = on ? offsets[lane] : 0, r1 = on ? offsets[lane + 1] : 0;
    const int rows = r1 - r0 > 0 ? r1 - r0 : 0;
    const int f = rows / ROWS;
    const bool p = (rows % ROWS) != 0;
    int incl = f;                                        // whole row tiles of groups 0 .. lane
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    const int full = __builtin_amdgcn_readlane(incl, 63);
    const uint64_t pm = __ballot(p);
    int idx;
    if (!grouped_cell(full + __popcll(pm), tiles_n, chunk, b, idx, t.tile_n)) return false;
    const bool want_full = idx < full;
    if (!want_full) idx -= full;
    const uint64_t hit = want_full ? __ballot(incl - f <= idx && idx < incl)
                                   : __ballot(p && __popcll(pm & ((1ull << lane) - 1ull)) == idx);
    if (!hit) return false;
    const int g = __ffsll((unsigned long long)hit) - 1;
    const int gf = __builtin_amdgcn_readlane(f, g);
    t.group = g;
    t.m0 = __builtin_amdgcn_readlane(r0, g) + (want_full ? idx - (__builtin_amdgcn_readlane(incl, g) - gf) : gf) * ROWS;
    t.m_end = __builtin_amdgcn_readlane(r1, g);
    return true;
}
template <int ROWS>
__device__ inline bool grouped_tile(const int32_t *__restrict__ offsets, int n_groups, int tiles_n, int chunk, int b,
                                    GroupTile &t) {
    if (n_groups <= 64) return grouped_tile_lanes<ROWS>(offsets, n_groups, tiles_n, chunk, b, t);
    int full = 0, part = 0;
    for (int e = 0; e < n_groups; e++) {
        const int rows = offsets[e + 1] - offsets[e];
        full += rows / ROWS;
        part += (rows % ROWS) != 0;
    }
    int idx;
    if (!grouped_cell(full + part, tiles_n, chunk, b, idx, t.tile_n)) return false;
    const bool want_full = idx < full;
    if (!want_full) idx -= full;
    for (int e = 0; e < n_groups; e++) {
        const int r0 = offsets[e], r1 = offsets[e + 1];
        const int f = (r1 - r0) / ROWS;
        if (want_full) {
            if (idx < f) { t.group = e; t.m0 = r0 + idx * ROWS; t.m_end = r1; return true; }
            idx -= f;
        } else if ((r1 - r0) % ROWS) {
            if (idx == 0) { t.group = e; t.m0 = r0 + f * ROWS; t.m_end = r1; return true; }
            idx--;
        }
    }
    return false;
}
// A 64-bit value that is the same in every lane, moved to scalar registers.  (The builtin returns a signed
// int: each half goes through uint32_t on its way back, or the low half would sign-extend into the high one.)
__device__ inline uint64_t uniform64(uint64_t v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (uint64_t)lo | ((uint64_t)hi << 32);
}

// Lane `l`'s 64-bit value (l the same in every lane), in scalar registers.
__device__ inline uint64_t lane_value64(uint64_t v, int l) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, l);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), l);
    return (uint64_t)lo | ((uint64_t)hi << 32);
}

// The lane's number within its wave, computed where it is called: the statement is opaque to the compiler, which
// therefore neither merges it with an earlier copy nor keeps that copy alive for it.
__device__ inline int fresh_lane_id() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

// activation of the gate branch: 0 = SiLU, 1 = GELU in its tanh form.  Written with the hardware's exp2 and
// reciprocal (1 ulp each; the result is rounded to 16 bits): the correctly rounded division and the library tanh
// that the build's flags would otherwise expand to are some thirty instructions per value, 128 values per lane in
// a full tile's epilogue.
__device__ inline float gemm_gate_act(float g, int act) {
    if (act == 0) return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
    const float u = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    // tanh(u) = 1 - 2 / (1 + e^(2u)); e^(2u) = inf gives 1, 0 gives -1
    const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.8853900817779268f * u));
    return 0.5f * g * (1.0f + t);
}


// GROUPED: the launch covers the row tiles of all groups (see GroupArgs); the tall form then takes one row
// tile for up to 256 rows of a group and runs only the 32-row blocks that hold rows.
// DUAL (grouped tall form only): the fused gate/up projection of a gated MLP.  The wave's two 32-row weight
// blocks are the same 32 rows of the gate and of the up weight (a workgroup covers 128 columns of both), and
// the epilogue stores act(gate) * up.  With eight waves a wave has one 32-row block: its first tile (16 rows) is
// the gate's, its second the same 16 rows of the up weight, so that both products of an output element still
// end in the same lane (accumulator i and i + 8).
// NARROW (dense 128-row DMA form only): 128 weight rows per workgroup instead of 256, one 32-row block per wave -
// twice the workgroups for a product whose 256-column tiles leave compute units idle, without the partial sums
// of a K split.
template <int QT, typename AT, bool DMA, int MB, bool GROUPED = false, bool DUAL = false, int WAVES = 4, bool NARROW = false>
__global__ __launch_bounds__(64 * WAVES, (DMA && MB == 4) ? 2 : 1) void gemm_mfma_kernel(const AT *__restrict__ x, const uint8_t *__restrict__ w,
                                                        AT *__restrict__ y, int M, int N, int K, int band_m,
                                                        const GroupArgs ga, int k_steps,
                                                        float *__restrict__ ws, int tn0, int tn_cnt) {
    using F = Fmt<QT>;
    using V8 = typename Vec8<AT>::type;
    static_assert(MB == 4 || (MB == 8 && DMA), "row tiles of 128 rows, or 256 rows in the DMA form");
    static_assert(!DUAL || (GROUPED && MB == 8), "the fused gate/up form exists for grouped launches of the tall form");
    static_assert(WAVES == 4 || (WAVES == 8 && MB == 8 && DMA), "eight waves: tall form only");
    static_assert(!NARROW || (DMA && MB == 4 && WAVES == 4 && !GROUPED && !DUAL), "the narrow tile is a dense 128-row DMA form");
    constexpr int MB32 = MB, GM = 32 * MB;            // shadow the 128-row constants of the file
    constexpr int GN = NARROW ? lowbit::GN / 2 : lowbit::GN;
    constexpr int NB32 = GN / WAVES / 32;             // 32-row weight blocks per wave: 2, or 1 with eight waves or a narrow tile
    // x block of a K step: 8 * MB32 pieces of 1 KiB (layout below), double buffered
    __shared__ __attribute__((aligned(16))) uint8_t xs[2 * 8 * MB32 * 1024];
    uint8_t *const xs0 = xs, *const xs1 = xs + 8 * MB32 * 1024;
    __shared__ float lut[16];
    if constexpr (QT == QT_NF4) {
        if (threadIdx.x < 16) lut[threadIdx.x] = NF4_CODEBOOK[threadIdx.x];
    }

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: scalar address arithmetic
    const int G = K / TILE_COLS;
    const int n_tiles = N / TILE_ROWS;

    // Workgroups are handed to the 8 XCDs round-robin (id % 8) and each XCD has its own L2.  The output tiles
    // are put in one line - bands of band_m row tiles; within a band column tile by column tile, the band's row
    // tiles side by side - and each XCD takes an equal eighth of that line (+- one tile): its L2 then holds one
    // band of x (two where its share crosses a band's end), re-read by every column tile, and sees each weight
    // tile from all row tiles of the band at about the same time.  Equal shares matter more than whole bands:
    // with a band per XCD group, 11 row tiles by 43 column tiles put 66 tiles on six XCDs and 44 on two, and 66
    // tiles are a second round for an XCD whose 32 CUs hold 64 workgroups.
    int m0, tile_n;
    const uint8_t *w_up = nullptr;
    if constexpr (!GROUPED) {
        const int tiles_m = (M + GM - 1) / GM, tiles_n = tn_cnt;
        const int64_t T = (int64_t)tiles_m * tiles_n;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int first = (int)(T * xcd / 8), count = (int)(T * (xcd + 1) / 8) - first;
        // A launch with fewer tiles than compute units goes out in half tiles, twice as many workgroups (the
        // launcher says how many tiles at the end of each XCD's share are cut: all of them or none).
        int idx = slot, half = -1;
        if constexpr (DMA && MB32 == 4) {
            const int whole = count - (ga.split_tail < count ? ga.split_tail : count);
            if (slot >= whole) {
                idx = whole + ((slot - whole) >> 1);
                half = (slot - whole) & 1;
            }
        }
        if (idx >= count) return;                                                    // whole workgroup leaves
        const int line = first + idx;
        const int per_band = band_m * tiles_n;
        const int band = line / per_band, r = line - band * per_band;
        const int rows_b = tiles_m - band * band_m < band_m ? tiles_m - band * band_m : band_m;   // the last band may be short
        tile_n = r / rows_b + tn0;
        m0 = (band * band_m + r % rows_b) * GM;
        if (half >= 0) {
            m0 += (GM / 2) * half;
            if (m0 >= M) return;                                                     // (a last row tile of at most 64 rows)
            M = M < m0 + GM / 2 ? M : m0 + GM / 2;                                   // rows past the half are clamped / not stored
        }
    } else if (DUAL && ga.offsets == nullptr) {
        // one group of all M rows: the cells are dealt as in a grouped launch, a row tile is 256 rows of x
        int idx;
        if (!grouped_cell((M + GM - 1) / GM, tn_cnt, ga.chunk, blockIdx.x, idx, tile_n)) return;     // whole workgroup leaves
        m0 = idx * GM;
        w_up = ga.w_up_one;
    } else {
        // every workgroup finds its row tile from the offsets itself
        // (up to 64 groups: lane e also fetches group e's weight pointers while the offsets are on their way)
        const bool by_lane = ga.n_groups <= 64;
        uint64_t w_lane = 0, w_up_lane = 0;
        if (by_lane && lane < ga.n_groups) {
            w_lane = (uint64_t)ga.w[lane];
            if constexpr (DUAL) w_up_lane = (uint64_t)ga.w_up[lane];
        }
        GroupTile gt;
        if (!grouped_tile<GM>(ga.offsets, ga.n_groups, tn_cnt, ga.chunk, blockIdx.x, gt)) return;    // whole workgroup leaves
        // (the compiler does not see that what comes out of the walk is the same in every lane)
        tile_n = __builtin_amdgcn_readfirstlane(gt.tile_n);
        m0 = __builtin_amdgcn_readfirstlane(gt.m0);
        M = __builtin_amdgcn_readfirstlane(gt.m_end);   // rows past the group's end are clamped / not stored
        const int group = __builtin_amdgcn_readfirstlane(gt.group);
        if (by_lane) {
            w = (const uint8_t *)lane_value64(w_lane, group);
            if constexpr (DUAL) w_up = (const uint8_t *)lane_value64(w_up_lane, group);
        } else {
            w = ga.w[group];
            if constexpr (DUAL) w_up = ga.w_up[group];
        }
    }
    constexpr int GN_WG = DUAL ? GN / 2 : GN, GN_W = GN_WG / WAVES;   // columns of y per workgroup, per wave
    constexpr bool DUAL1 = DUAL && NB32 == 1;     // gate and up rows share the wave's one 32-row block
    const int n0 = tile_n * GN_WG + wave * GN_W;

    // weight tiles of this lane: block nb covers rows n0 + 32*nb .. +31 (clamped: a tile row past N
    // is computed and never stored)
    const int kg = lane >> 5, i32 = lane & 31, r16 = lane & 15;
    const int slot_lo = kg * 16 + r16, slot_hi = (kg + 2) * 16 + r16;
    gbytes wt[NB32];
#pragma unroll
    for (int nb = 0; nb < NB32; nb++) {
        int trow = n0 / TILE_ROWS + (DUAL ? 0 : nb * 2) + (DUAL1 ? 0 : (i32 >> 4));
        trow = trow < n_tiles ? trow : n_tiles - 1;
        const uint8_t *wbase = (DUAL && nb == 1) ? w_up : w;
        if constexpr (DUAL1) wbase = (i32 >> 4) ? w_up : w;
        wt[nb] = (gbytes)wbase + (int64_t)trow * G * F::TILE_BYTES;
    }

    // The x block of a K step (128 rows x 256 bytes) sits in LDS as 32 pieces of 1 KiB: piece h * 16 + t
    // holds rows 8t .. 8t+7 of the half row h (64 columns = 128 bytes = one cache line per row), the 16 bytes
    // of (row r = 0..7, 16-byte chunk c = 0..7) at ((r ^ t % 2) * 8 + (c ^ r)) * 16.  Two things shape it:
    //   - One wave-wide load fills one piece with lane l at byte 16 l of it (LDS-DMA writes the lanes to LDS in
    //     lane order), and eight consecutive lanes fetch the eight chunks of ONE row, a whole cache line: lane
    //     l = 8 s + c' fetches row r = s ^ t % 2, chunk c' ^ r.  With the lanes running across rows instead
    //     (lane 8 c + r, eight lines per eight lanes) the same bytes load 3.6 times slower (measured from L2:
    //     38 against 135 GB/s per CU), and that was a quarter of the GEMM's time.
    //   - Lane (kg, i) of the MFMA reads, for 16-column step ks and row block mb, row r = i % 8 of piece
    //     (ks/4) * 16 + 4*mb + i/8 and chunk c = ks%4 * 2 + kg.  Rows lie 128 bytes apart and pieces 1 KiB,
    //     both a divisor or multiple of the 256 bytes the LDS banks span: the xor with r spreads the eight rows
    //     of a piece over the banks, the xor with t % 2 puts the next piece's rows on the other half of them,
    //     so that every 16 lanes cover all banks once (without it a wave-wide 16-byte read runs at half rate:
    //     303 against 598 GB/s per CU, measured with 8 waves reading back to back).
    // This lane's row and byte column within an even / odd piece, when it loads one:
    const int xr_l[2] = {lane >> 3, (lane >> 3) ^ 1};
    const int xc_l[2] = {(((lane & 7) ^ xr_l[0]) * 16), (((lane & 7) ^ xr_l[1]) * 16)};
    //
    // Register-staged form: x goes global -> registers -> LDS, piece by piece as above: wave w moves the
    // pieces 8w .. 8w+7 (half row w/2, rows 64*(w%2) + 8i ..).
    uint32_t xoff[DMA ? 1 : 8];
    int xl[DMA ? 1 : 8];
    // DMA form: x goes global -> LDS without passing through registers, one instruction per piece.  Wave
    // w fills pieces 8w .. 8w+7: half row w/2, rows 64*(w%2) + 8j ...  Rows past M are clamped.  Each piece has
    // its lane offset from the tile's first row in a register of its own (below 2^31: the launcher keeps K
    // below 2^23), fixed for the whole walk along K; what changes from step to step is a scalar base.
    uint32_t xone_off[(DMA && MB32 == 4) ? 8 : 1];
    if constexpr (!DMA) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int row = m0 + 64 * (wave & 1) + 8 * i + xr_l[i & 1];
            row = row < M ? row : M - 1;
            xoff[i] = (uint32_t)(((int64_t)row * K + (wave >> 1) * 64) * (int64_t)sizeof(AT) + xc_l[i & 1]);
            xl[i] = (wave * 8 + i) * 1024 + lane * 16;
        }
    } else if constexpr (MB32 == 4) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            int row = (GM / 2) * (wave & 1) + 8 * j + xr_l[j & 1];
            row = m0 + row < M ? row : M - 1 - m0;
            xone_off[j] = (uint32_t)row * (uint32_t)K * (uint32_t)sizeof(AT) + (uint32_t)((wave >> 1) * 128 + xc_l[j & 1]);
        }
    }
    const uint64_t xone_base = (uint64_t)(uintptr_t)x + (uint64_t)m0 * (uint64_t)K * sizeof(AT);
    constexpr int PW = 8 * MB32 / WAVES;                  // pieces of 1 KiB (8 rows of a half row) a wave fetches per K step
    // Split-K: with a workspace the grid has a second dimension, workgroup (t, s) walks the K steps
    // s * k_steps .. and leaves its fp32 partial tile in ws[s]; a second kernel sums the splits.  It
    // fills the machine when the output alone has too few tiles (small M, narrow N).
    const int kt0 = ws ? blockIdx.y * k_steps : 0;
    const int Gs = ws ? (k_steps < G - kt0 ? k_steps : G - kt0) : G;
    const int last = Gs - 1;
    // the same loads one at a time, for spreading them over a step: a burst of 8 + 6 loads per wave,
    // from eight waves at once, queues up at the CU's address unit and the waves stand still meanwhile
    // (measured with cycle counters: 41 % of a K step at M = 2048)
    auto dma_x_one = [&](int kt, uint8_t *buf, int j) __attribute__((always_inline)) {
        kt = kt0 + (kt < last ? kt : last);
        // Issued from inline assembly: the compiler's wait-count pass treats an LDS-DMA as aliasing
        // every later LDS access and would wait for it immediately.  Completion is awaited by the
        // explicit vmcnt(0) ahead of the workgroup barrier that publishes the buffer.
        const uint64_t src = uniform64(xone_base + (uint64_t)kt * (TILE_COLS * sizeof(AT)));
        const uint32_t lbase = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)buf + wave * PW * 1024);
        asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(xone_off[(DMA && MB32 == 4) ? j : 0]), "s"(src), "s"(lbase), "n"(j * 1024) : "memory", "m0", "scc");
    };
    // Tall form: the per-lane part of the address is a 32-bit offset, one register per piece (the dense tall form
    // has registers to spare), and the scalar base changes once per K step: a load is three instructions - M0 from
    // the buffer's base plus an immediate, the wait state that M0 needs, the load.  (With the piece's rows added to
    // the scalar base instead it was six, and a load's slot between two MFMAs overran the 28 cycles the MFMA ahead
    // of it covers.)  Dense launches hand this form whole 256-row tiles only, so no row is clamped.
    const uint32_t xlane_off = (uint32_t)xr_l[0] * (uint32_t)K * (uint32_t)sizeof(AT) + (uint32_t)xc_l[0];       // even pieces
    const uint32_t xlane_off_odd = (uint32_t)xr_l[1] * (uint32_t)K * (uint32_t)sizeof(AT) + (uint32_t)xc_l[1];   // odd pieces
    const uint64_t xwave_base = (uint64_t)(uintptr_t)x +
        ((uint64_t)(m0 + (GM / (WAVES / 2)) * (wave % (WAVES / 2))) * (uint64_t)K + (uint64_t)(wave / (WAVES / 2)) * 64u) * sizeof(AT);
    uint32_t xpiece_off[(MB32 == 8 && !GROUPED) ? PW : 1];
    if constexpr (MB32 == 8 && !GROUPED) {
#pragma unroll
        for (int j = 0; j < PW; j++)            // (whole tile below 2^31 bytes from its first row: K < 2^23)
            xpiece_off[j] = ((j & 1) ? xlane_off_odd : xlane_off) + (uint32_t)j * 8u * (uint32_t)K * (uint32_t)sizeof(AT);
    }
    auto dma_x_scalar = [&](int kt, uint8_t *buf, const int j) __attribute__((always_inline)) {
        kt = kt0 + (kt < last ? kt : last);
        const uint64_t src = xwave_base + (uint64_t)kt * (TILE_COLS * sizeof(AT));
        const uint32_t lbase = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)buf + wave * PW * 1024);
        asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(xpiece_off[(MB32 == 8 && !GROUPED) ? j : 0]), "s"(src), "s"(lbase), "n"(j * 1024) : "memory", "m0", "scc");
    };
    // Grouped tall form: a tile holds rows_here <= 256 rows of its group and only the first MBC 32-row blocks are
    // computed.  With HW = WAVES / 2 waves per half row, wave w fills the pieces HW * j + w % HW (rows
    // 8 * (HW * j + w % HW) ..) of half row w / HW for j < 4 * MBC / HW:
    // the same count for every wave and a bound known at compile time, so that the main loop stays free of
    // branches.  The wave's pieces of the last block (two with four waves, one with eight) may reach past the
    // group's rows: they take their rows from a
    // per-lane offset relative to the tile's first row, with the row clamped to the group's last one (rows past
    // it are computed from a copy of that row and never stored).
    constexpr unsigned HW = WAVES / 2; constexpr int XPB = 4 / HW;         // waves per half row; pieces per wave and 32-row block
    const int rows_here = __builtin_amdgcn_readfirstlane(M - m0 < GM ? M - m0 : GM);
    uint64_t xtile_base = (uint64_t)(uintptr_t)x + ((uint64_t)m0 * (uint64_t)K + (uint64_t)((unsigned)wave / HW) * 64u) * sizeof(AT);
    auto tail_offset = [&](int j) __attribute__((always_inline)) {            // piece j of this wave, rows clamped
        int row = 8 * (int)(HW * j + ((unsigned)wave % HW)) + xr_l[wave & 1];
        row = row < rows_here ? row : rows_here - 1;
        return (uint32_t)row * (uint32_t)K * (uint32_t)sizeof(AT) + (uint32_t)xc_l[wave & 1];
    };
    const uint32_t xlane_off_wave = (wave & 1) ? xlane_off_odd : xlane_off;     // this wave's pieces are all odd or all even
    // (voff_tail: this lane's offset from the tile's first row for each of the wave's pieces, the rows of the last
    // block's two clamped; fixed for the walk along K, like the dense forms' - see grouped_piece_offsets below)
    constexpr bool GTALL = GROUPED && MB32 == 8;
    // Eight waves have half the vector registers: there a wave's pieces share one lane offset (its first piece's)
    // and the rows of piece j are added to the scalar base; the one piece of the last block keeps its own,
    // clamped, offset.  (Scalar arithmetic is cheap with two waves per SIMD; with one, every instruction between
    // two MFMAs is issue time.)
    constexpr bool SCALAR_ROWS = GTALL && WAVES == 8;
    constexpr int NVOFF = SCALAR_ROWS ? 2 : GTALL ? XPB * MB32 : 2;
    // What a variant of the main loop keeps for its LDS-DMAs of x: the lane offsets of the wave's pieces and where
    // the pieces start within an x buffer (a scalar: the wave index is one)
    struct XGrouped {
        uint32_t voff[NVOFF];
        uint32_t lds_wave_off;
    };
    auto dma_x_grouped = [&](int kt, uint8_t *buf, const int j, auto mbc_, const XGrouped &xg) __attribute__((always_inline)) {
        constexpr int MBC = decltype(mbc_)::value;
        const uint32_t (&voff_tail)[NVOFF] = xg.voff;
        const uint32_t lds_wave_off = xg.lds_wave_off;
        kt = kt0 + (kt < last ? kt : last);
        const bool tail = j >= XPB * (MBC - 1);
        // the same in every lane, which the compiler does not always see after the walk over the groups
        uint64_t src = xtile_base + (uint64_t)kt * (TILE_COLS * sizeof(AT));
        if (SCALAR_ROWS && !tail) src += (uint64_t)((uint32_t)(8 * HW * j) * (uint32_t)K * (uint32_t)sizeof(AT));
        src = uniform64(src);
        const uint32_t lbase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)buf + lds_wave_off;
        asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(voff_tail[SCALAR_ROWS ? (tail ? 1 : 0) : GTALL ? j : 0]), "s"(src), "s"(lbase), "n"((int)HW * j * 1024) : "memory", "m0", "scc");
    };
    auto dma_x = [&](int kt, uint8_t *buf, auto mbc_, const XGrouped &xg) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < (GTALL ? XPB * decltype(mbc_)::value : PW); j++) {
            if constexpr (GTALL) dma_x_grouped(kt, buf, j, mbc_, xg);
            else if constexpr (MB32 == 8) dma_x_scalar(kt, buf, j);
            else dma_x_one(kt, buf, j);
        }
    };
    auto load_x = [&](int kt, u32x4 (&xr)[8]) __attribute__((always_inline)) {
        kt = kt0 + (kt < last ? kt : last);              // past the end: a harmless re-read, never used
        const uint8_t *xk = (const uint8_t *)x + (int64_t)kt * TILE_COLS * sizeof(AT);
#pragma unroll
        for (int i = 0; i < 8; i++) xr[i] = *(const u32x4 *)(xk + xoff[i]);
    };
    auto load_x_one = [&](int kt, u32x4 (&xr)[8], int i) __attribute__((always_inline)) {
        kt = kt0 + (kt < last ? kt : last);
        xr[i] = *(const u32x4 *)((const uint8_t *)x + (int64_t)kt * TILE_COLS * sizeof(AT) + xoff[DMA ? 0 : i]);
    };
    auto store_x = [&](uint8_t *buf, const u32x4 (&xr)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 8; i++) *(u32x4 *)(buf + xl[i]) = xr[i];
    };
    struct WRegs {
        TileRegs<QT> lo[NB32], hi[NB32];
    };
    auto load_w = [&](int kt, WRegs &t) __attribute__((always_inline)) {
        kt = kt0 + (kt < last ? kt : last);
#pragma unroll
        for (int nb = 0; nb < NB32; nb++) {
            const gbytes tile = wt[nb] + (int64_t)kt * F::TILE_BYTES;
            load_tile<QT>(tile, slot_lo, r16, t.lo[nb]);
            t.hi[nb].q0 = ld<u32x4>(tile + slot_hi * 16);
            if constexpr (F::BITS == 8) t.hi[nb].q1 = ld<u32x4>(tile + 1024 + slot_hi * 16);
        }
    };

    auto load_w_nb = [&](int kt, WRegs &t, int nb) __attribute__((always_inline)) {
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
    auto fetch_units = [&](int kt, uint8_t *buf, WRegs &t, const int point, const int points, auto mbc_,
                           const XGrouped &xg) __attribute__((always_inline)) {
        constexpr int UNITS = NB32 + (GTALL ? XPB * decltype(mbc_)::value : PW);
        const int spread = points * 5 / 8 > 0 ? points * 5 / 8 : 1;
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            if (u < point * UNITS / spread || u >= (point + 1) * UNITS / spread || point >= spread) continue;
            if (u < NB32) load_w_nb(kt, t, u);
            else if constexpr (GTALL) dma_x_grouped(kt, buf, u - NB32, mbc_, xg);
            else if constexpr (MB32 == 8) dma_x_scalar(kt, buf, u - NB32);
            else dma_x_one(kt, buf, u - NB32);
        }
    };

    // The same for the deeper pipeline of the grouped tall form (below): the pieces of x of step kt_x first, then the
    // weight registers of step kt_w, so that the weight loads are the youngest loads in flight when the step ends.
    auto fetch_units_deep = [&](int kt_x, uint8_t *buf, int kt_w, WRegs &t, const int point, const int points, auto mbc_,
                                const XGrouped &xg) __attribute__((always_inline)) {
        constexpr int XU = GTALL ? XPB * decltype(mbc_)::value : PW, UNITS = XU + NB32;
        const int spread = points * 5 / 8 > 0 ? points * 5 / 8 : 1;
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            if (u < point * UNITS / spread || u >= (point + 1) * UNITS / spread || point >= spread) continue;
            if (u < XU) {
                if constexpr (GTALL) dma_x_grouped(kt_x, buf, u, mbc_, xg);
                else if constexpr (MB32 == 8) dma_x_scalar(kt_x, buf, u);
                else dma_x_one(kt_x, buf, u);
            }
            else load_w_nb(kt_w, t, u - XU);
        }
    };

    // One set of accumulators for all variants of the main loop, cleared here.  Every MFMA names its
    // accumulator as an in-out operand of its assembly statement, which keeps each block in the same accumulation
    // registers from here to the epilogue.  It has to: the compiler does not know that the statements are MFMAs
    // and would copy a block to other registers without the wait states a fresh MFMA result needs.  (With the
    // accumulators declared per variant it did: the last K step was lost.  check_gemm_asm.py looks for such
    // copies in the generated assembly.)
    f32x16 acc[MB32][NB32];
#pragma unroll
    for (int mb = 0; mb < MB32; mb++)
#pragma unroll
        for (int nb = 0; nb < NB32; nb++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mb][nb][i] = 0.0f;

    const DqCtx ctx = {lut, dq_magic<QT, AT>()};
    // weights of 16-column step ks for block nb: sub-block ks/2, lo or hi registers
    auto dequant_pair = [&](const WRegs &t, int ks, int nb, int p) __attribute__((always_inline)) -> uint32_t {
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
    auto x_piece = [](int ks, int mb) __attribute__((always_inline)) { return ((ks / 4) * 4 * MB32 + 4 * mb) * 1024; };
    int xlane[4];                                     // by ks % 4: the chunk index is xor-ed with the row, not added
#pragma unroll
    for (int t = 0; t < 4; t++)
        xlane[t] = (i32 >> 3) * 1024 + (((i32 & 7) ^ ((i32 >> 3) & 1)) * 8 + ((2 * t + kg) ^ (i32 & 7))) * 16;
    auto compute = [&](auto &acc, const uint8_t *cur, const WRegs &t, auto mbc_, auto &&between) __attribute__((always_inline)) {
        constexpr int MBC = decltype(mbc_)::value;
        constexpr int SLOTS = MBC * NB32, PAIRS = 4 * NB32;   // MFMAs per 16-column step; register pairs to dequantize meanwhile
        // MFMA slots that carry the dequantization of the next 16-column step.  A wave with one weight block uses
        // what it dequantizes in the very next MFMA after the step's last one: that last slot then stays empty,
        // so that a whole MFMA lies between the last write of an operand and its use.
        constexpr int SPREAD = (NB32 == 1 && SLOTS > 1) ? SLOTS - 1 : SLOTS;
        V8 xv[MBC];
        u32x4 wv[NB32];
#pragma unroll
        for (int mb = 0; mb < MBC; mb++) xv[mb] = *(const V8 *)(cur + xlane[0] + x_piece(0, mb));
#pragma unroll
        for (int nb = 0; nb < NB32; nb++)
#pragma unroll
            for (int p = 0; p < 4; p++) wv[nb][p] = dequant_pair(t, 0, nb, p);
        // From here on every operand of an MFMA is written at least a 16-column step ahead of it - except with a
        // single row block, where the next step's weights are dequantized right behind the MFMA that precedes
        // their use: those variants keep the two wait states ahead of every MFMA, the others spend them once.
        constexpr bool WAIT_STATES = MBC * NB32 < 4;
        if constexpr (!WAIT_STATES) {
            asm volatile("s_nop 1" : "+v"(wv[0]));
            if constexpr (NB32 == 2) asm volatile("" : "+v"(wv[1]));
        }
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            u32x4 wn[NB32];
#pragma unroll
            for (int mb = 0; mb < MBC; mb++) {
#pragma unroll
                for (int nb = 0; nb < NB32; nb++) {
                    // (a wave with one weight block uses what the step before dequantized last in the very first MFMA of a
                    // step, and where the compiler puts that last instruction is its choice: the two wait states stay)
                    if (NB32 == 1 && mb == 0) mfma_acc<true>(acc[mb][nb], __builtin_bit_cast(V8, wv[nb]), xv[mb]);
                    else mfma_acc<WAIT_STATES>(acc[mb][nb], __builtin_bit_cast(V8, wv[nb]), xv[mb]);
                    if (ks < 7) {
                        // pairs [ceil(slot * PAIRS / SLOTS), ceil((slot + 1) * PAIRS / SLOTS)): spread evenly over the
                        // MFMA slots, the first slot of a row block served first (the second is followed by the LDS
                        // read and the loads)
                        const int slot_i = mb * NB32 + nb;
#pragma unroll
                        for (int idx = 0; idx < PAIRS; idx++) {
                            if (slot_i >= SPREAD || idx < (slot_i * PAIRS + SPREAD - 1) / SPREAD || idx >= ((slot_i + 1) * PAIRS + SPREAD - 1) / SPREAD) continue;
                            wn[idx >> 2][idx & 3] = dequant_pair(t, ks + 1, idx >> 2, idx & 3);   // (weight block, pair)
                        }
                    }
                    // An MFMA occupies its pipe for 32 cycles and the wave issues in order: what stands between two
                    // MFMAs runs in the shadow of the first, and anything beyond 28 cycles of it leaves the pipe idle.
                    // Left alone the scheduler issues the MFMAs of a row block back to back and everything else after
                    // them (the second MFMA then waits 32 cycles with nothing to do, and a dozen instructions follow).
                    // (Not for nf4: its dequantization waits for code book reads from LDS, which the scheduler
                    // starts earlier when it is free to.)
                    if (nb + 1 < NB32 && QT != QT_NF4) __builtin_amdgcn_sched_barrier(0);
                }
                if (ks < 7) xv[mb] = *(const V8 *)(cur + xlane[(ks + 1) % 4] + x_piece(ks + 1, mb));
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
        // Where variants of the main loop meet, the compiler may move an accumulator block to other registers, and
        // it does not know that the block written last is still in the MFMA pipe: leave it the time to land (the
        // wave is on its way to a barrier here, the wait is hidden behind it).
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 1" : "+a"(acc[MBC - 1][NB32 - 1]));
    };
    // The same K step for the loop that runs one step ahead (x by LDS-DMA into the other buffer, the other weight
    // register set), with no seam between steps: a step begins with its first operands in registers.  Behind row
    // block BMB of its last 16-column step - when every read of this step's buffer has long returned - the step
    // waits for the next step's loads and passes the workgroup's one barrier per step; what is left of the last
    // 16-column step then reads the next step's first x operands from the other buffer and dequantizes its first
    // weights, work that a step otherwise does ahead of its first MFMA with the pipe idle (together with the wait
    // and the barrier about a tenth of a step).  The last step of a walk does the same (it reads a stale buffer and
    // dequantizes stale registers into operands nobody uses): one shape of step for the whole loop keeps every
    // accumulator block in its registers from the first step to the epilogue.
    auto first_operands = [&](const uint8_t *cur, const WRegs &t, auto mbc_, auto &xv, u32x4 (&wv)[NB32]) __attribute__((always_inline)) {
        constexpr int MBC = decltype(mbc_)::value;
#pragma unroll
        for (int mb = 0; mb < MBC; mb++) xv[mb] = *(const V8 *)(cur + xlane[0] + x_piece(0, mb));
#pragma unroll
        for (int nb = 0; nb < NB32; nb++)
#pragma unroll
            for (int p = 0; p < 4; p++) wv[nb][p] = dequant_pair(t, 0, nb, p);
        asm volatile("s_nop 1" : "+v"(wv[0]));          // VALU write of an MFMA operand: two wait states
        if constexpr (NB32 == 2) asm volatile("" : "+v"(wv[1]));
    };
    auto step_ahead = [&](auto &acc, const uint8_t *cur, const uint8_t *nxt, const WRegs &t, const WRegs &tn, auto mbc_,
                          auto &xv, u32x4 (&wv)[NB32], auto &&between) __attribute__((always_inline)) {
        constexpr int MBC = decltype(mbc_)::value;
        constexpr bool HAS_NEXT = true;
        constexpr int SLOTS = MBC * NB32, PAIRS = 4 * NB32;
        constexpr int SPREAD = (NB32 == 1 && SLOTS > 1) ? SLOTS - 1 : SLOTS;     // (see compute)
        constexpr bool WAIT_STATES = SLOTS < 4;          // (see compute)
        constexpr int BMB = MBC > 2 ? 1 : 0;
        constexpr int TAIL = (MBC - 1 - BMB) * NB32;     // MFMA slots of the last 16-column step behind the barrier
        constexpr int TSPREAD = (NB32 == 1 && TAIL > 1) ? TAIL - 1 : TAIL;      // of them, those that carry dequantization
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            u32x4 wn[NB32];
#pragma unroll
            for (int mb = 0; mb < MBC; mb++) {
#pragma unroll
                for (int nb = 0; nb < NB32; nb++) {
                    // (a wave with one weight block uses what the step before dequantized last in the very first MFMA of a
                    // step, and where the compiler puts that last instruction is its choice: the two wait states stay)
                    if (NB32 == 1 && mb == 0) mfma_acc<true>(acc[mb][nb], __builtin_bit_cast(V8, wv[nb]), xv[mb]);
                    else mfma_acc<WAIT_STATES>(acc[mb][nb], __builtin_bit_cast(V8, wv[nb]), xv[mb]);
                    if (ks < 7) {
                        const int slot_i = mb * NB32 + nb;
#pragma unroll
                        for (int idx = 0; idx < PAIRS; idx++) {
                            if (slot_i >= SPREAD || idx < (slot_i * PAIRS + SPREAD - 1) / SPREAD || idx >= ((slot_i + 1) * PAIRS + SPREAD - 1) / SPREAD) continue;
                            wn[idx >> 2][idx & 3] = dequant_pair(t, ks + 1, idx >> 2, idx & 3);
                        }
                    } else if constexpr (HAS_NEXT && TAIL > 0) {
                        if (mb > BMB) {                  // the next step's first weights, over the slots behind the barrier
                            const int ts = (mb - BMB - 1) * NB32 + nb;
#pragma unroll
                            for (int idx = 0; idx < PAIRS; idx++) {
                                if (ts >= TSPREAD || idx < (ts * PAIRS + TSPREAD - 1) / TSPREAD || idx >= ((ts + 1) * PAIRS + TSPREAD - 1) / TSPREAD) continue;
                                wn[idx >> 2][idx & 3] = dequant_pair(tn, 0, idx >> 2, idx & 3);
                            }
                        }
                    }
                    if (nb + 1 < NB32 && QT != QT_NF4) __builtin_amdgcn_sched_barrier(0);
                }
                if (ks < 7) xv[mb] = *(const V8 *)(cur + xlane[(ks + 1) % 4] + x_piece(ks + 1, mb));
                else if (HAS_NEXT && mb > BMB) xv[mb] = *(const V8 *)(nxt + xlane[0] + x_piece(0, mb));
                __builtin_amdgcn_sched_barrier(0);
                between(ks * MBC + mb, 8 * MBC);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (HAS_NEXT) {
                    if (ks == 7 && mb == BMB) {
                        wait_all_loads();                // this wave's part of the next step's x and weights has landed
                        __syncthreads();                 // (waits for this wave's LDS reads too) the other buffer is complete,
                                                         // and nobody reads this one any more
#pragma unroll
                        for (int m2 = 0; m2 <= BMB; m2++) xv[m2] = *(const V8 *)(nxt + xlane[0] + x_piece(0, m2));
                        if constexpr (TAIL == 0) {
#pragma unroll
                            for (int idx = 0; idx < PAIRS; idx++) wn[idx >> 2][idx & 3] = dequant_pair(tn, 0, idx >> 2, idx & 3);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            if (ks < 7 || HAS_NEXT) {
#pragma unroll
                for (int nb = 0; nb < NB32; nb++) wv[nb] = wn[nb];
            }
        }
    };
    typedef std::integral_constant<int, MB32> full_t;
    auto nothing = [](int, int) __attribute__((always_inline)) {};

    auto epilogue = [&](auto &acc, auto mbc_) __attribute__((always_inline)) {
        constexpr int MBC = decltype(mbc_)::value;
        // The lane's number, asked for anew: the values derived from threadIdx at the head of the kernel would
        // have to stay in registers (or, where those run out, in scratch memory with a reload inside the K loop)
        // all the way down to here.
        const int lane = fresh_lane_id(), kg = lane >> 5, i32 = lane & 31;
    // The MFMAs above are opaque to the compiler's hazard tracking: give the last results time to
    // land before the accumulation registers are read back (a 16-pass MFMA needs 18 wait states
    // before its result may be read; 64 are spent).  The accumulators are operands of the statement,
    // so that no read of them can be scheduled ahead of it.
#pragma unroll
    for (int mb = 0; mb < MBC; mb++) {
        if constexpr (NB32 == 2)
            asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7"
                         : "+a"(acc[mb][0]), "+a"(acc[mb][1]));
        else
            asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7"
                         : "+a"(acc[mb][0]));
    }
    // C layout of the 32x32 block: lane = 32*g + col (col = x row within the block), register i =
    // weight row 8*(i/4) + 4*g + i%4: four consecutive n per group of registers
    //
    // Straight from these registers a store instruction writes 16 bytes to each of 32 rows of y, 32 partly written
    // cache lines per instruction, under a row and a column test each.  So each wave first lays its rows out in
    // LDS - the x buffers, which nobody reads any more - and then stores them with eight (four) consecutive
    // lanes per row, whole 128 (64) byte runs, eight (sixteen) rows per instruction.  Row r of the wave's part
    // takes CH 16-byte chunks, chunk c at position c ^ r % CH, which spreads the writes of the 32 rows of a block
    // over the LDS banks.  Needs y 16-byte aligned; split-K partial sums keep their own layout.
    constexpr int CH = GN_W * (int)sizeof(AT) / 16;          // 16-byte chunks per row of this wave's columns
    constexpr int REGION = GM * CH * 16;                     // bytes per wave: WAVES / 2 of them fit an x buffer
    static_assert(REGION * (WAVES / 2) <= 8 * MB32 * 1024, "a wave's rows fit its share of an x buffer");
    static_assert(CH == (DUAL1 ? 2 : DUAL ? 4 : NB32 * 4), "one chunk per group of four accumulator registers and kg pair");
    constexpr int QN = DUAL1 ? 2 : 4;                        // register groups of a block that hold columns of y
    if constexpr (!DUAL) {
        if (ws) {
            // Partial sums of a K split keep the register layout (split, tile, wave, register group, lane): every
            // store is 1 KiB contiguous, straight from the accumulation registers, whole tiles whatever M and N
            // (the workspace holds whole tiles; the reduction kernel reads what lies inside y and undoes the layout).
            // dense: tiles in row-major order; grouped: in the order of the launch
            const int64_t tile_id = GROUPED ? (int64_t)blockIdx.x : (int64_t)(m0 / GM) * ((N + GN - 1) / GN) + tile_n;
            const int64_t n_tiles_all = GROUPED ? (int64_t)gridDim.x : (int64_t)((M + GM - 1) / GM) * ((N + GN - 1) / GN);
            float *const wp = ws + ((((int64_t)blockIdx.y * n_tiles_all + tile_id) * WAVES + wave) * (MB32 * NB32 * 4)) * 256 + lane * 4;
#pragma unroll
            for (int mb = 0; mb < MBC; mb++) {
#pragma unroll
                for (int nb = 0; nb < NB32; nb++) {
                    asm volatile("" : "+a"(acc[mb][nb]));            // (stay in accumulation registers up to here)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const f32x4 o = {acc[mb][nb][q * 4], acc[mb][nb][q * 4 + 1], acc[mb][nb][q * 4 + 2], acc[mb][nb][q * 4 + 3]};
                        *(f32x4 *)(wp + ((mb * NB32 + nb) * 4 + q) * 256) = o;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            return;
        }
    }
    if ((((uintptr_t)y) & 15) == 0) {
        typedef AT at4 __attribute__((ext_vector_type(4)));
        __syncthreads();                                     // every wave is done with its operand reads
        uint8_t *const stage = (wave < WAVES / 2 ? xs0 : xs1) + (wave % (WAVES / 2)) * REGION;
        uint8_t *wpos[CH];                                   // where this lane's 8 bytes of chunk c go, row block 0
#pragma unroll
        for (int c = 0; c < CH; c++) wpos[c] = stage + i32 * (CH * 16) + ((c ^ (i32 & (CH - 1))) * 16) + kg * 8;
#pragma unroll
        for (int mb = 0; mb < MBC; mb++) {
#pragma unroll
            for (int nb = 0; nb < (DUAL ? 1 : NB32); nb++) {
                // (keeps the block in its accumulation registers up to here: the compiler would otherwise read
                // all blocks into vector registers ahead of the branch that picks this form of the epilogue)
                if constexpr (DUAL && !DUAL1) asm volatile("" : "+a"(acc[mb][0]), "+a"(acc[mb][1]));
                else asm volatile("" : "+a"(acc[mb][nb]));
#pragma unroll
                for (int q = 0; q < QN; q++) {
                    at4 o;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        // (one block for both: registers 0..7 hold the gate's 16 rows, 8..15 the up weight's)
                        if constexpr (DUAL1) o[i] = to_at<AT>(gemm_gate_act(acc[mb][0][q * 4 + i], ga.act) * acc[mb][0][8 + q * 4 + i]);
                        else if constexpr (DUAL) o[i] = to_at<AT>(gemm_gate_act(acc[mb][0][q * 4 + i], ga.act) * acc[mb][1][q * 4 + i]);
                        else o[i] = to_at<AT>(acc[mb][nb][q * 4 + i]);
                    }
                    *(at4 *)(wpos[nb * 4 + q] + mb * 32 * (CH * 16)) = o;
                }
                __builtin_amdgcn_sched_barrier(0);           // one 32x32 block at a time (register footprint)
            }
        }
        // the rows were written by other lanes of this wave: LDS serves a wave's accesses in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        constexpr int RPI = 64 / CH;                         // rows per store instruction
        const int row_l = lane / CH, cs = lane % CH;
        const int n = n0 + ((cs ^ (row_l & (CH - 1))) * 8);  // (RPI is a multiple of CH: the same for every j)
        const int rows_left = n < N ? M - m0 - row_l : 0;    // this lane stores row j * RPI + row_l while that is below
        AT *const yp = y + (int64_t)(m0 + row_l) * N + n;
        const uint8_t *const rpos = stage + lane * 16;
#pragma unroll
        for (int j0 = 0; j0 < MBC * 32 / RPI; j0 += 8) {
            u32x4 v[8];
#pragma unroll
            for (int j = j0; j < j0 + 8 && j < MBC * 32 / RPI; j++) v[j - j0] = *(const u32x4 *)(rpos + j * 1024);
#pragma unroll
            for (int j = j0; j < j0 + 8 && j < MBC * 32 / RPI; j++)
                if (j * RPI < rows_left) *(u32x4 *)(yp + (int64_t)j * RPI * N) = v[j - j0];
        }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < MBC; mb++) {
        const int m = m0 + mb * 32 + i32;
        if constexpr (DUAL) {
            // both blocks hold the same 32 columns of y: the gate branch in block 0, the up branch in block 1
            if constexpr (DUAL1) asm volatile("" : "+a"(acc[mb][0]));
            else asm volatile("" : "+a"(acc[mb][0]), "+a"(acc[mb][NB32 - 1]));     // (stay in accumulation registers up to here)
            if (m < M) {
#pragma unroll
                for (int q = 0; q < QN; q++) {
                    const int n = n0 + q * 8 + kg * 4;
                    if (n < N) {
                        typedef AT at4 __attribute__((ext_vector_type(4)));
                        at4 o;
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            o[i] = to_at<AT>(gemm_gate_act(acc[mb][0][q * 4 + i], ga.act) *
                                             (DUAL1 ? acc[mb][0][8 + q * 4 + i] : acc[mb][NB32 - 1][q * 4 + i]));
                        *(at4 *)(y + (int64_t)m * N + n) = o;
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
#pragma unroll
            for (int nb = 0; nb < NB32; nb++) {
                asm volatile("" : "+a"(acc[mb][nb]));                    // (stay in accumulation registers up to here)
                if (m < M) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int n = n0 + nb * 32 + q * 8 + kg * 4;
                    if (n < N) {
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
        auto run = [&](auto mbc) __attribute__((always_inline)) {
            WRegs w0, w1;
            constexpr int MBC = decltype(mbc)::value;
            if constexpr (GTALL) {
                // Each variant of the main loop derives its addresses from values that are new to the compiler
                // here: otherwise it computes the scalar addresses of all variants ahead of the branch that
                // picks one, runs out of scalar registers and spills them (through vector registers to memory).
                uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)xtile_base);
                uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(xtile_base >> 32));
                asm volatile("" : "+s"(lo), "+s"(hi));
                xtile_base = (uint64_t)lo | ((uint64_t)hi << 32);
                if constexpr (NB32 == 2) asm volatile("" : "+v"(wt[0]), "+v"(wt[1]));
                else asm volatile("" : "+v"(wt[0]));
            }
            XGrouped xg = {};                             // grouped_piece_offsets
            uint32_t (&voff_tail)[NVOFF] = xg.voff;
            xg.lds_wave_off = (uint32_t)__builtin_amdgcn_readfirstlane(
                (int)((((unsigned)wave / HW) * (4 * MB32) + ((unsigned)wave % HW)) * 1024));
            if constexpr (SCALAR_ROWS) {
                voff_tail[0] = xlane_off_wave + (uint32_t)(8 * ((unsigned)wave % HW)) * (uint32_t)K * (uint32_t)sizeof(AT);
                voff_tail[1] = tail_offset(XPB * (MBC - 1));
            } else if constexpr (GTALL) {
#pragma unroll
                for (int j = 0; j < XPB * MBC; j++)
                    voff_tail[j] = j >= XPB * (MBC - 1) ? tail_offset(j)
                                                         : xlane_off_wave + (uint32_t)(8 * (HW * j + ((unsigned)wave % HW))) * (uint32_t)K * (uint32_t)sizeof(AT);
            }
            if constexpr (GTALL && MBC < 8) {
                // Tiles of a few row blocks have short K steps: with one step of prefetch a step lasted as long as
                // a weight load takes to come back from HBM, whatever it computed (removing the MFMAs of a four-block
                // tile saved 7 % of its time, removing the weight loads 21 %).  These variants have registers to
                // spare, so the weights run two steps ahead, through three register sets, and a step ends when
                // everything but the weight loads it has just issued has landed.  x keeps its two LDS buffers and
                // one step of prefetch (it comes from L2).  Three weight sets and two buffers: a period of six.
                constexpr int WLOADS = NB32 * ((F::BITS == 8 ? 2 : 1) * 2 + 1);      // load instructions of load_w_nb, all blocks
                WRegs w2;
                dma_x(0, xs0, mbc, xg);
                load_w(0, w0);
                load_w(1, w1);
                wait_all_loads();
                __syncthreads();
#define LOWBIT_DEEP_STEP(i, cur, nxt, wc, wl)                                                                  \
                if (kt + (i) < Gs) {                                                                           \
                    compute(acc, cur, wc, mbc, [&](const int point, const int points) __attribute__((always_inline)) { \
                        fetch_units_deep(kt + (i) + 1, nxt, kt + (i) + 2, wl, point, points, mbc, xg); \
                    });                                                                                        \
                    wait_loads_but<WLOADS>();                                                                  \
                    __syncthreads();                                                                           \
                }
                for (int kt = 0; kt < Gs; kt += 6) {
                    LOWBIT_DEEP_STEP(0, xs0, xs1, w0, w2)
                    LOWBIT_DEEP_STEP(1, xs1, xs0, w1, w0)
                    LOWBIT_DEEP_STEP(2, xs0, xs1, w2, w1)
                    LOWBIT_DEEP_STEP(3, xs1, xs0, w0, w2)
                    LOWBIT_DEEP_STEP(4, xs0, xs1, w1, w0)
                    LOWBIT_DEEP_STEP(5, xs1, xs0, w2, w1)
                }
#undef LOWBIT_DEEP_STEP
                wait_all_loads();                   // the loads past the end (clamped re-reads) must not outlive the wave's registers
                epilogue(acc, mbc);
                return;
            }
            dma_x(0, xs0, mbc, xg);
            load_w(0, w0);
            wait_all_loads();
            __syncthreads();
            w1 = w0;                                     // (never used before it is loaded: a defined value for the last step's look ahead)
            V8 xv[MBC];
            u32x4 wv[NB32];
            first_operands(xs0, w0, mbc, xv, wv);
            for (int kt = 0; kt + 1 < Gs; kt += 2) {
                step_ahead(acc, xs0, xs1, w0, w1, mbc, xv, wv, [&](const int point, const int points) __attribute__((always_inline)) {
                    fetch_units(kt + 1, xs1, w1, point, points, mbc, xg);
                });
                step_ahead(acc, xs1, xs0, w1, w0, mbc, xv, wv, [&](const int point, const int points) __attribute__((always_inline)) {   // past the end: clamped, unused re-reads
                    fetch_units(kt + 2, xs0, w0, point, points, mbc, xg);
                });
            }
            if (Gs & 1) step_ahead(acc, xs0, xs1, w0, w1, mbc, xv, wv, nothing);
            // (the compiler may move an accumulator block to other registers where the variants of the loop meet
            // and does not know that the block written last is still in the MFMA pipe: leave it the time to land)
            asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 1" : "+a"(acc[MBC - 1][NB32 - 1]));
            epilogue(acc, mbc);
        };
        // tail tiles and small expert groups: 32-row blocks without rows of x skip their MFMAs
        const int mb_cnt = (M - m0 + 31) / 32;
        if constexpr (MB32 == 8 && !GROUPED) {
            // the dense launcher hands the tall form whole 256-row tiles only
            run(full_t());
        } else if constexpr (MB32 == 8) {
            // one variant per count: only the last block of a variant may then hold rows past the group's end,
            // which is what the clamped offsets of its two pieces per wave cover
            switch (mb_cnt) {
            case 1: run(std::integral_constant<int, 1>()); break;
            case 2: run(std::integral_constant<int, 2>()); break;
            case 3: run(std::integral_constant<int, 3>()); break;
            case 4: run(std::integral_constant<int, 4>()); break;
            case 5: run(std::integral_constant<int, 5>()); break;
            case 6: run(std::integral_constant<int, 6>()); break;
            case 7: run(std::integral_constant<int, 7>()); break;
            default: run(full_t()); break;
            }
        } else if (mb_cnt <= 1) {
            run(std::integral_constant<int, 1>());
        } else if (mb_cnt <= 2) {
            run(std::integral_constant<int, 2>());
        } else {
            run(full_t());
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
        compute(acc, cur, wc, full_t(), [&](const int point, const int points) __attribute__((always_inline)) { \
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
    epilogue(acc, full_t());
    }
}


}  // namespace lowbit
