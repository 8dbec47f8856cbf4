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
#include "lowbit_gemm_kernel.h"

namespace lowbit {

int launch_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                int waves, hipStream_t st);

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

// A launch of the 128-row DMA form whose tiles leave most compute units idle goes out in half tiles of 64 rows, twice
// as many workgroups (see the kernel).  Half a tile pays the whole tile's dequantization and takes three quarters of
// its time per K step.  Measured on sym_int4 fp16 without a workspace, each launch on weights it has not just read:
// [4096 x 4096] at M = 128 / 512 / 768 (16 / 64 / 96 tiles): 38.9 -> 31.6 / 41.3 -> 34.1 / 41.7 -> 37.4 us;
// [11008 x 4096] at M = 128 / 256 (43 / 86 tiles): 40.3 -> 33.9 / 41.3 -> 35.8 us; [4096 x 11008] at M = 512:
// 99.4 -> 82.7 us.  At 112-128 tiles the two are level, and as soon as two halves share a unit it loses: 129 tiles
// 47 -> 57 us, 256 tiles ([4096 x 4096] at M = 2048) 64 -> 75 us.  Cutting only the tiles of a large launch's last,
// partly filled round changes nothing (688 tiles: 161 us either way) or loses 2-6 %.
static bool half_tiles(int M, int64_t tiles, int n_cus) { return M > GM / 2 && tiles * 8 <= (int64_t)n_cus * 3; }

// Estimated run time in microseconds of the 128-row GEMM with K split `splits` ways (1 = no split), fitted to
// measurements on MI355X: 40 weight shapes from [1024 x 8192] to [28672 x 8192] in all five formats, M = 17 .. 768,
// 1 .. 16 splits, each launch on weights it has not just read (6200 launches; 9.6 % rms).  What the fit holds:
//   - a 128-column step takes a workgroup 1.2 us while the launch has up to 128 workgroups, 1.5 us at one per CU,
//     and 2.1 us and more as soon as two share a CU - a launch of 258 workgroups takes as long as its two shared
//     CUs ([11008 x 4096] at M = 256: 2 splits = 172 workgroups 36.7 us, 3 splits = 258 workgroups 45.9 us), so the
//     splits that pay keep the workgroups at or below the number of CUs;
//   - a row tile that is partly empty skips the MFMAs of its empty 32-row blocks (a sixth of the step per quarter);
//   - launch, prologue and epilogue come to 2 us, the second launch of a split to 5.4 us, a workgroup's fp32 partial
//     tile to 0.043 us to write and sum (a quarter of it fixed, the rest by the rows it holds);
//   - the formats with more work per weight take longer per step: sym_int8 1.30, fp8_e4m3 1.15, nf4 1.30 - 2.48 in
//     the register-staged form it uses up to one workgroup per CU; half tiles take 0.88 (0.83) of a tile's step.
double gemm_time_us(int M, int N, int K, int splits, int qtype) {
    const int tiles_m = (M + GM - 1) / GM;
    const double tiles = (double)tiles_m * (double)((N + GN - 1) / GN);
    const int G = K / TILE_COLS;
    const int k_steps = (G + splits - 1) / splits;
    const int ny = (G + k_steps - 1) / k_steps;
    const bool halves = ny == 1 && qtype != QT_NF4 && half_tiles(M, (int64_t)tiles, 256);   // (nf4: register-staged form)
    const double wgs = tiles * ny * (halves ? 2.0 : 1.0);
    const bool heavy = qtype == QT_SYM_INT8 || qtype == QT_FP8_E4M3;
    const double format = qtype == QT_NF4 ? (wgs <= 256.0 ? 2.48 : 1.30) : qtype == QT_SYM_INT8 ? 1.30 : qtype == QT_FP8_E4M3 ? 1.15 : 1.0;
    const double half = !halves ? 1.0 : heavy ? 0.83 : 0.88;
    const double over128 = wgs > 128.0 ? (wgs - 128.0) / 128.0 : 0.0;
    const double step = wgs <= 256.0 ? 1.21 + 0.29 * over128 : 2.12 + 0.56 * ((wgs < 512.0 ? wgs : 512.0) - 256.0) / 256.0;
    // workgroups beyond two per CU wait for a slot: the launch lasts as long as the CU that gets most of them
    const double rounds = wgs > 512.0 ? (double)(((int64_t)wgs + 255) / 256) / 2.0 : 1.0;
    const double fill = (double)M / ((double)tiles_m * GM);
    double t = 2.1 + (double)k_steps * step * format * half * rounds * (0.83 + 0.17 * fill);
    if (ny > 1) t += 5.4 + 0.043 * (double)ny * tiles * (0.24 + 0.76 * fill);
    return t;
}

// Number of K splits to use for this shape given `ws_bytes` of workspace (1 = none): the fastest by the estimate
// above among 1 .. 16 splits of at least two K steps that fit the workspace.  On the shapes the estimate was fitted
// to, the split it picks is within 2 % of the best measured one on average.
int gemm_splits(int M, int N, int K, size_t ws_bytes, int qtype) {
    const size_t tiles = (size_t)((M + GM - 1) / GM) * (size_t)((N + GN - 1) / GN);
    const size_t per_split = tiles * GM * GN * sizeof(float);     // whole tiles: partial sums keep the tile layout
    const int G = K / TILE_COLS;
    int best = 1;
    double best_t = gemm_time_us(M, N, K, 1, qtype);
    for (int s = 2; s <= 16 && s * 2 <= G; s++) {
        if ((size_t)s * per_split > ws_bytes) break;
        const double t = gemm_time_us(M, N, K, s, qtype);
        if (t < best_t) {
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
static int tall_columns(int M, int N, int K, int n_cus, bool heavy_dequant) {
    if (M < 2 * GM_TALL || M % GM_TALL || M >= (1 << 24) || K >= (1 << 23)) return 0;
    const int tiles_m = M / GM_TALL, tiles_n = (N + GN - 1) / GN;
    const int rounds = tiles_m * tiles_n / n_cus;
    if (rounds < 1) return 0;
    int cols = rounds * n_cus / tiles_m;
    if (cols >= tiles_n) return tiles_n;
    const int left = (tiles_n - cols) * (M / GM);        // 128-row tiles of the remainder
    // sym_int8 and nf4 pay most per weight for the dequantization, which the tall form does half as often: for them
    // it wins with any remainder ([11008 x 4096] at M = 2048: +11 % and +5 %; sym_int4 +1 %, fp8_e4m3 -3 %)
    if (heavy_dequant) return cols;
    return 2 * left >= 3 * n_cus ? cols : 0;
}

// How many tiles at the end of each XCD's share of a 128-row launch go out as two half tiles: all of them or none.
static int split_tail_tiles(int M, int64_t tiles, int n_cus) {
    return half_tiles(M, tiles, n_cus) ? (int)(tiles / 8) + 1 : 0;
}

// Row tiles per band of the kernel's tile order (see the kernel): the row tiles are cut into at most 8 bands, a
// power of two of them, so that a band of x (band_m * rows per tile * K activations) stays small enough for an
// XCD's L2 where M allows it.
static int band_rows(int tiles_m) {
    int bands = 1;
    while (bands * 2 <= 8 && bands * 2 <= tiles_m) bands *= 2;
    return (tiles_m + bands - 1) / bands;
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
    const int tall = ws ? 0 : tall_columns(M, N, K, n_cus, QT == QT_SYM_INT8 || QT == QT_NF4);
    if (tall > 0) {
        const int tiles_m = M / GM_TALL;
        const unsigned grid = 8 * (unsigned)(((int64_t)tiles_m * tall + 7) / 8);
        // nf4 runs the tall tile with eight waves of 32 columns (two per SIMD cover each other's waits for the code
        // book reads from LDS: 5-9 % faster than four waves of 64 columns); the other formats are 2-4 % faster
        // with four waves, which read each x operand from LDS once per two MFMAs.
        if constexpr (QT == QT_NF4)
            hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, false, false, 8>), dim3(grid), dim3(512), 0, st,
                               (const AT *)x, (const uint8_t *)w, (AT *)y, M, N, K, band_rows(tiles_m), GroupArgs{}, G, (float *)nullptr, 0, tall);
        else
            hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL>), dim3(grid), dim3(256), 0, st,
                               (const AT *)x, (const uint8_t *)w, (AT *)y, M, N, K, band_rows(tiles_m), GroupArgs{}, G, (float *)nullptr, 0, tall);
        if (tall == tiles_n_all) return 0;
    }
    const int tn0 = tall, tiles_n = tiles_n_all - tall;
    const int tiles_m = (M + GM - 1) / GM;
    const int band_m = band_rows(tiles_m);
    const int k_steps = ws ? (G + splits - 1) / splits : G;
    const int ny = ws ? (G + k_steps - 1) / k_steps : 1;             // splits that actually hold steps
    const bool fits24 = M < (1 << 24) && K < (1 << 23);              // 24-bit row offsets
    const bool dma = fits24 && (QT != QT_NF4 || tiles_m * tiles_n * ny > 256);
    GroupArgs ga{};
    ga.split_tail = (dma && !ws) ? split_tail_tiles(M, (int64_t)tiles_m * tiles_n, n_cus) : 0;
    dim3 grid(8 * (unsigned)(((int64_t)tiles_m * tiles_n + 7) / 8 + ga.split_tail), ny);
    // Two forms of the kernel.  The DMA form (x straight into LDS, one K step of prefetch, 128 vector registers)
    // lets a CU hold two workgroups that cover each other's waits, and is 4-8 % ahead with a single workgroup per
    // CU as well - except with nf4, whose code book reads compete with the DMA for LDS: there the register-staged
    // form with its deeper prefetch is 4 % faster while there is at most one workgroup per CU.
    if (dma)
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32>), grid, dim3(256), 0, st, (const AT *)x, (const uint8_t *)w,
                           (AT *)y, M, N, K, band_m, ga, k_steps, ws, tn0, tiles_n);
    else
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, false, MB32>), grid, dim3(256), 0, st, (const AT *)x, (const uint8_t *)w,
                           (AT *)y, M, N, K, band_m, GroupArgs{}, k_steps, ws, tn0, tiles_n);
    if (ws) {
        const int64_t threads = (int64_t)tiles_m * tiles_n * (GM * GN / 4);
        hipLaunchKernelGGL((splitk_reduce_kernel<AT>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, ws,
                           (AT *)y, M, N, ny);
    }
    return 0;
}

// Whether a launch of narrow tiles goes out in half tiles of 64 rows: while the halves are no more than one per CU.
bool narrow_halves(int M, int N) {
    const int64_t tiles = (int64_t)((M + GM - 1) / GM) * ((N + GN / 2 - 1) / (GN / 2));
    return M > GM / 2 && tiles * 2 <= 256;
}

// Estimated run time in microseconds of the narrow form, fitted like gemm_time_us (760 launches, 8.5 % rms): a
// 128-column step takes a workgroup 1.05 us up to 128 workgroups, 1.24 at one per CU, 1.55 - 1.96 once two share a
// CU; half tiles 0.87 of it.
double narrow_time_us(int M, int N, int K, int qtype) {
    const int tiles_m = (M + GM - 1) / GM;
    const bool halves = narrow_halves(M, N);
    const double wgs = (double)tiles_m * (double)((N + GN / 2 - 1) / (GN / 2)) * (halves ? 2.0 : 1.0);
    const double format = qtype == QT_NF4 ? 1.24 : qtype == QT_SYM_INT8 ? 1.11 : qtype == QT_FP8_E4M3 ? 1.05 : 1.0;
    const double over128 = wgs > 128.0 ? (wgs - 128.0) / 128.0 : 0.0;
    const double step = wgs <= 256.0 ? 1.05 + 0.20 * over128 : 1.55 + 0.41 * ((wgs < 512.0 ? wgs : 512.0) - 256.0) / 256.0;
    const double rounds = wgs > 512.0 ? (double)(((int64_t)wgs + 255) / 256) / 2.0 : 1.0;
    const double fill = (double)M / ((double)tiles_m * GM);
    return 0.5 + (double)(K / TILE_COLS) * step * format * rounds * (halves ? 0.87 : 1.0) * (0.84 + 0.16 * fill);
}

// The narrow form of the 128-row DMA kernel: tiles of 128 x 128, or 64 x 128 (narrow_halves).
template <int QT, typename AT>
static int launch_gemm_narrow_t(const void *x, const void *w, void *y, int M, int N, int K, hipStream_t st) {
    if (M >= (1 << 24) || K >= (1 << 23)) return -3;                 // 24-bit row offsets
    const int G = K / TILE_COLS;
    const int tiles_n = (N + GN / 2 - 1) / (GN / 2), tiles_m = (M + GM - 1) / GM;
    const bool halves = narrow_halves(M, N);
    GroupArgs ga{};
    ga.split_tail = halves ? (int)(((int64_t)tiles_m * tiles_n) / 8) + 1 : 0;
    dim3 grid(8 * (unsigned)(((int64_t)tiles_m * tiles_n + 7) / 8 + ga.split_tail), 1);
    hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32, false, false, 4, true>), grid, dim3(256), 0, st, (const AT *)x,
                       (const uint8_t *)w, (AT *)y, M, N, K, band_rows(tiles_m), ga, G, (float *)nullptr, 0, tiles_n);
    return 0;
}

template <int QT>
static int launch_gemm_narrow_q(const void *x, const void *w, void *y, int dt, int M, int N, int K, hipStream_t st) {
    if (dt == DT_F16) return launch_gemm_narrow_t<QT, _Float16>(x, w, y, M, N, K, st);
    if (dt == DT_BF16) return launch_gemm_narrow_t<QT, __bf16>(x, w, y, M, N, K, st);
    return -4;
}

int launch_gemm_narrow(const void *x, const void *w, void *y, int qtype, int act_dtype, int M, int N, int K, hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    switch (qtype) {
    case QT_SYM_INT4: return launch_gemm_narrow_q<QT_SYM_INT4>(x, w, y, act_dtype, M, N, K, st);
    case QT_ASYM_INT4: return launch_gemm_narrow_q<QT_ASYM_INT4>(x, w, y, act_dtype, M, N, K, st);
    case QT_SYM_INT8: return launch_gemm_narrow_q<QT_SYM_INT8>(x, w, y, act_dtype, M, N, K, st);
    case QT_NF4: return launch_gemm_narrow_q<QT_NF4>(x, w, y, act_dtype, M, N, K, st);
    case QT_FP8_E4M3: return launch_gemm_narrow_q<QT_FP8_E4M3>(x, w, y, act_dtype, M, N, K, st);
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
    const int splits = !ws ? 1 : want_splits > 0 ? want_splits : gemm_splits(M, N, K, workspace_bytes, qtype);
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
