// Grouped products for mixture-of-experts layers: one launch covers the rows routed to every expert.
//
// The reference has no single call for it: it loops over the experts in Python and calls each expert's
// LowBitLinear on the rows routed to it (python/llm/src/ipex_llm/transformers/models/qwen2_moe.py:375-430
// is the pattern; the gated MLP of an expert is models/common.py:145-158).
//
// Two forms of the tiled MFMA GEMM kernel serve it:
//   - 128-row tiles, two workgroups per compute unit: a group of r rows takes ceil(r / 128) row tiles, each
//     of which walks (loads and dequantizes) the group's weights once;
//   - 256-row tiles ("tall"), one workgroup per compute unit: one walk for up to 256 rows, only the 32-row
//     blocks that hold rows are computed.  With a hundred and more rows per group - a prefill batch spread over
//     the experts - every group above 128 rows would otherwise walk its weights twice.
// The tall form also has the fused gate/up variant (act(x Wg^T) * (x Wu^T) in one pass over x) and can split
// K over a second grid dimension when the output alone has too few tiles for the machine (the down
// projection: few columns, long K); the fp32 partial tiles go through a workspace and a second kernel.
//
// This file: the choice of form and K splits, and the dispatch over the weight formats (instantiated in
// gemm_grouped_<format>.hip from lowbit_gemm_grouped.h).
#include <hip/hip_runtime.h>
#include "lowbit_formats.h"
#include "lowbit_grouped_plan.h"

namespace lowbit {

template <int QT>
int launch_grouped_q(const void *x, const void *const *w, const void *const *w_up, void *y, const int32_t *offsets,
                     int n_groups, int total_rows, int dt, int N, int K, int act, const GroupedPlan &plan, float *ws,
                     hipStream_t st);

template <int QT>
int launch_mlp_gemm_q(const void *x, const void *wg, const void *wu, void *y, int dt, int M, int N, int K, int act, int waves,
                      bool one_round, hipStream_t st);

static int device_cus() {
    static const int n_cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            n = 256;
        return n > 0 ? n : 256;
    }();
    return n_cus;
}

// Bytes of workspace per K split of the tall form: a partial tile per workgroup of the launch, whichever of the two
// tile orders it takes (the grid, and with it a workgroup's slot in the workspace, depends on the order).
static int tall_grid(int total_rows, int n_groups, int tiles_n, bool one_round) {
    return grouped_grid(grouped_max_row_tiles(total_rows, n_groups, G_GM_TALL), tiles_n, grouped_chunk(tiles_n, one_round));
}
static size_t tall_split_bytes(int total_rows, int n_groups, int N) {
    const int tiles_n = (N + G_GN - 1) / G_GN;
    const int a = tall_grid(total_rows, n_groups, tiles_n, false), b = tall_grid(total_rows, n_groups, tiles_n, true);
    return (size_t)(a > b ? a : b) * G_GM_TALL * G_GN * sizeof(float);
}

// Form and K splits for a grouped product given `ws_bytes` of workspace.  Measured on MI355X (8 groups of
// fp8_e4m3 weights, [14336 x 4096] and [4096 x 14336]):
//   - K is split when the tall tiles alone would leave compute units idle: as many splits as it takes for about
//     one workgroup per unit, at most 4, at least 8 K steps each.  With few columns and a long K (the down
//     projection) that beats both unsplit forms at every row count (32 rows per group: 131 against 193 us).
//   - Otherwise the 128-row form with two workgroups per unit is ahead up to about 96 rows per group (147
//     against 156 us at 96) and the tall form from there on (108-150 rows per group: 195 against 245 us).
// Waves per workgroup of the tall form.  Eight (32 weight rows each, two per SIMD) cover part of each other's waits
// where a tile has few MFMAs per weight: measured on MI355X with eight groups of 110-151 rows of fp8_e4m3 weights,
// the fused gate/up launch ([14336 x 4096] twice) takes 341-352 us with eight waves against 372-375 with four; the
// plain product of the down projection ([4096 x 14336], two K splits) 169 against 153-156 - its workgroups are a
// single round, and eight waves read every x operand from LDS twice as often.
static int grouped_waves(int total_rows, int n_groups, bool fused) {
    return fused && (int64_t)total_rows <= (int64_t)n_groups * 192 ? 8 : 4;
}

// Whether the workgroups that hold rows (an estimate: the host never sees the offsets) all run at once: the tall
// form holds one workgroup per compute unit, the 128-row form two.  The tile order then keeps a row tile's column
// tiles on one XCD (see grouped_tile) - when there are row tiles for every XCD.
static bool grouped_one_round(int total_rows, int n_groups, int tiles_n, bool tall, int splits) {
    const int rows = tall ? G_GM_TALL : G_GM_TALL / 2;
    const int row_tiles = total_rows / rows > n_groups ? total_rows / rows : n_groups;
    return row_tiles >= 8 && (int64_t)row_tiles * tiles_n * splits <= (int64_t)device_cus() * (tall ? 1 : 2);
}

GroupedPlan grouped_plan(int total_rows, int n_groups, int N, int K, size_t ws_bytes) {
    const int tiles_n = (N + G_GN - 1) / G_GN, G = K / TILE_COLS;
    const int row_tiles = total_rows / G_GM_TALL > n_groups ? total_rows / G_GM_TALL : n_groups;   // estimate of the tiles that hold rows
    int s = device_cus() / (tiles_n * row_tiles);
    s = s > 4 ? 4 : s;
    while (s > 1 && G / s < 8) s--;
    const size_t per_split = tall_split_bytes(total_rows, n_groups, N);
    while (s > 1 && (size_t)s * per_split > ws_bytes) s--;
    if (s < 1) s = 1;
    const bool tall = s > 1 || (int64_t)total_rows > (int64_t)n_groups * 96;
    return {tall, s, grouped_waves(total_rows, n_groups, false), grouped_one_round(total_rows, n_groups, tiles_n, tall, s)};
}

// What launch_grouped_gemm would do for a plain grouped product: {tall, splits, waves, grid.x}.
void grouped_plan_query(int total_rows, int n_groups, int N, int K, size_t ws_bytes, int out[4]) {
    const GroupedPlan p = grouped_plan(total_rows, n_groups, N, K, ws_bytes);
    const int tiles_n = (N + G_GN - 1) / G_GN;
    out[0] = p.tall;
    out[1] = p.splits;
    out[2] = p.tall ? p.waves : 4;
    out[3] = p.tall ? tall_grid(total_rows, n_groups, tiles_n, p.one_round)
                    : grouped_grid(grouped_max_row_tiles(total_rows, n_groups, G_GM_TALL / 2), tiles_n, grouped_chunk(tiles_n, p.one_round));
}

size_t grouped_workspace_bytes(int total_rows, int n_groups, int N, int K) {
    const GroupedPlan p = grouped_plan(total_rows, n_groups, N, K, (size_t)-1);
    return p.splits > 1 ? (size_t)p.splits * tall_split_bytes(total_rows, n_groups, N) : 0;
}

// y[rows of group e] = x[rows of group e] * dequant(w[e])^T, or, with w_up, act(x w[e]^T) * (x w_up[e]^T).
// workspace (may be null): lets the plain product split K.
int launch_grouped_gemm(const void *x, const void *const *w, const void *const *w_up, void *y, const int32_t *offsets,
                        int n_groups, int total_rows, int qtype, int act_dtype, int N, int K, int act, void *workspace,
                        size_t workspace_bytes, hipStream_t st) {
    if (total_rows == 0 || N == 0 || n_groups == 0) return 0;
    if (total_rows >= (1 << 24) || K >= (1 << 23)) return -3;        // 24-bit row offsets in the kernel
    float *ws = (float *)workspace;
    const GroupedPlan plan = w_up ? GroupedPlan{true, 1, grouped_waves(total_rows, n_groups, true),
                                                grouped_one_round(total_rows, n_groups, (N + G_GN / 2 - 1) / (G_GN / 2), true, 1)}
                                  : grouped_plan(total_rows, n_groups, N, K, ws ? workspace_bytes : 0);
    switch (qtype) {
    case QT_SYM_INT4: return launch_grouped_q<QT_SYM_INT4>(x, w, w_up, y, offsets, n_groups, total_rows, act_dtype, N, K, act, plan, ws, st);
    case QT_ASYM_INT4: return launch_grouped_q<QT_ASYM_INT4>(x, w, w_up, y, offsets, n_groups, total_rows, act_dtype, N, K, act, plan, ws, st);
    case QT_SYM_INT8: return launch_grouped_q<QT_SYM_INT8>(x, w, w_up, y, offsets, n_groups, total_rows, act_dtype, N, K, act, plan, ws, st);
    case QT_NF4: return launch_grouped_q<QT_NF4>(x, w, w_up, y, offsets, n_groups, total_rows, act_dtype, N, K, act, plan, ws, st);
    case QT_FP8_E4M3: return launch_grouped_q<QT_FP8_E4M3>(x, w, w_up, y, offsets, n_groups, total_rows, act_dtype, N, K, act, plan, ws, st);
    default: return -2;
    }
}

// y = act(x wg^T) * (x wu^T) for a dense gated MLP of M rows: the fused gate/up form of the grouped kernel on one
// group, its weights passed as arguments (nothing is read from tables in device memory).  Measured on MI355X
// against the two products as separate launches plus the activation as an elementwise kernel, sym_int4
// [11008 x 4096] twice: fp16 M = 512 / 2048: 117.5 -> 94.9 / 362.6 -> 318.1 us, bf16 137.2 -> 94.3 / 401.6 -> 316.6;
// nf4 [28672 x 8192] bf16 at M = 256 / 1024: 354.8 -> 233.6 / 1008 -> 892.
int launch_mlp_gemm(const void *x, const void *wg, const void *wu, void *y, int qtype, int act_dtype, int M, int N, int K,
                    int act, hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    if (M >= (1 << 24) || K >= (1 << 23)) return -3;                 // 24-bit row offsets in the kernel
    const int waves = grouped_waves(M, 1, true);
    const bool one_round = grouped_one_round(M, 1, (N + G_GN / 2 - 1) / (G_GN / 2), true, 1);
    switch (qtype) {
    case QT_SYM_INT4: return launch_mlp_gemm_q<QT_SYM_INT4>(x, wg, wu, y, act_dtype, M, N, K, act, waves, one_round, st);
    case QT_ASYM_INT4: return launch_mlp_gemm_q<QT_ASYM_INT4>(x, wg, wu, y, act_dtype, M, N, K, act, waves, one_round, st);
    case QT_SYM_INT8: return launch_mlp_gemm_q<QT_SYM_INT8>(x, wg, wu, y, act_dtype, M, N, K, act, waves, one_round, st);
    case QT_NF4: return launch_mlp_gemm_q<QT_NF4>(x, wg, wu, y, act_dtype, M, N, K, act, waves, one_round, st);
    case QT_FP8_E4M3: return launch_mlp_gemm_q<QT_FP8_E4M3>(x, wg, wu, y, act_dtype, M, N, K, act, waves, one_round, st);
    default: return -2;
    }
}

}  // namespace lowbit
