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
// This header holds the launch code as templates over the weight format; gemm_grouped_<format>.hip instantiate
// it, one file per format (the kernels of one format take about a minute to compile), gemm_grouped.hip
// holds the choice of form and splits and the dispatch over the formats.
#pragma once
#include "lowbit_gemm_kernel.h"

namespace lowbit {

constexpr int GROUPED_TALL_REGS = MB32_TALL * NB32 * 4;       // groups of 4 accumulators per lane and wave

// How a grouped launch runs: chosen on the host from the row count, never from the rows per group, which only
// the device knows.
struct GroupedPlan {
    bool tall;      // 256-row tiles (always for the fused gate/up form)
    int splits;     // K splits of the tall form (1 = none)
};

// Upper bound of the number of `rows`-row tiles: every group adds at most one partly filled tile.
inline int grouped_max_row_tiles(int total_rows, int n_groups, int rows) { return total_rows / rows + n_groups; }

// Sums the fp32 partial tiles of the K splits of a grouped tall launch (register layout: split, workgroup,
// wave, register group, lane) and writes y, rounded once.  One block of 256 threads per (workgroup, wave) of
// the GEMM: its 64 register groups of 64 lanes x 4 floats, four groups at a time; groups of 32-row blocks
// without rows are skipped.
template <typename AT>
__global__ __launch_bounds__(256) void grouped_splitk_reduce_kernel(const float *__restrict__ ws, AT *__restrict__ y,
                                                                    const int32_t *__restrict__ offsets, int n_groups,
                                                                    int N, int tiles_n, int n_wg, int splits) {
    const int b = blockIdx.x >> 2, wave = blockIdx.x & 3;              // workgroup and wave of the GEMM
    GroupTile gt;
    if (!grouped_tile<GM_TALL>(offsets, n_groups, tiles_n, b, gt)) return;
    const int lane = threadIdx.x & 63;
    const int64_t per_split = (int64_t)n_wg * 4 * GROUPED_TALL_REGS * 64 * 4;      // floats
    const float *base = ws + ((int64_t)(b * 4 + wave) * GROUPED_TALL_REGS * 64 + lane) * 4;
    const int blocks = (gt.m_end - gt.m0 + 31) / 32;                   // 32-row blocks that hold rows
    for (int grp = threadIdx.x >> 6; grp < GROUPED_TALL_REGS && grp / (NB32 * 4) < blocks; grp += 4) {
        const int mb = grp / (NB32 * 4), nb = grp / 4 % NB32, q = grp % 4;
        const int m = gt.m0 + mb * 32 + (lane & 31);
        const int n = gt.tile_n * GN + wave * GN_WAVE + nb * 32 + q * 8 + (lane >> 5) * 4;
        f32x4 a = *(const f32x4 *)(base + (int64_t)grp * 256);
        for (int s = 1; s < splits; s++) a += *(const f32x4 *)(base + (int64_t)s * per_split + (int64_t)grp * 256);
        if (m < gt.m_end && n < N) {
            typedef AT at4 __attribute__((ext_vector_type(4)));
            at4 o;
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = to_at<AT>(a[k]);
            *(at4 *)(y + (int64_t)m * N + n) = o;
        }
    }
}

template <int QT, typename AT>
static int launch_grouped_t(const void *x, const void *const *w, void *y, const int32_t *offsets, int n_groups,
                            int total_rows, int N, int K, const GroupedPlan &plan, float *ws, hipStream_t st) {
    const int tiles_n = (N + GN - 1) / GN, G = K / TILE_COLS;
    const GroupArgs ga = {offsets, (const uint8_t *const *)w, nullptr, n_groups, 0};
    if (!plan.tall) {
        const int grid = tiles_n * grouped_max_row_tiles(total_rows, n_groups, GM);
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32, true>), dim3(grid), dim3(256), 0, st, (const AT *)x,
                           (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
        return 0;
    }
    const int n_wg = tiles_n * grouped_max_row_tiles(total_rows, n_groups, GM_TALL);
    if (plan.splits <= 1) ws = nullptr;
    const int k_steps = ws ? (G + plan.splits - 1) / plan.splits : G;
    const int ny = (G + k_steps - 1) / k_steps;                      // splits that actually hold steps
    hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true>), dim3(n_wg, ny), dim3(256), 0, st, (const AT *)x,
                       (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, k_steps, ws, 0, tiles_n);
    if (ws) {
        hipLaunchKernelGGL((grouped_splitk_reduce_kernel<AT>), dim3((unsigned)(n_wg * 4)), dim3(256), 0, st, ws,
                           (AT *)y, offsets, n_groups, N, tiles_n, n_wg, ny);
    }
    return 0;
}

template <int QT, typename AT>
static int launch_grouped_mlp_t(const void *x, const void *const *wg, const void *const *wu, void *y,
                                const int32_t *offsets, int n_groups, int total_rows, int N, int K, int act,
                                hipStream_t st) {
    const int tiles_n = (N + GN / 2 - 1) / (GN / 2), G = K / TILE_COLS;      // 128 columns of both weights per workgroup
    const GroupArgs ga = {offsets, (const uint8_t *const *)wg, (const uint8_t *const *)wu, n_groups, act};
    const int n_wg = tiles_n * grouped_max_row_tiles(total_rows, n_groups, GM_TALL);
    hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true, true>), dim3(n_wg), dim3(256), 0, st, (const AT *)x,
                       (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
    return 0;
}

// One weight format: y = x w^T per group, or act(x w^T) * (x w_up^T) when w_up is given.
template <int QT>
int launch_grouped_q(const void *x, const void *const *w, const void *const *w_up, void *y, const int32_t *offsets,
                     int n_groups, int total_rows, int dt, int N, int K, int act, const GroupedPlan &plan, float *ws,
                     hipStream_t st) {
    if (dt == DT_F16)
        return w_up ? launch_grouped_mlp_t<QT, _Float16>(x, w, w_up, y, offsets, n_groups, total_rows, N, K, act, st)
                    : launch_grouped_t<QT, _Float16>(x, w, y, offsets, n_groups, total_rows, N, K, plan, ws, st);
    if (dt == DT_BF16)
        return w_up ? launch_grouped_mlp_t<QT, __bf16>(x, w, w_up, y, offsets, n_groups, total_rows, N, K, act, st)
                    : launch_grouped_t<QT, __bf16>(x, w, y, offsets, n_groups, total_rows, N, K, plan, ws, st);
    return -4;
}

}  // namespace lowbit
