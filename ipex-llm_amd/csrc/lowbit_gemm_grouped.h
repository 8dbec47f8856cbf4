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
#include "lowbit_grouped_plan.h"

namespace lowbit {

static_assert(G_GN == GN && G_GM_TALL == GM_TALL, "the host-side plan sizes workspaces for the kernel's tiles");
// a workgroup's fp32 partial tile: WAVES waves x (MB32_TALL * 256 / WAVES / 32 * 4) register groups x 64 lanes x 4
static_assert(4 * (MB32_TALL * (GN / 4 / 32) * 4) * 64 * 4 == GM_TALL * GN && 8 * (MB32_TALL * (GN / 8 / 32) * 4) * 64 * 4 == GM_TALL * GN,
              "a split's partial tile is GM_TALL x GN floats with four waves and with eight");


// Sums the fp32 partial tiles of the K splits of a grouped tall launch (register layout: split, workgroup,
// wave, register group, lane) and writes y, rounded once.  One block of 256 threads per (workgroup, wave) of
// the GEMM: its 64 register groups of 64 lanes x 4 floats, four groups at a time; groups of 32-row blocks
// without rows are skipped.
template <typename AT, int WAVES>
__global__ __launch_bounds__(256) void grouped_splitk_reduce_kernel(const float *__restrict__ ws, AT *__restrict__ y,
                                                                    const int32_t *__restrict__ offsets, int n_groups,
                                                                    int N, int tiles_n, int chunk, int n_wg, int splits) {
    constexpr int NBW = GN / WAVES / 32;                               // 32-row weight blocks per wave of the GEMM
    constexpr int REGS = MB32_TALL * NBW * 4;                          // groups of 4 accumulators per lane and wave
    const int b = blockIdx.x / WAVES, wave = blockIdx.x % WAVES;       // workgroup and wave of the GEMM
    GroupTile gt;
    if (!grouped_tile<GM_TALL>(offsets, n_groups, tiles_n, chunk, b, gt)) return;
    const int lane = threadIdx.x & 63;
    const int64_t per_split = (int64_t)n_wg * WAVES * REGS * 64 * 4;   // floats
    const float *base = ws + ((int64_t)(b * WAVES + wave) * REGS * 64 + lane) * 4;
    const int blocks = (gt.m_end - gt.m0 + 31) / 32;                   // 32-row blocks that hold rows
    for (int grp = threadIdx.x >> 6; grp < REGS && grp / (NBW * 4) < blocks; grp += 4) {
        const int mb = grp / (NBW * 4), nb = grp / 4 % NBW, q = grp % 4;
        const int m = gt.m0 + mb * 32 + (lane & 31);
        const int n = gt.tile_n * GN + wave * (GN / WAVES) + nb * 32 + q * 8 + (lane >> 5) * 4;
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
    const int chunk = grouped_chunk(tiles_n, plan.one_round);
    const GroupArgs ga = {offsets, (const uint8_t *const *)w, nullptr, n_groups, 0, 0, chunk};
    if (!plan.tall) {
        const int grid = grouped_grid(grouped_max_row_tiles(total_rows, n_groups, GM), tiles_n, chunk);
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32, true>), dim3(grid), dim3(256), 0, st, (const AT *)x,
                           (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
        return 0;
    }
    const int n_wg = grouped_grid(grouped_max_row_tiles(total_rows, n_groups, GM_TALL), tiles_n, chunk);
    if (plan.splits <= 1) ws = nullptr;
    const int k_steps = ws ? (G + plan.splits - 1) / plan.splits : G;
    const int ny = (G + k_steps - 1) / k_steps;                      // splits that actually hold steps
    // (four waves: the plain product gains nothing from eight, see grouped_waves)
    hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true>), dim3(n_wg, ny), dim3(256), 0, st, (const AT *)x,
                       (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, k_steps, ws, 0, tiles_n);
    if (ws) {
        hipLaunchKernelGGL((grouped_splitk_reduce_kernel<AT, 4>), dim3((unsigned)(n_wg * 4)), dim3(256), 0, st, ws,
                           (AT *)y, offsets, n_groups, N, tiles_n, chunk, n_wg, ny);
    }
    return 0;
}

template <int QT, typename AT>
static int launch_grouped_mlp_t(const void *x, const void *const *wg, const void *const *wu, void *y,
                                const int32_t *offsets, int n_groups, int total_rows, int N, int K, int act,
                                const GroupedPlan &plan, hipStream_t st) {
    const int tiles_n = (N + GN / 2 - 1) / (GN / 2), G = K / TILE_COLS;      // 128 columns of both weights per workgroup
    const int chunk = grouped_chunk(tiles_n, plan.one_round);
    const GroupArgs ga = {offsets, (const uint8_t *const *)wg, (const uint8_t *const *)wu, n_groups, act, 0, chunk};
    const int n_wg = grouped_grid(grouped_max_row_tiles(total_rows, n_groups, GM_TALL), tiles_n, chunk);
    // nf4 always takes the eight-wave form: its two waves per SIMD cover each other's code book reads (the dense
    // tall form gains 5-9 % from it), and with four waves, two weight blocks and the lookups' temporaries the fused
    // kernel sits at the register limit, where the compiler has moved accumulator blocks around inside the loop.
    if (plan.waves == 8 || QT == QT_NF4) {
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true, true, 8>), dim3(n_wg), dim3(512), 0, st, (const AT *)x,
                           (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
        return 0;
    }
    if constexpr (QT != QT_NF4)
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true, true>), dim3(n_wg), dim3(256), 0, st, (const AT *)x,
                           (const uint8_t *)nullptr, (AT *)y, 0, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
    return 0;
}

// The fused gate/up form on a dense gated MLP: y = act(x wg^T) * (x wu^T) for all M rows of x, the two weights
// given directly (no tables in device memory: see GroupArgs).
template <int QT, typename AT>
static int launch_mlp_gemm_t(const void *x, const void *wg, const void *wu, void *y, int M, int N, int K, int act, int waves,
                             bool one_round, hipStream_t st) {
    const int tiles_n = (N + GN / 2 - 1) / (GN / 2), G = K / TILE_COLS;
    const int chunk = grouped_chunk(tiles_n, one_round);
    const GroupArgs ga = {nullptr, nullptr, nullptr, 1, act, 0, chunk, (const uint8_t *)wu};
    const int n_wg = grouped_grid((M + GM_TALL - 1) / GM_TALL, tiles_n, chunk);
    if (waves == 8 || QT == QT_NF4) {                 // (nf4: see launch_grouped_mlp_t)
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true, true, 8>), dim3(n_wg), dim3(512), 0, st, (const AT *)x,
                           (const uint8_t *)wg, (AT *)y, M, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
        return 0;
    }
    if constexpr (QT != QT_NF4)
        hipLaunchKernelGGL((gemm_mfma_kernel<QT, AT, true, MB32_TALL, true, true>), dim3(n_wg), dim3(256), 0, st, (const AT *)x,
                           (const uint8_t *)wg, (AT *)y, M, N, K, 1, ga, G, (float *)nullptr, 0, tiles_n);
    return 0;
}

template <int QT>
int launch_mlp_gemm_q(const void *x, const void *wg, const void *wu, void *y, int dt, int M, int N, int K, int act, int waves,
                      bool one_round, hipStream_t st) {
    if (dt == DT_F16) return launch_mlp_gemm_t<QT, _Float16>(x, wg, wu, y, M, N, K, act, waves, one_round, st);
    if (dt == DT_BF16) return launch_mlp_gemm_t<QT, __bf16>(x, wg, wu, y, M, N, K, act, waves, one_round, st);
    return -4;
}

// One weight format: y = x w^T per group, or act(x w^T) * (x w_up^T) when w_up is given.
template <int QT>
int launch_grouped_q(const void *x, const void *const *w, const void *const *w_up, void *y, const int32_t *offsets,
                     int n_groups, int total_rows, int dt, int N, int K, int act, const GroupedPlan &plan, float *ws,
                     hipStream_t st) {
    if (dt == DT_F16)
        return w_up ? launch_grouped_mlp_t<QT, _Float16>(x, w, w_up, y, offsets, n_groups, total_rows, N, K, act, plan, st)
                    : launch_grouped_t<QT, _Float16>(x, w, y, offsets, n_groups, total_rows, N, K, plan, ws, st);
    if (dt == DT_BF16)
        return w_up ? launch_grouped_mlp_t<QT, __bf16>(x, w, w_up, y, offsets, n_groups, total_rows, N, K, act, plan, st)
                    : launch_grouped_t<QT, __bf16>(x, w, y, offsets, n_groups, total_rows, N, K, plan, ws, st);
    return -4;
}

}  // namespace lowbit
