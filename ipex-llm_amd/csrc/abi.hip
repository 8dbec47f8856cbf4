// extern "C" surface of liblowbit_hip.so (declared in include/lowbit_abi.h).
#include "../../include/lowbit_abi.h"
#include "lowbit_formats.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

namespace lowbit {
int launch_dequantize_rows(const void *w, const int64_t *rows, int64_t n_rows, void *out, int qtype, int64_t N,
                           int64_t K, int layout, int out_dtype, hipStream_t st);
int launch_mlp_gemv(const void *x, const void *wg, const void *wu, void *y, int qtype, int act_dtype, int M, int N,
                    int K, int act, hipStream_t st);
int launch_mlp_gemm(const void *x, const void *wg, const void *wu, void *y, int qtype, int act_dtype, int M, int N, int K,
                    int act, hipStream_t st);
int launch_moe_gemv(const void *x, const int32_t *ids, const float *route_w, int slots, int n_exp, const void *gates,
                    const void *ups, const void *downs, void *h, void *y, int qtype, int act_dtype, int hidden,
                    int inter, int act, hipStream_t st);
int launch_quantize(const float *src, void *dst, int qtype, int64_t N, int64_t K, int layout, hipStream_t st);
int launch_relayout(const void *src, void *dst, int qtype, int64_t N, int64_t K, int src_layout, hipStream_t st);
int launch_dequantize(const void *w, void *out, int qtype, int64_t N, int64_t K, int layout, int out_dtype,
                      hipStream_t st);
int launch_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                int waves, hipStream_t st);
size_t ring_workspace_bytes(int M, int N, int K, int wgs);
double ring_time_us(int M, int N, int K, int qtype, bool have_ws);
int launch_gemm_ring(const void *x, const void *w, void *y, int qtype, int act_dtype, int M, int N, int K,
                     void *workspace, size_t workspace_bytes, int wgs, hipStream_t st);
int launch_gemm(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                void *workspace, size_t workspace_bytes, int want_splits, hipStream_t st);
int launch_gemm_narrow(const void *x, const void *w, void *y, int qtype, int act_dtype, int M, int N, int K, hipStream_t st);
double narrow_time_us(int M, int N, int K, int qtype);
int gemm_splits(int M, int N, int K, size_t ws_bytes, int qtype);
double gemm_time_us(int M, int N, int K, int splits, int qtype);
int launch_gemv_bf16_f32out(const void *x, const void *w, void *y, int qtype, int layout, int M, int N, int K,
                            hipStream_t st);
int launch_grouped_gemm(const void *x, const void *const *w, const void *const *w_up, void *y, const int32_t *offsets,
                        int n_groups, int total_rows, int qtype, int act_dtype, int N, int K, int act, void *workspace,
                        size_t workspace_bytes, hipStream_t st);
size_t grouped_workspace_bytes(int total_rows, int n_groups, int N, int K);
void grouped_plan_query(int total_rows, int n_groups, int N, int K, size_t ws_bytes, int out[4]);
}  // namespace lowbit

using namespace lowbit;

static thread_local char g_err[512] = "";

static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    return fail(LOWBIT_EHIP, "%s: %s", what, hipGetErrorString(e));
}

static int check_launch(int rc, const char *what) {
    if (rc == -2) return fail(LOWBIT_EQTYPE, "%s: unsupported qtype", what);
    if (rc == -3) return fail(LOWBIT_ESIZE, "%s: tensor too large for one launch", what);
    if (rc == -4) return fail(LOWBIT_EDTYPE, "%s: unsupported element type", what);
    if (rc == -5) return fail(LOWBIT_ESHAPE, "%s: shape cannot be held in the tiled layout", what);
    if (rc != 0) return fail(LOWBIT_EARG, "%s: error %d", what, rc);
    return check_hip(hipGetLastError(), what);
}

static bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

static int check_weight_shape(const char *what, int qtype, int64_t N, int64_t K, int layout) {
    const int qk = qk_size(qtype);
    if (!qk) return fail(LOWBIT_EQTYPE, "%s: unsupported qtype %d", what, qtype);
    if (N < 0 || K < 0) return fail(LOWBIT_EARG, "%s: negative shape", what);
    if (K % qk) return fail(LOWBIT_ESHAPE, "%s: K=%lld is not a multiple of the block size %d", what, (long long)K, qk);
    if (layout != LOWBIT_LAYOUT_GGML && layout != LOWBIT_LAYOUT_TILED)
        return fail(LOWBIT_EARG, "%s: unknown layout %d", what, layout);
    if (layout == LOWBIT_LAYOUT_TILED && N * K != 0 && !lowbit_tileable(qtype, N, K))   // empty: nothing to lay out
        return fail(LOWBIT_ESHAPE, "%s: [%lld, %lld] needs N %% 16 == 0 and K %% 128 == 0 for the tiled layout", what,
                    (long long)N, (long long)K);
    if (N > 0x7fffffff || K > 0x7fffffff) return fail(LOWBIT_ESIZE, "%s: dimension exceeds 2^31", what);
    return 0;
}

extern "C" {

int lowbit_abi_version(void) { return LOWBIT_ABI_VERSION; }

int lowbit_device_info(char *name, size_t name_bytes, int *compute_units, int *shader_clock_khz, int *memory_clock_khz,
                       int *memory_bus_bits) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (int rc = check_hip(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties")) return rc;
    if (name && name_bytes) {
        snprintf(name, name_bytes, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (shader_clock_khz) *shader_clock_khz = prop.clockRate;
    if (memory_clock_khz) *memory_clock_khz = prop.memoryClockRate;
    if (memory_bus_bits) *memory_bus_bits = prop.memoryBusWidth;
    return 0;
}
const char *lowbit_last_error(void) { return g_err; }

size_t ggml_type_size(int qtype) { return (size_t)type_size(qtype); }
int ggml_qk_size(int qtype) { return qk_size(qtype); }

size_t lowbit_blob_bytes(int qtype, int64_t n_weights) {
    const int qk = qk_size(qtype);
    if (!qk || n_weights < 0) return 0;
    return (size_t)(n_weights / qk) * (size_t)type_size(qtype);
}

int lowbit_tileable(int qtype, int64_t N, int64_t K) {
    return qk_size(qtype) != 0 && N > 0 && K > 0 && (N % TILE_ROWS) == 0 && (K % TILE_COLS) == 0;
}

int lowbit_quantize(const float *src, void *dst, int qtype, int64_t N, int64_t K, int layout, void *stream) {
    if (int rc = check_weight_shape("lowbit_quantize", qtype, N, K, layout)) return rc;
    if (N * K == 0) return 0;
    if (!src || !dst || !aligned16(src) || !aligned16(dst))
        return fail(LOWBIT_EARG, "lowbit_quantize: pointers must be non-null and 16-byte aligned");
    return check_launch(launch_quantize(src, dst, qtype, N, K, layout, (hipStream_t)stream), "lowbit_quantize");
}

int lowbit_relayout(const void *src, void *dst, int qtype, int64_t N, int64_t K, int src_layout, void *stream) {
    if (int rc = check_weight_shape("lowbit_relayout", qtype, N, K, LOWBIT_LAYOUT_TILED)) return rc;
    if (src_layout != LOWBIT_LAYOUT_GGML && src_layout != LOWBIT_LAYOUT_TILED)
        return fail(LOWBIT_EARG, "lowbit_relayout: unknown layout %d", src_layout);
    if (!src || !dst || !aligned16(src) || !aligned16(dst))
        return fail(LOWBIT_EARG, "lowbit_relayout: pointers must be non-null and 16-byte aligned");
    const size_t bytes = lowbit_blob_bytes(qtype, N * K);
    const uintptr_t a = (uintptr_t)src, b = (uintptr_t)dst;
    if (a < b + bytes && b < a + bytes) return fail(LOWBIT_EARG, "lowbit_relayout: src and dst overlap");
    return check_launch(launch_relayout(src, dst, qtype, N, K, src_layout, (hipStream_t)stream), "lowbit_relayout");
}

int lowbit_dequantize(const void *w, void *dst, int qtype, int64_t N, int64_t K, int layout, int out_dtype,
                      void *stream) {
    if (int rc = check_weight_shape("lowbit_dequantize", qtype, N, K, layout)) return rc;
    if (N * K == 0) return 0;
    if (!w || !dst || !aligned16(w) || !aligned16(dst))
        return fail(LOWBIT_EARG, "lowbit_dequantize: null or misaligned pointer");
    return check_launch(launch_dequantize(w, dst, qtype, N, K, layout, out_dtype, (hipStream_t)stream),
                        "lowbit_dequantize");
}

static int check_mm(const char *what, const void *x, const void *w, void *y, int qtype, int layout, int act_dtype,
                    int64_t M, int64_t N, int64_t K) {
    if (int rc = check_weight_shape(what, qtype, N, K, layout)) return rc;
    if (M < 0 || M > 0x7fffffff) return fail(LOWBIT_EARG, "%s: bad M", what);
    if (act_dtype != LOWBIT_DT_F16 && act_dtype != LOWBIT_DT_BF16)
        return fail(LOWBIT_EDTYPE, "%s: activations must be f16 or bf16", what);
    if (M * N * K == 0) return 0;
    if (!x || !w || !y || !aligned16(x) || !aligned16(w) || (((uintptr_t)y) & 1))
        return fail(LOWBIT_EARG, "%s: null or misaligned pointer (x, w: 16 bytes)", what);
    if (K % 8) return fail(LOWBIT_ESHAPE, "%s: K must be a multiple of 8", what);
    return 0;
}

int lowbit_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                int64_t K, int waves, void *stream) {
    if (int rc = check_mm("lowbit_gemv", x, w, y, qtype, layout, act_dtype, M, N, K)) return rc;
    if (M * N == 0) return 0;
    if (K == 0) return fail(LOWBIT_ESHAPE, "lowbit_gemv: K == 0");
    return check_launch(launch_gemv(x, w, y, qtype, layout, act_dtype, (int)M, (int)N, (int)K, waves,
                                    (hipStream_t)stream), "lowbit_gemv");
}

int lowbit_gemm_ring(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                     int64_t K, void *workspace, size_t workspace_bytes, int wgs, void *stream) {
    const char *what = "lowbit_gemm_ring";
    if (int rc = check_mm(what, x, w, y, qtype, layout, act_dtype, M, N, K)) return rc;
    if (M * N == 0) return 0;
    if (layout != LOWBIT_LAYOUT_TILED || K < 128) return fail(LOWBIT_ESHAPE, "%s: needs the tiled layout", what);
    if (((uintptr_t)y) & 7) return fail(LOWBIT_EARG, "%s: y must be 8-byte aligned", what);
    if (wgs < 0 || wgs > 65535) return fail(LOWBIT_EARG, "%s: wgs must be 0 (automatic) .. 65535", what);
    if (workspace && !aligned16(workspace)) return fail(LOWBIT_EARG, "%s: workspace must be 16-byte aligned", what);
    return check_launch(launch_gemm_ring(x, w, y, qtype, act_dtype, (int)M, (int)N, (int)K, workspace,
                                         workspace ? workspace_bytes : 0, wgs, (hipStream_t)stream), what);
}

static size_t split_bytes(int64_t M, int64_t N, int splits) {
    return (size_t)splits * (size_t)((M + 127) / 128) * (size_t)((N + 255) / 256) * 128 * 256 * sizeof(float);
}

static int gemm_entry(const char *what, const void *x, const void *w, void *y, int qtype, int layout, int act_dtype,
                      int64_t M, int64_t N, int64_t K, void *workspace, size_t workspace_bytes, int splits,
                      void *stream) {
    if (int rc = check_mm(what, x, w, y, qtype, layout, act_dtype, M, N, K)) return rc;
    if (M * N == 0) return 0;
    if (K == 0) return fail(LOWBIT_ESHAPE, "%s: K == 0", what);
    if (((uintptr_t)y) & 7) return fail(LOWBIT_EARG, "%s: y must be 8-byte aligned", what);     // 8-byte stores at the least
    if (workspace && !aligned16(workspace)) return fail(LOWBIT_EARG, "%s: workspace must be 16-byte aligned", what);
    if (splits < 0 || splits > 64) return fail(LOWBIT_EARG, "%s: splits must be 0 (automatic) .. 64", what);
    if (splits > 1) {
        if (!workspace || split_bytes(M, N, splits) > workspace_bytes)
            return fail(LOWBIT_ESIZE, "%s: %d splits need %zu bytes of workspace", what, splits, split_bytes(M, N, splits));
        if (layout != LOWBIT_LAYOUT_TILED || splits > K / 128)
            return fail(LOWBIT_ESHAPE, "%s: %d splits need the tiled layout and at least as many 128-column steps", what,
                        splits);
    }
    return check_launch(launch_gemm(x, w, y, qtype, layout, act_dtype, (int)M, (int)N, (int)K, workspace,
                                    workspace ? workspace_bytes : 0, splits, (hipStream_t)stream), what);
}

int lowbit_gemm(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                int64_t K, void *stream) {
    return gemm_entry("lowbit_gemm", x, w, y, qtype, layout, act_dtype, M, N, K, nullptr, 0, 0, stream);
}

int lowbit_gemm_ws(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                   int64_t K, void *workspace, size_t workspace_bytes, int splits, void *stream) {
    return gemm_entry("lowbit_gemm_ws", x, w, y, qtype, layout, act_dtype, M, N, K, workspace, workspace_bytes, splits,
                      stream);
}

int lowbit_gemm_narrow(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                       int64_t K, void *stream) {
    const char *what = "lowbit_gemm_narrow";
    if (int rc = check_mm(what, x, w, y, qtype, layout, act_dtype, M, N, K)) return rc;
    if (M * N == 0) return 0;
    if (K == 0) return fail(LOWBIT_ESHAPE, "%s: K == 0", what);
    if (layout != LOWBIT_LAYOUT_TILED) return fail(LOWBIT_ESHAPE, "%s: needs the tiled layout", what);
    if (((uintptr_t)y) & 7) return fail(LOWBIT_EARG, "%s: y must be 8-byte aligned", what);
    return check_launch(launch_gemm_narrow(x, w, y, qtype, act_dtype, (int)M, (int)N, (int)K, (hipStream_t)stream), what);
}

// Row counts up to which lowbit_forward_ws considers the ring kernel (its estimate is fitted up to there): the
// tiled GEMM's half as many dequantizations per MFMA win beyond, except with nf4, whose code-book lookups weigh on
// the GEMM's tighter loop.
static bool ring_range(int qtype, int64_t M) { return M <= (qtype == LOWBIT_QT_NF4 ? 2048 : 256); }

// Choice of kernel behind lowbit_forward: the one with the shortest estimated run time (estimates fitted to
// measurements on MI355X: 640 combinations of format, weight shape and M = 17 .. 768, every kernel and split count
// timed on each; the pick is within 1.5 % of the fastest measured one on average, 21 % at worst).
//   - The GEMV streams the weights once per 16 rows of x: 4.0 TB/s for the 4-bit integer formats, 5.0 for the 8-bit
//     ones, 3.3 for nf4, a pass of fewer rows up to 1.46 times that, plus 3.5 us per pass, and never shorter than
//     its workgroups' walk along K (narrow weights leave CUs idle); the whole scaled by 0.9, see ring_time_us.
//   - The MFMA GEMM amortizes the dequantization over 128 x 256 tiles but is latency-bound while its tiles do not
//     fill the machine.  With a workspace it can split K over more workgroups at the price of writing and
//     re-reading fp32 partial sums (gemm_time_us).
//   - The ring kernel (32 / 64 / 128-row tiles, units dealt out evenly; needs the workspace) covers the batch
//     sizes in between (ring_time_us).
//   - The GEMM in narrow tiles (128 weight rows) doubles the workgroups without partial sums: ahead by 10 - 20 % on
//     small weights ([2048 x 2048], [5632 x 2048], [4096 x 4096]) at a hundred to two thousand rows
//     (narrow_time_us).
enum { PLAN_GEMV = LOWBIT_PLAN_GEMV, PLAN_RING = LOWBIT_PLAN_RING, PLAN_GEMM = LOWBIT_PLAN_GEMM,
       PLAN_GEMM_SPLIT = LOWBIT_PLAN_GEMM_SPLIT, PLAN_GEMM_NARROW = LOWBIT_PLAN_GEMM_NARROW };

static double gemv_time_us(int qtype, int64_t M, int64_t N, int64_t K) {
    const double rate = qtype == LOWBIT_QT_SYM_INT8 || qtype == LOWBIT_QT_FP8_E4M3 ? 5.03e6 : qtype == LOWBIT_QT_NF4 ? 3.31e6 : 3.97e6;
    const double bytes = (double)lowbit_blob_bytes(qtype, N * K);
    const double walk_us = (qtype == LOWBIT_QT_NF4 ? 0.09 : 0.07) * (double)(K / 128);
    double t = 0.0;
    for (int64_t m = M; m > 0; m -= 16) {
        const double rows = m < 16 ? (double)m : 16.0;
        const double stream_us = bytes / (rate * (1.0 + 0.456 * (16.0 - rows) / 16.0));
        t += (stream_us > walk_us ? stream_us : walk_us) + 3.5;
    }
    return 0.9 * t;
}

// which kernel, and for PLAN_GEMM_SPLIT into how many K splits
static int plan_forward(int qtype, int layout, int64_t M, int64_t N, int64_t K, bool have_ws, size_t workspace_bytes,
                        bool y_aligned8, int *splits_out) {
    if (splits_out) *splits_out = 1;
    if (M <= 16 || layout != LOWBIT_LAYOUT_TILED || !y_aligned8) return PLAN_GEMV;            // the MFMA kernels store 8 bytes and more
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff || K < 128) return PLAN_GEMM;     // reports the error
    const int splits = have_ws ? gemm_splits((int)M, (int)N, (int)K, workspace_bytes, qtype) : 1;
    double best_t = gemm_time_us((int)M, (int)N, (int)K, splits, qtype);
    int best = splits > 1 ? PLAN_GEMM_SPLIT : PLAN_GEMM;
    if (M < (1 << 24) && K < (1 << 23)) {        // 24-bit row offsets
        const double t = narrow_time_us((int)M, (int)N, (int)K, qtype);
        if (t < best_t) { best_t = t; best = PLAN_GEMM_NARROW; }
    }
    if (M <= 128) {                              // (beyond that eight and more passes never win)
        const double t = gemv_time_us(qtype, M, N, K);
        if (t < best_t) { best_t = t; best = PLAN_GEMV; }
    }
    if (have_ws && ring_range(qtype, M) && ring_workspace_bytes((int)M, (int)N, (int)K, 0) <= workspace_bytes) {
        const double t = ring_time_us((int)M, (int)N, (int)K, qtype, true);
        if (t < best_t) { best_t = t; best = PLAN_RING; }
    }
    if (best == PLAN_GEMM_SPLIT && splits_out) *splits_out = splits;
    return best;
}

static size_t plan_workspace(int plan, int splits, int64_t M, int64_t N, int64_t K) {
    if (plan == PLAN_RING) return ring_workspace_bytes((int)M, (int)N, (int)K, 0);
    if (plan == PLAN_GEMM_SPLIT) return split_bytes(M, N, splits);
    return 0;
}

size_t lowbit_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 16 || N <= 0 || K < 128 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return 0;   // M <= 16: GEMV
    if (N % 16 || K % 128) return 0;                                                                  // not tileable: GEMV
    // the query carries no qtype: the most that the plan of any format takes when nothing limits it
    size_t most = 0;
    for (const int qt : {LOWBIT_QT_SYM_INT4, LOWBIT_QT_ASYM_INT4, LOWBIT_QT_SYM_INT8, LOWBIT_QT_NF4, LOWBIT_QT_FP8_E4M3}) {
        int splits = 1;
        const int plan = plan_forward(qt, LOWBIT_LAYOUT_TILED, M, N, K, true, (size_t)-1, true, &splits);
        const size_t need = plan_workspace(plan, splits, M, N, K);
        most = need > most ? need : most;
    }
    return most;
}

// What lowbit_forward_ws will use of a workspace of at most max_bytes for this format and shape: the bytes of the
// plan it then picks (0 when that plan leaves no partial tiles).
extern "C" size_t lowbit_workspace_bytes_for(int qtype, int layout, int64_t M, int64_t N, int64_t K, size_t max_bytes) {
    if (!qk_size(qtype) || M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return 0;
    int splits = 1;
    if (max_bytes < 16) return 0;
    switch (plan_forward(qtype, layout, M, N, K, true, max_bytes, true, &splits)) {
    case PLAN_RING: {
        // (a run that cuts no tile needs no bytes, but the plan is only made for a caller that brings a workspace)
        const size_t need = ring_workspace_bytes((int)M, (int)N, (int)K, 0);
        return need ? need : 16;
    }
    case PLAN_GEMM_SPLIT: return split_bytes(M, N, splits);
    default: return 0;
    }
}

extern "C" int lowbit_forward_plan(int qtype, int layout, int64_t M, int64_t N, int64_t K, int have_workspace,
                                   size_t workspace_bytes) {
    if (!qk_size(qtype) || M < 0 || N < 0 || K < 0) return -1;
    return plan_forward(qtype, layout, M, N, K, have_workspace != 0, have_workspace ? workspace_bytes : 0, true, nullptr);
}

static int forward_any(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                       int64_t N, int64_t K, void *workspace, size_t workspace_bytes, void *stream) {
    int splits = 1;
    switch (plan_forward(qtype, layout, M, N, K, workspace != nullptr, workspace_bytes, !(((uintptr_t)y) & 7), &splits)) {
    case PLAN_GEMV: return lowbit_gemv(x, w, y, qtype, layout, act_dtype, M, N, K, 0, stream);
    case PLAN_RING: return lowbit_gemm_ring(x, w, y, qtype, layout, act_dtype, M, N, K, workspace, workspace_bytes, 0, stream);
    case PLAN_GEMM_SPLIT:
        return lowbit_gemm_ws(x, w, y, qtype, layout, act_dtype, M, N, K, workspace, workspace_bytes, splits, stream);
    case PLAN_GEMM_NARROW: return lowbit_gemm_narrow(x, w, y, qtype, layout, act_dtype, M, N, K, stream);
    default: return lowbit_gemm(x, w, y, qtype, layout, act_dtype, M, N, K, stream);
    }
}

int lowbit_forward(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                   int64_t K, void *stream) {
    return forward_any(x, w, y, qtype, layout, act_dtype, M, N, K, nullptr, 0, stream);
}

int lowbit_forward_ws(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                      int64_t K, void *workspace, size_t workspace_bytes, void *stream) {
    if (workspace && !aligned16(workspace))
        return fail(LOWBIT_EARG, "lowbit_forward_ws: workspace must be 16-byte aligned");
    return forward_any(x, w, y, qtype, layout, act_dtype, M, N, K, workspace, workspace ? workspace_bytes : 0, stream);
}

// ---- lowbit_forward_f32: fp32 activations in, fp32 out
//
// The MFMA operands are 16-bit, so x is split into two bf16 planes, hi = bf16(x) and lo = bf16(x - hi)
// (16 mantissa bits together, fp32's exponent range: no overflow whatever the magnitude of x), the product
// runs on the 2M rows with fp32 output and the two halves are added.
__global__ __launch_bounds__(256) void split_bf16_kernel(const float *__restrict__ x, __bf16 *__restrict__ hi,
                                                         __bf16 *__restrict__ lo, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    const __bf16 h = (__bf16)v;                              // round to nearest even
    const float r = v - (float)h;                            // exact: both share the leading bits
    hi[i] = h;
    lo[i] = (r == r && (r - r) == 0.0f) ? (__bf16)r : (__bf16)0.0f;   // inf / nan stay in the hi plane only
}
__global__ __launch_bounds__(256) void add_f32_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                      float *__restrict__ y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = a[i] + b[i];
}

static size_t f32_plane_bytes(int64_t M, int64_t K) { return ((size_t)(2 * M * K * 2) + 255) & ~(size_t)255; }

extern "C" size_t lowbit_forward_f32_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return f32_plane_bytes(M, K) + (size_t)(2 * M * N) * sizeof(float);
}

extern "C" int lowbit_forward_f32(const float *x, const void *w, float *y, int qtype, int layout, int64_t M, int64_t N,
                                  int64_t K, void *workspace, size_t workspace_bytes, void *stream) {
    const char *what = "lowbit_forward_f32";
    if (int rc = check_weight_shape(what, qtype, N, K, layout)) return rc;
    if (M < 0 || M > 0x3fffffff) return fail(LOWBIT_EARG, "%s: bad M", what);
    if (M * N * K == 0) return 0;
    if (!x || !w || !y || !aligned16(x) || !aligned16(w) || (((uintptr_t)y) & 3))
        return fail(LOWBIT_EARG, "%s: null or misaligned pointer (x, w: 16 bytes)", what);
    if (K % 8) return fail(LOWBIT_ESHAPE, "%s: K must be a multiple of 8", what);
    const size_t need = lowbit_forward_f32_workspace_bytes(M, N, K);
    if (!workspace || !aligned16(workspace) || workspace_bytes < need)
        return fail(LOWBIT_ESIZE, "%s: needs %zu bytes of 16-byte aligned workspace", what, need);
    hipStream_t st = (hipStream_t)stream;
    __bf16 *planes = (__bf16 *)workspace;
    float *y2 = (float *)((uint8_t *)workspace + f32_plane_bytes(M, K));
    const int64_t nx = M * K, ny = M * N;
    hipLaunchKernelGGL(split_bf16_kernel, dim3((unsigned)((nx + 255) / 256)), dim3(256), 0, st, x, planes, planes + nx, nx);
    if (int rc = check_launch(launch_gemv_bf16_f32out(planes, w, y2, qtype, layout, (int)(2 * M), (int)N, (int)K, st), what))
        return rc;
    hipLaunchKernelGGL(add_f32_kernel, dim3((unsigned)((ny + 255) / 256)), dim3(256), 0, st, y2, y2 + ny, y, ny);
    return check_hip(hipGetLastError(), what);
}

// ---- lowbit_forward_noalloc: lowbit_forward_ws over a workspace that is part of the library's image.
//
// `scratch` is the HOST-side handle of a device array: host code never passes the name itself to a kernel
// or a copy.  Its device address differs per GPU and is looked up once per device with that device current
// (llama_init_backend does it for device 0, the first call on any other device for that one).
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)64 << 20;
static __device__ __align__(256) uint8_t scratch[NOALLOC_SCRATCH_BYTES];
constexpr int NOALLOC_MAX_DEVICES = 64;
static void *g_scratch_ptr[NOALLOC_MAX_DEVICES];
static std::mutex g_scratch_mu;

// device address of `scratch` on the current device; nullptr (with the error text set) on failure
static void *scratch_of_current_device(const char *what) {
    int dev = -1;
    if (check_hip(hipGetDevice(&dev), what)) return nullptr;
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) {
        fail(LOWBIT_EHIP, "%s: device ordinal %d is beyond the %d this library keeps scratch for", what, dev,
             NOALLOC_MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        if (check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
        if (!p || (((uintptr_t)p) & 255)) {
            fail(LOWBIT_EHIP, "%s: scratch array resolved to a null or misaligned address", what);
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

size_t lowbit_noalloc_scratch_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

int lowbit_forward_noalloc(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                           int64_t N, int64_t K, void *stream) {
    const char *what = "lowbit_forward_noalloc";
    // the same workspace lowbit_forward_ws would be given by a caller that follows lowbit_workspace_bytes
    const size_t need = layout == LOWBIT_LAYOUT_TILED ? lowbit_workspace_bytes(M, N, K) : 0;
    if (need > NOALLOC_SCRATCH_BYTES)
        return fail(LOWBIT_ESIZE, "%s: [%lld x %lld] at M = %lld wants %zu bytes of workspace, the built-in scratch holds "
                    "%zu; use lowbit_forward_ws with a caller-owned workspace", what, (long long)N, (long long)K,
                    (long long)M, need, NOALLOC_SCRATCH_BYTES);
    if (!need) return forward_any(x, w, y, qtype, layout, act_dtype, M, N, K, nullptr, 0, stream);
    void *ws = scratch_of_current_device(what);
    if (!ws) return LOWBIT_EHIP;
    return forward_any(x, w, y, qtype, layout, act_dtype, M, N, K, ws, need, stream);
}

int lowbit_dequantize_rows(const void *w, const int64_t *rows, int64_t n_rows, void *dst, int qtype, int64_t N,
                           int64_t K, int layout, int out_dtype, void *stream) {
    if (int rc = check_weight_shape("lowbit_dequantize_rows", qtype, N, K, layout)) return rc;
    if (n_rows < 0) return fail(LOWBIT_EARG, "lowbit_dequantize_rows: negative row count");
    if (n_rows * K == 0) return 0;
    if (!w || !rows || !dst || !aligned16(w) || !aligned16(dst))
        return fail(LOWBIT_EARG, "lowbit_dequantize_rows: null or misaligned pointer");
    return check_launch(launch_dequantize_rows(w, rows, n_rows, dst, qtype, N, K, layout, out_dtype,
                                               (hipStream_t)stream), "lowbit_dequantize_rows");
}

int lowbit_mlp_forward(const void *x, const void *w_gate, const void *w_up, void *y, int qtype, int act_dtype,
                       int64_t M, int64_t N, int64_t K, int act, void *stream) {
    if (int rc = check_mm("lowbit_mlp_forward", x, w_gate, y, qtype, LOWBIT_LAYOUT_TILED, act_dtype, M, N, K)) return rc;
    if (act != LOWBIT_ACT_SILU && act != LOWBIT_ACT_GELU)
        return fail(LOWBIT_EARG, "lowbit_mlp_forward: activation must be LOWBIT_ACT_SILU or LOWBIT_ACT_GELU");
    if (M * N == 0) return 0;
    if (K == 0) return fail(LOWBIT_ESHAPE, "lowbit_mlp_forward: K == 0");
    if (!w_up || !aligned16(w_up)) return fail(LOWBIT_EARG, "lowbit_mlp_forward: null or misaligned pointer");
    // up to 16 rows (decode): one pass of the streaming kernel over both weights.  17 .. 31 rows: two passes while
    // a weight is small enough for that to beat the GEMM form (measured on MI355X at M = 24: sym_int4 [11008 x 4096],
    // 25 MB a weight, 32.1 against 36.7 us; fp8_e4m3 [14336 x 4096], 61 MB, 53.6 against 47.3; nf4 [28672 x 8192],
    // 125 MB, 152 against 104).  More rows: the fused gate/up form of the tiled MFMA GEMM.
    if (M <= 16 || (M < 32 && lowbit_blob_bytes(qtype, N * K) <= ((size_t)32 << 20)))
        return check_launch(launch_mlp_gemv(x, w_gate, w_up, y, qtype, act_dtype, (int)M, (int)N, (int)K, act,
                                            (hipStream_t)stream), "lowbit_mlp_forward");
    if (((uintptr_t)y) & 7) return fail(LOWBIT_EARG, "lowbit_mlp_forward: y must be 8-byte aligned");
    return check_launch(launch_mlp_gemm(x, w_gate, w_up, y, qtype, act_dtype, (int)M, (int)N, (int)K, act,
                                        (hipStream_t)stream), "lowbit_mlp_forward");
}

int lowbit_moe_forward(const void *x, const int32_t *topk_ids, const float *topk_weight, int top_k, int n_experts,
                       const void *const *gates, const void *const *ups, const void *const *downs, void *workspace,
                       void *y, int qtype, int act_dtype, int64_t hidden, int64_t inter, int act, void *stream) {
    if (int rc = check_weight_shape("lowbit_moe_forward", qtype, inter, hidden, LOWBIT_LAYOUT_TILED)) return rc;
    if (int rc = check_weight_shape("lowbit_moe_forward", qtype, hidden, inter, LOWBIT_LAYOUT_TILED)) return rc;
    if (act_dtype != LOWBIT_DT_F16 && act_dtype != LOWBIT_DT_BF16)
        return fail(LOWBIT_EDTYPE, "lowbit_moe_forward: activations must be f16 or bf16");
    if (act != LOWBIT_ACT_SILU && act != LOWBIT_ACT_GELU)
        return fail(LOWBIT_EARG, "lowbit_moe_forward: activation must be LOWBIT_ACT_SILU or LOWBIT_ACT_GELU");
    if (top_k < 1 || top_k > 64 || top_k * inter > 0x7fffffff || n_experts < 1)
        return fail(LOWBIT_ESIZE, "lowbit_moe_forward: top_k must be 1 .. 64 and n_experts positive");
    if (hidden == 0 || inter == 0) return 0;
    if (!x || !topk_ids || !topk_weight || !gates || !ups || !downs || !workspace || !y || !aligned16(x) ||
        !aligned16(workspace))
        return fail(LOWBIT_EARG, "lowbit_moe_forward: null or misaligned pointer");
    return check_launch(launch_moe_gemv(x, topk_ids, topk_weight, top_k, n_experts, gates, ups, downs, workspace, y, qtype,
                                        act_dtype, (int)hidden, (int)inter, act, (hipStream_t)stream),
                        "lowbit_moe_forward");
}

static int grouped_any(const char *who, const void *x, const void *const *w, const void *const *w_up, void *y,
                       const int32_t *group_offsets, int n_groups, int64_t total_rows, int qtype, int act_dtype, int64_t N,
                       int64_t K, int act, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = check_weight_shape(who, qtype, N, K, LOWBIT_LAYOUT_TILED)) return rc;
    if (n_groups < 0 || total_rows < 0 || total_rows > 0x7fffffff)
        return fail(LOWBIT_EARG, "%s: bad group count or row count", who);
    if (act_dtype != LOWBIT_DT_F16 && act_dtype != LOWBIT_DT_BF16)
        return fail(LOWBIT_EDTYPE, "%s: activations must be f16 or bf16", who);
    if (act != LOWBIT_ACT_SILU && act != LOWBIT_ACT_GELU)
        return fail(LOWBIT_EARG, "%s: activation must be LOWBIT_ACT_SILU or LOWBIT_ACT_GELU", who);
    if (total_rows == 0 || n_groups == 0 || N == 0) return 0;
    if (!x || !w || !y || !group_offsets || !aligned16(x) || (((uintptr_t)y) & 7) || (workspace && !aligned16(workspace)))
        return fail(LOWBIT_EARG, "%s: null or misaligned pointer", who);
    return check_launch(launch_grouped_gemm(x, w, w_up, y, group_offsets, n_groups, (int)total_rows, qtype, act_dtype, (int)N,
                                            (int)K, act, workspace, workspace_bytes, (hipStream_t)stream), who);
}

int lowbit_grouped_forward(const void *x, const void *const *w, void *y, const int32_t *group_offsets, int n_groups,
                           int64_t total_rows, int qtype, int act_dtype, int64_t N, int64_t K, void *stream) {
    return grouped_any("lowbit_grouped_forward", x, w, nullptr, y, group_offsets, n_groups, total_rows, qtype, act_dtype, N, K,
                       LOWBIT_ACT_SILU, nullptr, 0, stream);
}

size_t lowbit_grouped_workspace_bytes(int n_groups, int64_t total_rows, int64_t N, int64_t K) {
    if (n_groups <= 0 || total_rows <= 0 || total_rows > 0x7fffffff || N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff)
        return 0;
    return grouped_workspace_bytes((int)total_rows, n_groups, (int)N, (int)K);
}

int lowbit_grouped_forward_plan(int n_groups, int64_t total_rows, int64_t N, int64_t K, int have_workspace,
                                size_t workspace_bytes, int *plan4) {
    if (!plan4 || n_groups <= 0 || total_rows <= 0 || total_rows > 0x7fffffff || N <= 0 || K < 128 || N > 0x7fffffff ||
        K > 0x7fffffff)
        return fail(LOWBIT_EARG, "lowbit_grouped_forward_plan: bad argument");
    grouped_plan_query((int)total_rows, n_groups, (int)N, (int)K, have_workspace ? workspace_bytes : 0, plan4);
    return 0;
}

int lowbit_grouped_forward_ws(const void *x, const void *const *w, void *y, const int32_t *group_offsets, int n_groups,
                              int64_t total_rows, int qtype, int act_dtype, int64_t N, int64_t K, void *workspace,
                              size_t workspace_bytes, void *stream) {
    return grouped_any("lowbit_grouped_forward_ws", x, w, nullptr, y, group_offsets, n_groups, total_rows, qtype, act_dtype, N,
                       K, LOWBIT_ACT_SILU, workspace, workspace_bytes, stream);
}

int lowbit_grouped_mlp_forward(const void *x, const void *const *w_gate, const void *const *w_up, void *y,
                               const int32_t *group_offsets, int n_groups, int64_t total_rows, int qtype, int act_dtype,
                               int64_t N, int64_t K, int act, void *stream) {
    if (!w_up) return fail(LOWBIT_EARG, "lowbit_grouped_mlp_forward: null pointer");
    return grouped_any("lowbit_grouped_mlp_forward", x, w_gate, w_up, y, group_offsets, n_groups, total_rows, qtype, act_dtype,
                       N, K, act, nullptr, 0, stream);
}

}  // extern "C"

// ---------------------------------------------------------------- host-pointer group

namespace {

struct DevBuf {
    void *p = nullptr;
    ~DevBuf() { if (p) (void)hipFree(p); }
    int alloc(size_t bytes) { return check_hip(hipMalloc(&p, bytes ? bytes : 16), "hipMalloc"); }
};

int host_dequantize(const void *src, void *dst, size_t k, int qtype) {
    const int qk = qk_size(qtype);
    if (!qk) return fail(LOWBIT_EQTYPE, "ggml_dequantize: unsupported qtype %d", qtype);
    if (k % qk) return fail(LOWBIT_ESHAPE, "ggml_dequantize: k not a multiple of %d", qk);
    if (k == 0) return 0;
    const size_t bytes = lowbit_blob_bytes(qtype, (int64_t)k);
    DevBuf w, o;
    if (int rc = w.alloc(bytes)) return rc;
    if (int rc = o.alloc(k * 4)) return rc;
    if (int rc = check_hip(hipMemcpy(w.p, src, bytes, hipMemcpyHostToDevice), "hipMemcpy")) return rc;
    // the ggml layout does not depend on the row length: one block per row
    const int64_t rows = (int64_t)(k / (size_t)qk), cols = qk;
    if (int rc = lowbit_dequantize(w.p, o.p, qtype, rows, cols, LOWBIT_LAYOUT_GGML, LOWBIT_DT_F32, nullptr)) return rc;
    return check_hip(hipMemcpy(dst, o.p, k * 4, hipMemcpyDeviceToHost), "hipMemcpy");
}

}  // namespace

extern "C" {

size_t ggml_quantize_tensor(const float *src, void *dst, int qtype, size_t n, int k, int64_t *hist,
                            bool scale_search) {
    (void)hist;
    g_err[0] = 0;
    if (scale_search) {
        // The search lives in the reference's closed binary and cannot be reproduced.  Its Python caller
        // ignores the return value (low_bit_linear.py:162), so refusing would leave an uninitialised blob
        // in a model: quantize with the plain absmax scale instead and say so once.
        static bool warned = false;
        if (!warned) {
            warned = true;
            fprintf(stderr, "liblowbit_hip: ggml_quantize_tensor: scale_search is not implemented; using the plain block scale\n");
        }
    }
    const int qk = qk_size(qtype);
    if (!qk) { fail(LOWBIT_EQTYPE, "ggml_quantize_tensor: unsupported qtype %d", qtype); return 0; }
    if (k <= 0 || k % qk || n % (size_t)k) { fail(LOWBIT_ESHAPE, "ggml_quantize_tensor: bad n/k"); return 0; }
    if (n == 0) return 0;
    const size_t bytes = lowbit_blob_bytes(qtype, (int64_t)n);
    DevBuf s, d;
    if (s.alloc(n * 4) || d.alloc(bytes)) return 0;
    if (check_hip(hipMemcpy(s.p, src, n * 4, hipMemcpyHostToDevice), "hipMemcpy")) return 0;
    if (lowbit_quantize((const float *)s.p, d.p, qtype, (int64_t)(n / (size_t)k), k, LOWBIT_LAYOUT_GGML, nullptr)) return 0;
    if (check_hip(hipMemcpy(dst, d.p, bytes, hipMemcpyDeviceToHost), "hipMemcpy")) return 0;
    return bytes;
}

void ggml_dequantize_q4_0(const void *src, void *dst, size_t k) {
    g_err[0] = 0;
    (void)host_dequantize(src, dst, k, LOWBIT_QT_SYM_INT4);
}

void ggml_dequantize(const void *src, void *dst, size_t k, int qtype) {
    g_err[0] = 0;
    (void)host_dequantize(src, dst, k, qtype);
}

void ggml_q_format_convet_cpu2xpu(const void *src, void *dst, size_t n, int qtype) {
    g_err[0] = 0;
    const size_t bytes = lowbit_blob_bytes(qtype, (int64_t)n);
    if (!bytes && n) { fail(LOWBIT_EQTYPE, "ggml_q_format_convet_cpu2xpu: unsupported qtype %d", qtype); return; }
    if (src != dst) memmove(dst, src, bytes);
}

void ggml_q_format_convet_xpu2cpu(const void *src, void *dst, size_t n, int qtype) {
    g_err[0] = 0;
    const size_t bytes = lowbit_blob_bytes(qtype, (int64_t)n);
    if (!bytes && n) { fail(LOWBIT_EQTYPE, "ggml_q_format_convet_xpu2cpu: unsupported qtype %d", qtype); return; }
    if (src != dst) memmove(dst, src, bytes);
}

void ggml_compute_forward_mul_mat_q_fp32(const int64_t *src0_ne, const void *src0, int qtype, const int64_t *src1_ne,
                                         const void *src1, void *dst) {
    g_err[0] = 0;
    const int64_t K = src0_ne[0], N = src0_ne[1], M = src1_ne[1];
    if (src1_ne[0] != K) { fail(LOWBIT_ESHAPE, "mul_mat: inner dimensions differ"); return; }
    if (check_weight_shape("ggml_compute_forward_mul_mat_q_fp32", qtype, N, K, LOWBIT_LAYOUT_GGML)) return;
    if (M * N == 0) return;
    const size_t wbytes = lowbit_blob_bytes(qtype, N * K);
    const bool tile = lowbit_tileable(qtype, N, K);
    const size_t ws_bytes = lowbit_forward_f32_workspace_bytes(M, N, K);
    DevBuf w, wt, xf, ws, yf;
    if (w.alloc(wbytes) || xf.alloc((size_t)M * K * 4) || ws.alloc(ws_bytes) || yf.alloc((size_t)M * N * 4)) return;
    if (tile && wt.alloc(wbytes)) return;
    if (check_hip(hipMemcpy(w.p, src0, wbytes, hipMemcpyHostToDevice), "hipMemcpy")) return;
    if (check_hip(hipMemcpy(xf.p, src1, (size_t)M * K * 4, hipMemcpyHostToDevice), "hipMemcpy")) return;
    const void *wdev = w.p;
    int layout = LOWBIT_LAYOUT_GGML;
    if (tile) {
        if (lowbit_relayout(w.p, wt.p, qtype, N, K, LOWBIT_LAYOUT_GGML, nullptr)) return;
        wdev = wt.p;
        layout = LOWBIT_LAYOUT_TILED;
    }
    // fp32 in, fp32 out, as the reference's CPU kernel: nothing is rounded to half precision on the way
    if (lowbit_forward_f32((const float *)xf.p, wdev, (float *)yf.p, qtype, layout, M, N, K, ws.p, ws_bytes, nullptr)) return;
    (void)check_hip(hipMemcpy(dst, yf.p, (size_t)M * N * 4, hipMemcpyDeviceToHost), "hipMemcpy");
}

void llama_init_backend(void) {
    g_err[0] = 0;
    int n = 0;
    if (check_hip(hipGetDeviceCount(&n), "hipGetDeviceCount")) return;
    if (n < 1) { fail(LOWBIT_EHIP, "llama_init_backend: no HIP device"); return; }
    if (check_hip(hipSetDevice(0), "hipSetDevice")) return;
    (void)scratch_of_current_device("llama_init_backend");      // device 0's address of the no-alloc scratch
}


// ------------------------------------------------ symbols the reference resolves but this path does not serve
//
// python/llm/src/ipex_llm/ggml/model/llama/llama_cpp.py touches every one of these at import
// (`_lib.<name>.argtypes = ...`), so a library named by LLAMA_CPP_LIB has to export them or the import
// raises AttributeError.  The quantizers for k-quants and the NPU return 0 bytes written with an error
// text; llama.cpp's model API (tokenizer, eval, sampling, sessions) is not part of a low-bit linear
// library: those stubs say so and abort, the reference's convention for failures inside native code.
size_t ggml_quantize_tensor_with_weights(const float *, void *, int qtype, int, int, int64_t *, const float *) {
    fail(LOWBIT_EQTYPE, "ggml_quantize_tensor_with_weights: importance-weighted (k-quant) quantizers are not implemented (qtype %d)", qtype);
    return 0;
}
size_t ggml_quantize_tensor_rtn(const float *, void *, float *, int qtype, size_t, int, int64_t *, bool) {
    fail(LOWBIT_EQTYPE, "ggml_quantize_tensor_rtn: the NPU quantizer is not implemented (qtype %d)", qtype);
    return 0;
}
size_t ggml_quantize_tensor_rtn_with_weights(const float *, void *, float *, int qtype, size_t, int, int64_t *, bool,
                                             const float *) {
    fail(LOWBIT_EQTYPE, "ggml_quantize_tensor_rtn_with_weights: the NPU quantizer is not implemented (qtype %d)", qtype);
    return 0;
}
[[noreturn]] static void absent(const char *name) {
    fprintf(stderr, "liblowbit_hip: %s is not provided by this library (low-bit linear path only)\n", name);
    abort();
}
// llama_cpp.py:1081 sets a restype on it (and nothing else); no caller in the reference
void ggml_quantize_q4_0(void) { absent("ggml_quantize_q4_0"); }
void llama_apply_lora_from_file(void) { absent("llama_apply_lora_from_file"); }
void llama_context_default_params(void) { absent("llama_context_default_params"); }
void llama_copy_state_data(void) { absent("llama_copy_state_data"); }
void llama_eval(void) { absent("llama_eval"); }
void llama_free(void) { absent("llama_free"); }
void llama_get_embeddings(void) { absent("llama_get_embeddings"); }
void llama_get_kv_cache_token_count(void) { absent("llama_get_kv_cache_token_count"); }
void llama_get_logits(void) { absent("llama_get_logits"); }
void llama_get_state_size(void) { absent("llama_get_state_size"); }
void llama_init_candidates(void) { absent("llama_init_candidates"); }
void llama_init_from_file(void) { absent("llama_init_from_file"); }
void llama_load_session_file(void) { absent("llama_load_session_file"); }
void llama_mlock_supported(void) { absent("llama_mlock_supported"); }
void llama_mmap_supported(void) { absent("llama_mmap_supported"); }
void llama_model_quantize(void) { absent("llama_model_quantize"); }
void llama_n_ctx(void) { absent("llama_n_ctx"); }
void llama_n_embd(void) { absent("llama_n_embd"); }
void llama_n_vocab(void) { absent("llama_n_vocab"); }
void llama_print_system_info(void) { absent("llama_print_system_info"); }
void llama_print_timings(void) { absent("llama_print_timings"); }
void llama_reset_timings(void) { absent("llama_reset_timings"); }
void llama_sample_frequency_and_presence_penalties(void) { absent("llama_sample_frequency_and_presence_penalties"); }
void llama_sample_repetition_penalty(void) { absent("llama_sample_repetition_penalty"); }
void llama_sample_softmax(void) { absent("llama_sample_softmax"); }
void llama_sample_tail_free(void) { absent("llama_sample_tail_free"); }
void llama_sample_temperature(void) { absent("llama_sample_temperature"); }
void llama_sample_token(void) { absent("llama_sample_token"); }
void llama_sample_token_greedy(void) { absent("llama_sample_token_greedy"); }
void llama_sample_token_mirostat(void) { absent("llama_sample_token_mirostat"); }
void llama_sample_token_mirostat_v2(void) { absent("llama_sample_token_mirostat_v2"); }
void llama_sample_top_k(void) { absent("llama_sample_top_k"); }
void llama_sample_top_p(void) { absent("llama_sample_top_p"); }
void llama_sample_typical(void) { absent("llama_sample_typical"); }
void llama_save_session_file(void) { absent("llama_save_session_file"); }
void llama_set_rng_seed(void) { absent("llama_set_rng_seed"); }
void llama_set_state_data(void) { absent("llama_set_state_data"); }
void llama_time_us(void) { absent("llama_time_us"); }
void llama_token_bos(void) { absent("llama_token_bos"); }
void llama_token_eos(void) { absent("llama_token_eos"); }
void llama_token_nl(void) { absent("llama_token_nl"); }
void llama_token_to_str(void) { absent("llama_token_to_str"); }
void llama_tokenize(void) { absent("llama_tokenize"); }

}  // extern "C"
