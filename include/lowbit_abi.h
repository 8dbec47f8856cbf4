/*
 * C ABI of liblowbit_hip.so: ipex-llm's low-bit linear path on one MI355X.
 *
 * Two groups of entry points:
 *
 *  (1) the ggml_* symbols that ipex-llm binds with ctypes
 *      (python/llm/src/ipex_llm/ggml/model/llama/llama_cpp.py:945-1185).  Same
 *      names, argument order and meaning; all pointers are HOST memory, calls
 *      are synchronous, buffers are caller-owned.  The work is staged through
 *      device memory and done by the same kernels as group (2).
 *
 *  (2) lowbit_* device entry points for callers that already hold device
 *      memory: what ipex-llm reaches through the torch ops of xe_linear /
 *      xe_batch (python/llm/src/ipex_llm/transformers/xpu_ops.py:23-62).  Plain
 *      device pointers, sizes and a hipStream_t passed as void*; work is
 *      enqueued on that stream and the call returns without synchronizing.
 *
 * Every lowbit_* function returns 0 on success or a negative LOWBIT_E* code;
 * lowbit_last_error() then describes the failure (thread-local).
 *
 * qtype values follow ipex_llm.ggml.quantize.ggml_tensor_qtype
 * (python/llm/src/ipex_llm/ggml/quantize.py:28-57).
 */
#ifndef LOWBIT_ABI_H
#define LOWBIT_ABI_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LOWBIT_ABI_VERSION 1

/* qtypes */
#define LOWBIT_QT_SYM_INT4 2   /* ggml Q4_0 */
#define LOWBIT_QT_ASYM_INT4 3  /* ggml Q4_1 */
#define LOWBIT_QT_SYM_INT8 8   /* ggml Q8_0 */
#define LOWBIT_QT_NF4 10
#define LOWBIT_QT_FP8_E4M3 15

/* weight layouts: GGML = the CPU blob of the reference; TILED = 16x128 tiles for the MFMA
 * kernels (needs N % 16 == 0 and K % 128 == 0).  Both have the same byte count. */
#define LOWBIT_LAYOUT_GGML 0
#define LOWBIT_LAYOUT_TILED 1

/* activation / output element types */
#define LOWBIT_DT_F16 0
#define LOWBIT_DT_BF16 1
#define LOWBIT_DT_F32 2

/* activation of the gate branch in lowbit_mlp_forward (values of SILU / GELU in
 * python/llm/src/ipex_llm/transformers/models/utils.py:30-31) */
#define LOWBIT_ACT_SILU 0
#define LOWBIT_ACT_GELU 1  /* tanh form, as in Gemma */

/* error codes */
#define LOWBIT_OK 0
#define LOWBIT_EARG (-1)     /* null / misaligned pointer, negative size */
#define LOWBIT_EQTYPE (-2)   /* qtype outside {2,3,8,10,15} */
#define LOWBIT_ESIZE (-3)    /* size too large for one launch */
#define LOWBIT_EDTYPE (-4)   /* element type not supported by this entry point */
#define LOWBIT_ESHAPE (-5)   /* K not a multiple of the block, or shape not tileable */
#define LOWBIT_EHIP (-6)     /* HIP runtime error (no device, launch failure, ...) */

int lowbit_abi_version(void);
const char *lowbit_last_error(void);
/* What the HIP runtime reports for the current device: marketing and architecture name, number of CUs, maximum
 * shader and memory clocks (kHz), memory bus width (bits).  For benchmark reports; any pointer may be null. */
int lowbit_device_info(char *name, size_t name_bytes, int *compute_units, int *shader_clock_khz, int *memory_clock_khz,
                       int *memory_bus_bits);

/* ------------------------------------------------------------------ (1) */

/* llama_cpp.py:946-967; called from low_bit_linear.py:162.  n = number of weights, k = row
 * length.  hist is ignored (the reference never reads it back, low_bit_linear.py:145);
 * scale_search = true (the closed binary's search for a better block scale) is not implemented: the
 * plain block scale is used and a warning goes to stderr once.  Returns bytes written, 0 on failure. */
size_t ggml_quantize_tensor(const float *src, void *dst, int qtype, size_t n, int k, int64_t *hist,
                            bool scale_search);
/* llama_cpp.py:1050-1056 and :1059-1065.  0 for a qtype this library does not implement. */
size_t ggml_type_size(int qtype);
int ggml_qk_size(int qtype);
/* llama_cpp.py:1068-1081 and :1084-1099; called from low_bit_linear.py:245,258.
 * k = number of weights to produce (fp32). */
void ggml_dequantize_q4_0(const void *src, void *dst, size_t k);
void ggml_dequantize(const void *src, void *dst, size_t k, int qtype);
/* llama_cpp.py:1102-1135; called from low_bit_linear.py:203,232.  These carry no row length,
 * so they cannot build the tiled layout: they copy the blob unchanged, and the result is a
 * valid device weight in LOWBIT_LAYOUT_GGML (served by the slower any-shape kernels).
 * Callers that know the shape use lowbit_relayout instead. */
void ggml_q_format_convet_cpu2xpu(const void *src, void *dst, size_t n, int qtype);
void ggml_q_format_convet_xpu2cpu(const void *src, void *dst, size_t n, int qtype);
/* llama_cpp.py:1154-1185; called from low_bit_linear.py:487.  ne = {K, rows} (ggml order),
 * src0 = ggml blob [N, K], src1 = fp32 [M, K], dst = fp32 [M, N].  Runs lowbit_forward_f32 on the device:
 * activations keep 16 mantissa bits and fp32's range (the reference rounds them to int8 blocks), the
 * result is never rounded to half precision. */
void ggml_compute_forward_mul_mat_q_fp32(const int64_t *src0_ne, const void *src0, int qtype,
                                         const int64_t *src1_ne, const void *src1, void *dst);
/* llama_cpp.py:1189-1193.  Selects device 0 and loads the kernels. */
void llama_init_backend(void);

/* llama_cpp.py:970-1047: quantizers for k-quants (importance weights) and for the NPU.  Not implemented:
 * they return 0 bytes written and leave a text for lowbit_last_error(). */
size_t ggml_quantize_tensor_with_weights(const float *src, void *dst, int qtype, int nrow, int n_per_row, int64_t *hist,
                                         const float *weights);
size_t ggml_quantize_tensor_rtn(const float *src, void *dst, float *scale, int qtype, size_t n, int k, int64_t *hist,
                                bool scale_search);
size_t ggml_quantize_tensor_rtn_with_weights(const float *src, void *dst, float *scale, int qtype, size_t n, int k,
                                             int64_t *hist, bool scale_search, const float *weights);
/* llama_cpp.py:1081 resolves this name (a restype assignment, no prototype, no caller).  Placeholder that aborts. */
void ggml_quantize_q4_0(void);
/* The library also exports the 45 names of llama.cpp's model API that llama_cpp.py:228-940 resolves at import
 * (llama_eval, llama_tokenize, ...), so that the import succeeds with LLAMA_CPP_LIB pointing here.  They are outside
 * the low-bit linear path and are not part of this interface: no prototypes are given, and each prints its name
 * and aborts when called (abi.hip). */

/* ------------------------------------------------------------------ (2) */

/* Bytes of a blob holding n_weights weights; 0 for an unknown qtype. */
size_t lowbit_blob_bytes(int qtype, int64_t n_weights);
/* 1 when [N, K] can be held in LOWBIT_LAYOUT_TILED. */
int lowbit_tileable(int qtype, int64_t N, int64_t K);

/* ggml_quantize_tensor on device memory: src fp32 [N, K] -> dst blob in `layout`. */
int lowbit_quantize(const float *src, void *dst, int qtype, int64_t N, int64_t K, int layout, void *stream);
/* ggml_q_format_convet_cpu2xpu / _xpu2cpu with the shape: src in `src_layout` -> dst in the
 * other layout.  src and dst must not overlap. */
int lowbit_relayout(const void *src, void *dst, int qtype, int64_t N, int64_t K, int src_layout, void *stream);
/* xe_linear.dequant (low_bit_linear.py:534-538) / ggml_dequantize: blob -> dense [N, K].  dst is
 * 16-byte aligned (so is dst of lowbit_dequantize_rows). */
int lowbit_dequantize(const void *w, void *dst, int qtype, int64_t N, int64_t K, int layout, int out_dtype,
                      void *stream);
/* xe_linear.forward_new / xe_batch.batch_forward (low_bit_linear.py:657-668, xpu_ops.py:23-26):
 * y[M, N] = x[M, K] * dequant(w)[N, K]^T, x and y of act_dtype (f16 or bf16), fp32 accumulation.
 * Picks the streaming GEMV (one pass over the weights per 16 rows) or the MFMA GEMM, whichever it
 * estimates to be faster for the shape. */
int lowbit_forward(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                   int64_t N, int64_t K, void *stream);
/* Which kernel lowbit_forward (have_workspace = 0) or lowbit_forward_ws (a non-null workspace of
 * workspace_bytes) runs for a shape with an 8-byte aligned y, without running anything: the streaming GEMV in 16-row passes, the ring kernel for batch
 * sizes, or the MFMA GEMM with or without a K split or in narrow tiles.  Negative for an unknown qtype.  Host arithmetic only. */
#define LOWBIT_PLAN_GEMV 0
#define LOWBIT_PLAN_RING 1
#define LOWBIT_PLAN_GEMM 2
#define LOWBIT_PLAN_GEMM_SPLIT 3
#define LOWBIT_PLAN_GEMM_NARROW 4  /* the MFMA GEMM in tiles of 128 weight rows (lowbit_gemm_narrow) */
/* What lowbit_forward_ws makes use of when the caller can spare at most max_bytes of workspace for this format
 * and shape: the size of the partial tiles of the plan it then picks, 0 when that plan has none.  A caller
 * with a budget asks this instead of capping lowbit_workspace_bytes (which carries no format and returns the most
 * any format could use): what it passes on is then exactly what the plan was made for. */
size_t lowbit_workspace_bytes_for(int qtype, int layout, int64_t M, int64_t N, int64_t K, size_t max_bytes);
int lowbit_forward_plan(int qtype, int layout, int64_t M, int64_t N, int64_t K, int have_workspace,
                        size_t workspace_bytes);
/* The two kernels behind lowbit_forward, for callers (and benchmarks) that choose themselves.
 * waves = 0 lets the library pick the workgroup size of the GEMV.  lowbit_gemm needs y 8-byte aligned
 * (lowbit_forward sends any other y through the GEMV) and is at its best with y 16-byte aligned: it
 * then stores whole cache lines. */
int lowbit_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                int64_t N, int64_t K, int waves, void *stream);
int lowbit_gemm(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                int64_t N, int64_t K, void *stream);
/* The MFMA GEMM in tiles of 128 rows of x by 128 weight rows (64 by 128 while those are no more than one per
 * compute unit) instead of 128 by 256: twice the workgroups for a product whose wider tiles leave compute
 * units idle, without the partial sums of a K split.  Tiled layout, y 8-byte aligned.  (Same reference
 * call as lowbit_forward: low_bit_linear.py:657-668.) */
int lowbit_gemm_narrow(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                       int64_t N, int64_t K, void *stream);

/* xe_linear.dequantize_rows (python/llm/src/ipex_llm/transformers/embedding.py:218-221; signature
 * xpu_ops.py:59-62): dst[i, :] = dequant(w)[rows[i], :] for i < n_rows, rows = int64 indices in
 * device memory; an index outside [0, N) yields zeros.  dst is [n_rows, K] of out_dtype. */
int lowbit_dequantize_rows(const void *w, const int64_t *rows, int64_t n_rows, void *dst, int qtype, int64_t N,
                           int64_t K, int layout, int out_dtype, void *stream);
/* xe_linear.mlp_forward_xpu (python/llm/src/ipex_llm/transformers/models/common.py:145-158; signature
 * xpu_ops.py:34-37): y[M, N] = act(x * Wg^T) .* (x * Wu^T) in one launch, both weights tiled [N, K].
 * Any M (the reference fuses at M == 1 only, models/utils.py:246-259): up to 16 rows run the streaming
 * kernel (one pass over both weights; two passes up to 31 rows while a weight has at most 32 MiB), more
 * rows the fused gate/up form of the tiled GEMM (y 8-byte aligned, M < 2^24, K < 2^23). */
int lowbit_mlp_forward(const void *x, const void *w_gate, const void *w_up, void *y, int qtype, int act_dtype,
                       int64_t M, int64_t N, int64_t K, int act, void *stream);

/* xe_linear.moe_forward_vec (python/llm/src/ipex_llm/transformers/models/deepseek.py:290-315): one
 * token through its top_k experts without the host reading the routing result.
 * y[hidden] = sum_j topk_weight[j] * down[e_j](act(gate[e_j] x) .* up[e_j] x), e_j = topk_ids[j].
 * topk_ids (int32, clamped to [0, n_experts)), topk_weight (fp32) and the three pointer tables (one tiled weight per expert,
 * gate / up [inter, hidden], down [hidden, inter]) live in DEVICE memory; workspace is caller-owned
 * device memory of top_k * inter activations (16-byte aligned).  Two launches on `stream`. */
int lowbit_moe_forward(const void *x, const int32_t *topk_ids, const float *topk_weight, int top_k, int n_experts,
                       const void *const *gates, const void *const *ups, const void *const *downs, void *workspace,
                       void *y, int qtype, int act_dtype, int64_t hidden, int64_t inter, int act, void *stream);

/* The same products with a caller-owned workspace in device memory (16-byte aligned): the GEMM may
 * then split K over more workgroups and sum fp32 partial tiles from the workspace in a second launch,
 * which fills the machine when M is small or N narrow.  No counterpart in the reference (its closed
 * kernels manage their own memory); lowbit_workspace_bytes says how much is worth passing for a
 * shape (0: the workspace would not be used).  A smaller or null workspace is always valid. */
size_t lowbit_workspace_bytes(int64_t M, int64_t N, int64_t K);
int lowbit_forward_ws(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                      int64_t N, int64_t K, void *workspace, size_t workspace_bytes, void *stream);
/* splits: 0 = the library's choice for the workspace given, n > 1 = exactly n K-splits (needs
 * n * ceil(M/128) * ceil(N/256) * 128 KiB of workspace), 1 = none. */
int lowbit_gemm_ws(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                   int64_t K, void *workspace, size_t workspace_bytes, int splits, void *stream);

/* fp32 activations in, fp32 out: what xe_linear.forward_new / xe_batch.batch_forward compute when LowBitLinear
 * hands them a float x (python/llm/src/ipex_llm/transformers/low_bit_linear.py:657-668: only M > 1 with
 * conver_to_half casts to half first) and what the CPU branch's ggml_compute_forward_mul_mat_q_fp32 returns.
 * x is split into two bf16 planes (16 mantissa bits, fp32's exponent range), the product of the 2M rows is
 * accumulated and stored in fp32 and the halves are added.  The streaming kernel serves every M (16 rows of
 * the planes per pass over the weights): meant for decode and small batches.  workspace: caller-owned device
 * memory of lowbit_forward_f32_workspace_bytes(M, N, K) bytes, 16-byte aligned. */
size_t lowbit_forward_f32_workspace_bytes(int64_t M, int64_t N, int64_t K);
int lowbit_forward_f32(const float *x, const void *w, float *y, int qtype, int layout, int64_t M, int64_t N, int64_t K,
                       void *workspace, size_t workspace_bytes, void *stream);

/* lowbit_forward_ws without a workspace argument and without any allocation: the partial tiles go to a
 * scratch array that is part of the library's image on every GPU (lowbit_noalloc_scratch_bytes() = 64 MiB,
 * held by each GPU the library runs on until the process ends).  No counterpart in the reference; it is for
 * callers that cannot allocate device memory: code under HIP-graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  Same result as lowbit_forward_ws given lowbit_workspace_bytes(M, N, K) bytes; a
 * shape that asks for more than the scratch holds fails with LOWBIT_ESIZE.  The call neither allocates nor
 * frees (the scratch address is looked up once per device: by llama_init_backend for device 0, by the first
 * call made with another device current for that device).  All calls on one GPU share the array: calls that
 * overlap in time on one GPU (two streams) race on it - serialize them or use lowbit_forward_ws. */
size_t lowbit_noalloc_scratch_bytes(void);
int lowbit_forward_noalloc(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M,
                           int64_t N, int64_t K, void *stream);

/* The kernel lowbit_forward_ws picks for M of a few dozen to a few hundred rows (tiled layout, y
 * 8-byte aligned): 128 / 64 / 32 rows of x by 256 weight rows per workgroup, the (tile, K-step) units
 * dealt out in equal runs over `wgs` workgroups (0 = the library's choice), partial tiles summed from
 * the workspace.  A null or too small workspace is valid: tiles are then not cut along K. */
int lowbit_gemm_ring(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int64_t M, int64_t N,
                     int64_t K, void *workspace, size_t workspace_bytes, int wgs, void *stream);

/* Grouped product for mixture-of-experts layers, one launch for all experts.  The reference has
 * no single call for it: it loops over the experts in Python and calls each expert's LowBitLinear
 * on the rows routed to it (python/llm/src/ipex_llm/transformers/models/qwen2_moe.py:375-430 is the
 * pattern).  Rows group_offsets[e] .. group_offsets[e+1]-1 of x [total_rows, K] are multiplied by
 * the tiled weight w[e] [N, K]; y is [total_rows, N].  w (n_groups device pointers) and
 * group_offsets (n_groups + 1 int32, ascending, group_offsets[n_groups] <= total_rows) live in
 * DEVICE memory; total_rows is the host-side row count the grid is sized from. */
int lowbit_grouped_forward(const void *x, const void *const *w, void *y, const int32_t *group_offsets,
                           int n_groups, int64_t total_rows, int qtype, int act_dtype, int64_t N, int64_t K,
                           void *stream);
/* The same with a workspace (caller-owned device memory, 16-byte aligned, lowbit_grouped_workspace_bytes(...)
 * bytes; null / 0 is valid): when the output alone has too few tiles for the machine - few columns, long K, the
 * down projection of an expert - K is split over a second grid dimension and the fp32 partial tiles are summed
 * from the workspace by a second kernel.  lowbit_grouped_workspace_bytes returns 0 for shapes that do not split. */
size_t lowbit_grouped_workspace_bytes(int n_groups, int64_t total_rows, int64_t N, int64_t K);
int lowbit_grouped_forward_ws(const void *x, const void *const *w, void *y, const int32_t *group_offsets,
                              int n_groups, int64_t total_rows, int qtype, int act_dtype, int64_t N, int64_t K,
                              void *workspace, size_t workspace_bytes, void *stream);
/* Host arithmetic only (no GPU call, like lowbit_forward_plan): how lowbit_grouped_forward(_ws) would run the
 * shape.  plan4 = {256-row tiles (1) or 128-row tiles (0), K splits, waves per workgroup, workgroups per split}.
 * Every workgroup of a split launch owns one 256 x 256 fp32 tile of the workspace: splits x workgroups x 256 KiB
 * never exceeds lowbit_grouped_workspace_bytes.  No counterpart in the reference (its expert loop has no plan). */
int lowbit_grouped_forward_plan(int n_groups, int64_t total_rows, int64_t N, int64_t K, int have_workspace,
                                size_t workspace_bytes, int *plan4);
/* The gated MLP's first half for all experts in one launch: rows of group e of y [total_rows, N] =
 * act(x w_gate[e]^T) .* (x w_up[e]^T), act as in lowbit_mlp_forward.  It is what the per-expert loop computes
 * with two LowBitLinear calls and an activation per expert
 * (python/llm/src/ipex_llm/transformers/models/qwen2_moe.py:375-430 calling the expert MLP of
 * models/common.py:145-158), without the gate and up products ever leaving the registers.  w_gate / w_up /
 * group_offsets as in lowbit_grouped_forward. */
int lowbit_grouped_mlp_forward(const void *x, const void *const *w_gate, const void *const *w_up, void *y,
                               const int32_t *group_offsets, int n_groups, int64_t total_rows, int qtype,
                               int act_dtype, int64_t N, int64_t K, int act, void *stream);

#ifdef __cplusplus
}
#endif
#endif
