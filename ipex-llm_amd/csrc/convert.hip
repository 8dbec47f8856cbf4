// Layout conversion (ggml <-> tiled) and full dequantization.
//
// relayout replaces ggml_q_format_convet_cpu2xpu / _xpu2cpu
// (python/llm/src/ipex_llm/transformers/low_bit_linear.py:178-233); dequantize
// replaces ggml_dequantize / ggml_dequantize_q4_0 (low_bit_linear.py:236-259)
// and xe_linear.dequant (low_bit_linear.py:534-538).  Both are one-off,
// HBM-bound passes: one thread moves one 32-column sub-block.
#include "lowbit_formats.h"

namespace lowbit {

template <int QT, int SRC_LAYOUT>
__global__ __launch_bounds__(256) void relayout_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                       int64_t N, int64_t K) {
    using F = Fmt<QT>;
    constexpr int SPB = F::QK / 32;
    const int64_t sbpr = K / 32;                               // sub-blocks per row
    if constexpr (QT == QT_NF4 && SRC_LAYOUT == LAYOUT_TILED) {
        // a ggml nf4 byte mixes both halves of a 64-block: one thread moves a whole block
        const int64_t blk = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (blk >= N * (K / 64)) return;
        const int64_t n = blk / (K / 64);
        const int kb = (int)(blk % (K / 64));
        SubBlock a, b;
        tiled_load_sub<QT>(src, n, K, kb * 2, a);
        tiled_load_sub<QT>(src, n, K, kb * 2 + 1, b);
        uint8_t code64[64];
        for (int i = 0; i < 32; i++) { code64[i] = a.code[i]; code64[32 + i] = b.code[i]; }
        ggml_store_nf4_block(dst, blk, code64, a.hdr);
    } else {
        const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (t >= N * sbpr) return;
        const int64_t n = t / sbpr;
        const int sb = (int)(t % sbpr);
        SubBlock s;
        if constexpr (SRC_LAYOUT == LAYOUT_GGML) {
            ggml_load_sub<QT>(src, n, K, sb, s);
            tiled_store_codes<QT>(dst, n, K, sb, s.code);
            if (sb % SPB == 0) tiled_store_hdr<QT>(dst, n, K, sb, s.hdr);
        } else {
            tiled_load_sub<QT>(src, n, K, sb, s);
            ggml_store_sub<QT>(dst, n, K, sb, s.code, s.hdr);
        }
    }
}

template <int QT> static int launch_rl(const void *src, void *dst, int64_t N, int64_t K, int src_layout, hipStream_t st) {
    int64_t threads = N * (K / 32);
    if (QT == QT_NF4 && src_layout == LAYOUT_TILED) threads = N * (K / 64);
    if (threads == 0) return 0;
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7fffffff) return -3;
    if (src_layout == LAYOUT_GGML)
        hipLaunchKernelGGL((relayout_kernel<QT, LAYOUT_GGML>), dim3((unsigned)grid), dim3(256), 0, st,
                           (const uint8_t *)src, (uint8_t *)dst, N, K);
    else
        hipLaunchKernelGGL((relayout_kernel<QT, LAYOUT_TILED>), dim3((unsigned)grid), dim3(256), 0, st,
                           (const uint8_t *)src, (uint8_t *)dst, N, K);
    return 0;
}

int launch_relayout(const void *src, void *dst, int qtype, int64_t N, int64_t K, int src_layout, hipStream_t st) {
    switch (qtype) {
    case QT_SYM_INT4: return launch_rl<QT_SYM_INT4>(src, dst, N, K, src_layout, st);
    case QT_ASYM_INT4: return launch_rl<QT_ASYM_INT4>(src, dst, N, K, src_layout, st);
    case QT_SYM_INT8: return launch_rl<QT_SYM_INT8>(src, dst, N, K, src_layout, st);
    case QT_NF4: return launch_rl<QT_NF4>(src, dst, N, K, src_layout, st);
    case QT_FP8_E4M3: return launch_rl<QT_FP8_E4M3>(src, dst, N, K, src_layout, st);
    default: return -2;
    }
}

// ------------------------------------------------------------ dequantize

template <typename T> __device__ inline T from_f32(float v);
template <> __device__ inline float from_f32<float>(float v) { return v; }
template <> __device__ inline _Float16 from_f32<_Float16>(float v) { return (_Float16)v; }
template <> __device__ inline __bf16 from_f32<__bf16>(float v) { return (__bf16)v; }

template <int QT, int LAYOUT, typename OT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t *__restrict__ w, OT *__restrict__ out,
                                                      int64_t n_out, int64_t N, int64_t K,
                                                      const int64_t *__restrict__ rows) {
    // rows == nullptr: output row i is weight row i.  Otherwise output row i is weight row rows[i]
    // (xe_linear.dequantize_rows, python/llm/src/ipex_llm/transformers/embedding.py:218-221); an
    // index outside [0, N) gives a row of zeros.
    // Every lane produces 16 bytes of output (4 fp32 or 8 16-bit columns) and loads only the bytes
    // that hold its own codes; adjacent lanes cover adjacent columns, so a wave stores 1 KiB runs.
    constexpr int CPL = 16 / (int)sizeof(OT), LPS = 32 / CPL;  // columns per lane, lanes per sub-block
    __shared__ float cb[16];
    if constexpr (QT == QT_NF4) {
        // divergent lookups: LDS serves them at full rate, the constant cache does not
        if (threadIdx.x < 16) cb[threadIdx.x] = NF4_CODEBOOK[threadIdx.x];
        __syncthreads();
    }
    const int64_t sbpr = K / 32;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_out * sbpr * LPS) return;
    int lp = (int)(t % LPS);
    int64_t i_out = (t / LPS) / sbpr;
    int sb = (int)((t / LPS) % sbpr);
    if constexpr (LAYOUT == LAYOUT_TILED && sizeof(OT) == 2) {
        if (!rows) {
            // whole matrix, 16-bit output: a workgroup covers one 16 x 128 tile, so that each line of
            // the tile is fetched by one compute unit only (fp32 output measured no gain from it)
            const int64_t wg_per_band = K / (16 * CPL);
            const int64_t col = (blockIdx.x % wg_per_band) * (16 * CPL) + (threadIdx.x % 16) * CPL;
            i_out = (blockIdx.x / wg_per_band) * TILE_ROWS + threadIdx.x / 16;
            sb = (int)(col / 32);
            lp = (int)(col % 32) / CPL;
        }
    }
    const int64_t n = rows ? rows[i_out] : i_out;
    typedef OT otv __attribute__((ext_vector_type(CPL)));
    otv v;
#pragma unroll
    for (int i = 0; i < CPL; i++) v[i] = from_f32<OT>(0.0f);
    if (n >= 0 && n < N) {
#pragma unroll
        for (int q = 0; q < CPL / 4; q++) {
            uint32_t code[4], hdr;
            const int part = lp * (CPL / 4) + q;
            if constexpr (LAYOUT == LAYOUT_GGML) ggml_load4<QT>(w, n, K, sb, part, code, hdr);
            else tiled_load4<QT>(w, n, K, sb, part, code, hdr);
            float d, m;
            hdr_to_scale<QT>(hdr, d, m);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if constexpr (QT == QT_NF4) v[q * 4 + i] = from_f32<OT>(cb[code[i]] * d);
                else v[q * 4 + i] = from_f32<OT>(decode<QT>(code[i], d, m));
            }
        }
    }
    *(otv *)(out + i_out * K + (int64_t)sb * 32 + lp * CPL) = v;
}

template <int QT, typename OT>
static int launch_dq2(const void *w, void *out, int64_t N, int64_t K, int layout, hipStream_t st, const int64_t *rows,
                      int64_t n_rows) {
    const int64_t n_out = rows ? n_rows : N;
    const int64_t threads = n_out * (K / 32) * (2 * (int64_t)sizeof(OT));  // one lane per 16 output bytes
    if (threads == 0) return 0;
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7fffffff) return -3;
    if (layout == LAYOUT_GGML)
        hipLaunchKernelGGL((dequant_kernel<QT, LAYOUT_GGML, OT>), dim3((unsigned)grid), dim3(256), 0, st,
                           (const uint8_t *)w, (OT *)out, n_out, N, K, rows);
    else
        hipLaunchKernelGGL((dequant_kernel<QT, LAYOUT_TILED, OT>), dim3((unsigned)grid), dim3(256), 0, st,
                           (const uint8_t *)w, (OT *)out, n_out, N, K, rows);
    return 0;
}

template <int QT>
static int launch_dq(const void *w, void *out, int64_t N, int64_t K, int layout, int dt, hipStream_t st,
                     const int64_t *rows, int64_t n_rows) {
    switch (dt) {
    case DT_F16: return launch_dq2<QT, _Float16>(w, out, N, K, layout, st, rows, n_rows);
    case DT_BF16: return launch_dq2<QT, __bf16>(w, out, N, K, layout, st, rows, n_rows);
    case DT_F32: return launch_dq2<QT, float>(w, out, N, K, layout, st, rows, n_rows);
    default: return -4;
    }
}

int launch_dequantize_rows(const void *w, const int64_t *rows, int64_t n_rows, void *out, int qtype, int64_t N,
                           int64_t K, int layout, int out_dtype, hipStream_t st) {
    switch (qtype) {
    case QT_SYM_INT4: return launch_dq<QT_SYM_INT4>(w, out, N, K, layout, out_dtype, st, rows, n_rows);
    case QT_ASYM_INT4: return launch_dq<QT_ASYM_INT4>(w, out, N, K, layout, out_dtype, st, rows, n_rows);
    case QT_SYM_INT8: return launch_dq<QT_SYM_INT8>(w, out, N, K, layout, out_dtype, st, rows, n_rows);
    case QT_NF4: return launch_dq<QT_NF4>(w, out, N, K, layout, out_dtype, st, rows, n_rows);
    case QT_FP8_E4M3: return launch_dq<QT_FP8_E4M3>(w, out, N, K, layout, out_dtype, st, rows, n_rows);
    default: return -2;
    }
}

int launch_dequantize(const void *w, void *out, int qtype, int64_t N, int64_t K, int layout, int out_dtype,
                      hipStream_t st) {
    return launch_dequantize_rows(w, nullptr, 0, out, qtype, N, K, layout, out_dtype, st);
}

}  // namespace lowbit
