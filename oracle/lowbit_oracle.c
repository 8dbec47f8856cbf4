/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement (plain C) of the arithmetic behind ipex-llm's low-bit linear
 * path.  Only tests, the smoke check and the cpu_baseline leg of the benchmark
 * may link or load this file; the shipped library never does.
 *
 * The reference keeps this arithmetic in a closed binary (libllama-api.so,
 * bound by python/llm/src/ipex_llm/ggml/model/llama/llama_cpp.py:945-1185) that
 * is not part of its source tree.  What is restated here is therefore the
 * published ggml block-quantization algorithm that the reference's own files
 * cite (python/llm/src/ipex_llm/transformers/gguf/gguf.py:273-342 point at
 * ggml-quants.c of llama.cpp), anchored on the reference's call sites:
 *
 *   oracle_qk_size / oracle_type_size   <- ggml_qk_size / ggml_type_size
 *       (llama_cpp.py:1050-1065; sizes pinned by gguf.py:167-205)
 *   oracle_quantize_tensor              <- ggml_quantize_tensor
 *       (llama_cpp.py:946-967, called from low_bit_linear.py:162)
 *   oracle_dequantize                   <- ggml_dequantize / ggml_dequantize_q4_0
 *       (llama_cpp.py:1068-1099, called from low_bit_linear.py:245,258;
 *        block decoding pinned by gguf.py:273-296,332-342 and the Q4_1 writer
 *        convert.py:417-453)
 *   oracle_mul_mat_q_fp32               <- ggml_compute_forward_mul_mat_q_fp32
 *       (llama_cpp.py:1154-1185, called from low_bit_linear.py:462-497)
 *   oracle_mul_mat_exact                <- the dequantize-then-matmul branch
 *       (low_bit_linear.py:699-702 and MatMulLowBitCPU, low_bit_linear.py:544-556)
 *
 * Pinning status (each check lives in tests/test_oracle_*.py):
 *   sym_int4 / asym_int4 / sym_int8 block layout and decoding: pinned by an
 *     independent numpy restatement of gguf.py's decoders and convert.py's
 *     Q4_1 writer, by closed forms and by brute force over tiny blocks.
 *   sym_int4 / asym_int4 / sym_int8 choice of d, m, q: pinned to the published
 *     ggml quantize_row_*_reference routines by an independent numpy
 *     transcription, closed forms and invariants; the closed binary's exact
 *     rounding (FMA contraction, tie handling) is "parity unpinned".
 *   nf4 and fp8_e4m3 byte formats: "parity unpinned" - the reference text holds
 *     no decoder for them.  The format used here is frozen in this file
 *     (nf4: 64-weight blocks, fp16 absmax, QLoRA codebook; fp8_e4m3: 128-weight
 *     blocks, fp32 scale, OCP E4M3FN codes) and is pinned only internally
 *     (closed forms, brute-force argmin, torch.float8_e4m3fn casts).
 *   oracle_mul_mat_q_fp32: pinned against oracle_mul_mat_exact (bounded
 *     difference), a hand-computed K=32 case and numpy restatements.
 *
 * Build: see oracle/Makefile.  No FMA contraction, no fast-math.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QT_SYM_INT4 2
#define QT_ASYM_INT4 3
#define QT_SYM_INT8 8
#define QT_NF4 10
#define QT_FP8_E4M3 15

/* ---------------------------------------------------------------- fp16 */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE binary32 -> binary16, round to nearest even, software only. */
uint16_t oracle_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) {               /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
    }
    if (absx >= 0x477ff000u) {               /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x38800000u) {                /* below 2^-14: subnormal half */
        if (absx < 0x33000000u) {            /* below 2^-25 -> 0 (2^-25 itself ties to even = 0) */
            return (uint16_t)sign;
        }
        uint32_t e = absx >> 23;             /* biased exponent, 102..112 */
        uint32_t m = (absx & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126 - e;            /* 14..24 */
        uint32_t h = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = (absx - 0x38000000u) >> 13; /* rebias exponent 127 -> 15 */
    uint32_t rem = absx & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    return (uint16_t)(sign | h);
}

float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f;
    uint32_t m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        float v = (float)m * 5.9604644775390625e-08f; /* m * 2^-24, exact */
        return sign ? -v : v;
    }
    if (e == 31) return bits_f32(sign | 0x7f800000u | (m << 13));
    return bits_f32(sign | ((e + 112) << 23) | (m << 13));
}

/* ------------------------------------------------------------ fp8 e4m3fn */

/* OCP E4M3FN: 1-4-3, bias 7, no infinities, max 448, NaN = S.1111.111.
 * Round to nearest even; magnitudes above the largest finite value saturate
 * to 448; NaN maps to 0x7f. */
uint8_t oracle_f32_to_e4m3fn(float f) {
    uint32_t x = f32_bits(f);
    uint8_t sign = (uint8_t)((x >> 24) & 0x80u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx > 0x7f800000u) return (uint8_t)(sign | 0x7f);
    if (absx >= 0x43e00000u) return (uint8_t)(sign | 0x7e);      /* >= 448 */
    if (absx < 0x3c800000u) {                                    /* below 2^-6: subnormal, step 2^-9 */
        float a = bits_f32(absx) * 512.0f;                       /* exact scaling */
        /* a in [0, 8); round to nearest even integer */
        float r = nearbyintf(a);                                 /* default rounding mode: RNE */
        return (uint8_t)(sign | (uint8_t)r);                     /* r == 8 encodes 2^-6 correctly */
    }
    uint32_t h = (absx - 0x3c000000u) >> 20;                     /* rebias 127 -> 7, keep 3 mantissa bits */
    uint32_t rem = absx & 0xfffffu;
    if (rem > 0x80000u || (rem == 0x80000u && (h & 1))) h++;
    if (h > 0x7e) h = 0x7e;
    return (uint8_t)(sign | h);
}

float oracle_e4m3fn_to_f32(uint8_t b) {
    uint32_t e = (b >> 3) & 0xf;
    uint32_t m = b & 7;
    float v;
    if (e == 0xf && m == 7) return bits_f32(0x7fc00000u);
    if (e == 0) v = (float)m * 0.001953125f;                     /* m * 2^-9 */
    else v = bits_f32(((e + 120) << 23) | (m << 20));
    return (b & 0x80) ? -v : v;
}

/* ------------------------------------------------------------- nf4 table */

/* QLoRA NF4 code book (arXiv 2305.14314), fp32. */
static const float NF4_CB[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};

const float *oracle_nf4_codebook(void) { return NF4_CB; }

static inline int nf4_index(float v) {
    /* nearest code; a value exactly on a midpoint takes the lower index */
    int idx = 0;
    for (int i = 0; i < 15; i++) {
        float mid = (NF4_CB[i] + NF4_CB[i + 1]) * 0.5f;
        idx += (v > mid);
    }
    return idx;
}

/* ------------------------------------------------------------ geometry */

int oracle_qk_size(int qtype) {
    switch (qtype) {
    case QT_SYM_INT4: case QT_ASYM_INT4: case QT_SYM_INT8: return 32;
    case QT_NF4: return 64;
    case QT_FP8_E4M3: return 128;
    default: return 0;
    }
}

size_t oracle_type_size(int qtype) {
    switch (qtype) {
    case QT_SYM_INT4: return 18;
    case QT_ASYM_INT4: return 20;
    case QT_SYM_INT8: return 34;
    case QT_NF4: return 34;
    case QT_FP8_E4M3: return 132;
    default: return 0;
    }
}

static inline void put_u16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)(v & 0xff); p[1] = (uint8_t)(v >> 8); }
static inline uint16_t get_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* ----------------------------------------------------------- quantizers */

/* ggml quantize_row_q4_0_reference: signed value of the first element of
 * largest magnitude becomes code 0 (-8), d = max / -8. */
static void quant_block_q4_0(const float *x, uint8_t *out) {
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < 32; j++) {
        float v = x[j];
        if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
    }
    const float d = max / -8.0f;
    const float id = d ? 1.0f / d : 0.0f;
    put_u16(out, oracle_f32_to_f16(d));
    for (int j = 0; j < 16; j++) {
        const float x0 = x[j] * id;
        const float x1 = x[j + 16] * id;
        int q0 = (int8_t)(x0 + 8.5f);
        int q1 = (int8_t)(x1 + 8.5f);
        if (q0 > 15) q0 = 15;
        if (q1 > 15) q1 = 15;
        out[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
}

/* ggml quantize_row_q4_1_reference */
static void quant_block_q4_1(const float *x, uint8_t *out) {
    float min = 3.402823466e+38f, max = -3.402823466e+38f;
    for (int j = 0; j < 32; j++) {
        float v = x[j];
        if (v < min) min = v;
        if (v > max) max = v;
    }
    const float d = (max - min) / 15.0f;
    const float id = d ? 1.0f / d : 0.0f;
    put_u16(out, oracle_f32_to_f16(d));
    put_u16(out + 2, oracle_f32_to_f16(min));
    for (int j = 0; j < 16; j++) {
        const float x0 = (x[j] - min) * id;
        const float x1 = (x[j + 16] - min) * id;
        int q0 = (int8_t)(x0 + 0.5f);
        int q1 = (int8_t)(x1 + 0.5f);
        if (q0 > 15) q0 = 15;
        if (q1 > 15) q1 = 15;
        out[4 + j] = (uint8_t)(q0 | (q1 << 4));
    }
}

/* ggml quantize_row_q8_0_reference; roundf = half away from zero */
static void quant_block_q8_0(const float *x, uint8_t *out) {
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) {
        float v = fabsf(x[j]);
        if (amax < v) amax = v;
    }
    const float d = amax / 127.0f;
    const float id = d ? 1.0f / d : 0.0f;
    put_u16(out, oracle_f32_to_f16(d));
    for (int j = 0; j < 32; j++) {
        out[2 + j] = (uint8_t)(int8_t)roundf(x[j] * id);
    }
}

/* frozen nf4 format: [fp16 absmax][32 bytes], byte j = idx[j] | idx[j+32] << 4 */
static void quant_block_nf4(const float *x, uint8_t *out) {
    float amax = 0.0f;
    for (int j = 0; j < 64; j++) {
        float v = fabsf(x[j]);
        if (amax < v) amax = v;
    }
    const float d = amax;
    const float id = d ? 1.0f / d : 0.0f;
    put_u16(out, oracle_f32_to_f16(d));
    for (int j = 0; j < 32; j++) {
        int q0 = nf4_index(x[j] * id);
        int q1 = nf4_index(x[j + 32] * id);
        out[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
}

/* frozen fp8_e4m3 format: [fp32 scale = absmax/448][128 E4M3FN codes] */
static void quant_block_fp8(const float *x, uint8_t *out) {
    float amax = 0.0f;
    for (int j = 0; j < 128; j++) {
        float v = fabsf(x[j]);
        if (amax < v) amax = v;
    }
    const float s = amax / 448.0f;
    const float is = s ? 1.0f / s : 0.0f;
    memcpy(out, &s, 4);
    for (int j = 0; j < 128; j++) out[4 + j] = oracle_f32_to_e4m3fn(x[j] * is);
}

/* n = total number of weights, k = row length (only its divisibility matters:
 * blocks never straddle rows because k % QK == 0).  Returns bytes written, or
 * 0 for an unsupported qtype / shape. */
size_t oracle_quantize_tensor(const float *src, void *dst, int qtype, size_t n, int k) {
    const int qk = oracle_qk_size(qtype);
    const size_t ts = oracle_type_size(qtype);
    if (!qk || k <= 0 || (k % qk) != 0 || (n % (size_t)qk) != 0) return 0;
    const size_t nb = n / (size_t)qk;
    uint8_t *out = (uint8_t *)dst;
#pragma omp parallel for schedule(static)
    for (long long b = 0; b < (long long)nb; b++) {
        const float *x = src + (size_t)b * qk;
        uint8_t *o = out + (size_t)b * ts;
        switch (qtype) {
        case QT_SYM_INT4: quant_block_q4_0(x, o); break;
        case QT_ASYM_INT4: quant_block_q4_1(x, o); break;
        case QT_SYM_INT8: quant_block_q8_0(x, o); break;
        case QT_NF4: quant_block_nf4(x, o); break;
        case QT_FP8_E4M3: quant_block_fp8(x, o); break;
        }
    }
    return nb * ts;
}

/* ---------------------------------------------------------- dequantizers */

static void dequant_block(const uint8_t *b, float *y, int qtype) {
    switch (qtype) {
    case QT_SYM_INT4: {
        const float d = oracle_f16_to_f32(get_u16(b));
        for (int j = 0; j < 16; j++) {
            y[j] = (float)((b[2 + j] & 0xf) - 8) * d;
            y[j + 16] = (float)((b[2 + j] >> 4) - 8) * d;
        }
    } break;
    case QT_ASYM_INT4: {
        const float d = oracle_f16_to_f32(get_u16(b));
        const float m = oracle_f16_to_f32(get_u16(b + 2));
        for (int j = 0; j < 16; j++) {
            y[j] = (float)(b[4 + j] & 0xf) * d + m;
            y[j + 16] = (float)(b[4 + j] >> 4) * d + m;
        }
    } break;
    case QT_SYM_INT8: {
        const float d = oracle_f16_to_f32(get_u16(b));
        for (int j = 0; j < 32; j++) y[j] = (float)(int8_t)b[2 + j] * d;
    } break;
    case QT_NF4: {
        const float d = oracle_f16_to_f32(get_u16(b));
        for (int j = 0; j < 32; j++) {
            y[j] = NF4_CB[b[2 + j] & 0xf] * d;
            y[j + 32] = NF4_CB[b[2 + j] >> 4] * d;
        }
    } break;
    case QT_FP8_E4M3: {
        float s;
        memcpy(&s, b, 4);
        for (int j = 0; j < 128; j++) y[j] = oracle_e4m3fn_to_f32(b[4 + j]) * s;
    } break;
    }
}

/* n = number of weights to produce */
void oracle_dequantize(const void *src, float *dst, size_t n, int qtype) {
    const int qk = oracle_qk_size(qtype);
    const size_t ts = oracle_type_size(qtype);
    if (!qk) return;
    const size_t nb = n / (size_t)qk;
    const uint8_t *in = (const uint8_t *)src;
#pragma omp parallel for schedule(static)
    for (long long b = 0; b < (long long)nb; b++)
        dequant_block(in + (size_t)b * ts, dst + (size_t)b * qk, qtype);
}

/* --------------------------------------------------------------- matmul */

/* Activation row -> ggml Q8_0 (fp16 d) or Q8_1 (fp32 d and s = d * sum q)
 * blocks of 32, as ggml's mul_mat does before the integer dot product. */
typedef struct { float d; float s; int8_t q[32]; } act_block;

static void quant_act_row(const float *x, int k, act_block *out, int q81) {
    for (int b = 0; b < k / 32; b++) {
        const float *xb = x + b * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) {
            float v = fabsf(xb[j]);
            if (amax < v) amax = v;
        }
        const float d = amax / 127.0f;
        const float id = d ? 1.0f / d : 0.0f;
        int sum = 0;
        for (int j = 0; j < 32; j++) {
            int8_t q = (int8_t)roundf(xb[j] * id);
            out[b].q[j] = q;
            sum += q;
        }
        if (q81) {
            out[b].d = d;
            out[b].s = (float)sum * d;
        } else {
            out[b].d = oracle_f16_to_f32(oracle_f32_to_f16(d));
            out[b].s = 0.0f;
        }
    }
}

/* y[m][n] = sum_k x[m][k] * dequant(W)[n][k], ggml style.
 * ne arrays follow ggml: ne[0] = K (fastest), ne[1] = rows
 * (low_bit_linear.py:477-483 reverses the torch shapes).
 * sym_int4 / sym_int8: activations to Q8_0, integer block dot, fp32 sum.
 * asym_int4: activations to Q8_1.
 * nf4 / fp8_e4m3: the reference has no CPU low-bit matmul for them
 * (low_bit_linear.py:689-692 raises); they are computed as fp32 dequantize +
 * fp32 dot so that every qtype has a CPU number. */
void oracle_mul_mat_q_fp32(const int64_t *src0_ne, const void *src0, int qtype,
                           const int64_t *src1_ne, const float *src1, float *dst) {
    const int64_t K = src0_ne[0], N = src0_ne[1], M = src1_ne[1];
    const int qk = oracle_qk_size(qtype);
    const size_t ts = oracle_type_size(qtype);
    if (!qk || src1_ne[0] != K || K % qk) return;
    const uint8_t *w = (const uint8_t *)src0;
    const size_t row_bytes = (size_t)(K / qk) * ts;

    if (qtype == QT_NF4 || qtype == QT_FP8_E4M3) {
#pragma omp parallel
        {
            float *wrow = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
            for (long long n = 0; n < N; n++) {
                for (int64_t b = 0; b < K / qk; b++)
                    dequant_block(w + (size_t)n * row_bytes + (size_t)b * ts, wrow + b * qk, qtype);
                for (int64_t m = 0; m < M; m++) {
                    const float *x = src1 + (size_t)m * K;
                    float acc = 0.0f;
                    for (int64_t k = 0; k < K; k++) acc += x[k] * wrow[k];
                    dst[(size_t)m * N + n] = acc;
                }
            }
            free(wrow);
        }
        return;
    }

    const int nbk = (int)(K / 32);
    act_block *act = (act_block *)malloc(sizeof(act_block) * (size_t)nbk * (size_t)M);
    const int q81 = (qtype == QT_ASYM_INT4);
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < M; m++) quant_act_row(src1 + (size_t)m * K, (int)K, act + (size_t)m * nbk, q81);

#pragma omp parallel for schedule(static)
    for (long long n = 0; n < N; n++) {
        const uint8_t *wr = w + (size_t)n * row_bytes;
        for (int64_t m = 0; m < M; m++) {
            const act_block *a = act + (size_t)m * nbk;
            float sumf = 0.0f;
            for (int b = 0; b < nbk; b++) {
                const uint8_t *wb = wr + (size_t)b * ts;
                int sumi = 0;
                if (qtype == QT_SYM_INT4) {
                    for (int j = 0; j < 16; j++) {
                        const int v0 = (wb[2 + j] & 0xf) - 8;
                        const int v1 = (wb[2 + j] >> 4) - 8;
                        sumi += v0 * a[b].q[j] + v1 * a[b].q[j + 16];
                    }
                    sumf += (float)sumi * oracle_f16_to_f32(get_u16(wb)) * a[b].d;
                } else if (qtype == QT_ASYM_INT4) {
                    for (int j = 0; j < 16; j++) {
                        const int v0 = wb[4 + j] & 0xf;
                        const int v1 = wb[4 + j] >> 4;
                        sumi += v0 * a[b].q[j] + v1 * a[b].q[j + 16];
                    }
                    sumf += (oracle_f16_to_f32(get_u16(wb)) * a[b].d) * (float)sumi +
                            oracle_f16_to_f32(get_u16(wb + 2)) * a[b].s;
                } else {
                    for (int j = 0; j < 32; j++) sumi += (int)(int8_t)wb[2 + j] * a[b].q[j];
                    sumf += (float)sumi * (oracle_f16_to_f32(get_u16(wb)) * a[b].d);
                }
            }
            dst[(size_t)m * N + n] = sumf;
        }
    }
    free(act);
}

/* y = x_f32 @ dequant(W)^T with fp32 dequantized weights and fp64 accumulation:
 * the value the reference's dequantize-then-linear branch aims at. */
void oracle_mul_mat_exact(const int64_t *src0_ne, const void *src0, int qtype,
                          const int64_t *src1_ne, const float *src1, float *dst) {
    const int64_t K = src0_ne[0], N = src0_ne[1], M = src1_ne[1];
    const int qk = oracle_qk_size(qtype);
    const size_t ts = oracle_type_size(qtype);
    if (!qk || src1_ne[0] != K || K % qk) return;
    const uint8_t *w = (const uint8_t *)src0;
    const size_t row_bytes = (size_t)(K / qk) * ts;
#pragma omp parallel
    {
        float *wrow = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (long long n = 0; n < N; n++) {
            for (int64_t b = 0; b < K / qk; b++)
                dequant_block(w + (size_t)n * row_bytes + (size_t)b * ts, wrow + b * qk, qtype);
            for (int64_t m = 0; m < M; m++) {
                const float *x = src1 + (size_t)m * K;
                double acc = 0.0;
                for (int64_t k = 0; k < K; k++) acc += (double)x[k] * (double)wrow[k];
                dst[(size_t)m * N + n] = (float)acc;
            }
        }
        free(wrow);
    }
}

int oracle_max_threads(void) {
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
