// Block formats and the two memory layouts of a quantized weight [N, K].
//
// Layout 0 ("ggml"): the array-of-structs blob the reference keeps on the CPU
//   (python/llm/src/ipex_llm/transformers/low_bit_linear.py:104-175):
//   row-major blocks, K fastest, each block = header (scale[, min]) + codes.
//     sym_int4  (2)  32 w: fp16 d | 16 B, byte j = code[j] | code[j+16] << 4
//     asym_int4 (3)  32 w: fp16 d | fp16 m | 16 B, same nibble order
//     sym_int8  (8)  32 w: fp16 d | 32 x int8
//     nf4       (10) 64 w: fp16 d | 32 B, byte j = idx[j] | idx[j+32] << 4
//     fp8_e4m3  (15) 128 w: fp32 s | 128 x E4M3FN
//
// Layout 1 ("tiled"): what the MFMA kernels stream.  It plays the part of the
//   reference's device re-layout (ggml_q_format_convet_cpu2xpu,
//   low_bit_linear.py:178-204) and has the same byte count.  The matrix is cut
//   into tiles of 16 rows x 128 columns, stored tile after tile ([N/16][K/128]),
//   so a wave reads one tile as one contiguous, 16-byte-per-lane load.  Inside
//   a tile, lane l = 16*c + n (n = row in tile, c = 0..3) owns, for each of the
//   four 32-column sub-blocks j, the 8 columns 32*j + 8*c .. +7 of row n: exactly
//   the B operand of v_mfma_f32_16x16x32 for that lane.
//     4-bit formats: codes = 64 lanes x 16 B (dword j = sub-block j; the eight
//       nibbles hold columns [0,2,4,6,1,3,5,7] so that masking with 0x000F000F
//       after shifts of 0,4,8,12 yields column pairs (0,1)(2,3)(4,5)(6,7)).
//     8-bit formats: codes = 2 x 64 lanes x 16 B (first KiB: sub-blocks 0,1;
//       second KiB: sub-blocks 2,3; 8 bytes per sub-block in column order).
//     The per-block headers of the tile follow its codes:
//       sym_int4  +1024: [16 rows][4] fp16 d              (tile = 1152 B)
//       asym_int4 +1024: [16 rows][4] (fp16 d, fp16 m)    (tile = 1280 B)
//       nf4       +1024: [16 rows][2] fp16 d              (tile = 1088 B)
//       sym_int8  +2048: [16 rows][4] fp16 d              (tile = 2176 B)
//       fp8_e4m3  +2048: [16 rows]    fp32 s              (tile = 2112 B)
//   The tiled layout needs N % 16 == 0 and K % 128 == 0.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lowbit {

enum : int { QT_SYM_INT4 = 2, QT_ASYM_INT4 = 3, QT_SYM_INT8 = 8, QT_NF4 = 10, QT_FP8_E4M3 = 15 };
enum : int { LAYOUT_GGML = 0, LAYOUT_TILED = 1 };
enum : int { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2 };

constexpr int TILE_ROWS = 16;
constexpr int TILE_COLS = 128;

template <int QT> struct Fmt;
template <> struct Fmt<QT_SYM_INT4> {
    static constexpr int QK = 32, TS = 18, HDR = 2, BITS = 4, TILE_CODE_BYTES = 1024, TILE_BYTES = 1152;
};
template <> struct Fmt<QT_ASYM_INT4> {
    static constexpr int QK = 32, TS = 20, HDR = 4, BITS = 4, TILE_CODE_BYTES = 1024, TILE_BYTES = 1280;
};
template <> struct Fmt<QT_SYM_INT8> {
    static constexpr int QK = 32, TS = 34, HDR = 2, BITS = 8, TILE_CODE_BYTES = 2048, TILE_BYTES = 2176;
};
template <> struct Fmt<QT_NF4> {
    static constexpr int QK = 64, TS = 34, HDR = 2, BITS = 4, TILE_CODE_BYTES = 1024, TILE_BYTES = 1088;
};
template <> struct Fmt<QT_FP8_E4M3> {
    static constexpr int QK = 128, TS = 132, HDR = 4, BITS = 8, TILE_CODE_BYTES = 2048, TILE_BYTES = 2112;
};

__host__ __device__ inline int qk_size(int qt) {
    switch (qt) {
    case QT_SYM_INT4: case QT_ASYM_INT4: case QT_SYM_INT8: return 32;
    case QT_NF4: return 64;
    case QT_FP8_E4M3: return 128;
    default: return 0;
    }
}
__host__ __device__ inline int type_size(int qt) {
    switch (qt) {
    case QT_SYM_INT4: return 18;
    case QT_ASYM_INT4: return 20;
    case QT_SYM_INT8: case QT_NF4: return 34;
    case QT_FP8_E4M3: return 132;
    default: return 0;
    }
}

// ---------------------------------------------------------------- scalars

__device__ inline float h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ inline uint16_t f2h(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }  // RNE

__device__ inline float e4m3_to_f32(uint32_t b) {
    const uint32_t e = (b >> 3) & 0xf, m = b & 7;
    float v;
    if (e == 0) v = (float)m * 0.001953125f;
    else v = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
    return (b & 0x80) ? -v : v;
}

// fp32 -> OCP E4M3FN, round to nearest even, saturating at 448; integer-only so
// that no compiler float option can change a bit of it.
__device__ inline uint32_t f32_to_e4m3(float f) {
    const uint32_t x = __builtin_bit_cast(uint32_t, f);
    const uint32_t sign = (x >> 24) & 0x80u;
    const uint32_t a = x & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7f;
    if (a >= 0x43e00000u) return sign | 0x7e;
    if (a < 0x3c800000u) {                       // |f| < 2^-6: multiples of 2^-9
        if (a < 0x3a800000u) return sign;        // < 2^-10: rounds to 0 (2^-10 ties to even = 0) ...
        // value = m * 2^(e-150) with 24-bit m; code = value / 2^-9 = m >> (141 - e), e in 117..120
        const uint32_t e = a >> 23;
        const uint32_t m = (a & 0x7fffffu) | 0x800000u;
        const uint32_t sh = 141u - e;            // 21..24
        uint32_t h = m >> sh;
        const uint32_t rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return sign | h;
    }
    uint32_t h = (a - 0x3c000000u) >> 20;
    const uint32_t rem = a & 0xfffffu;
    if (rem > 0x80000u || (rem == 0x80000u && (h & 1u))) h++;
    if (h > 0x7e) h = 0x7e;
    return sign | h;
}

__device__ __constant__ const float NF4_CODEBOOK[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};

// ------------------------------------------------------------- sub-blocks
//
// The unit every generic kernel works on is a "sub-block": 32 consecutive
// columns of one row (sb = column / 32).  SubBlock carries its 32 raw codes
// (nibble or byte values, column order) and the header of the block it is in.

struct SubBlock {
    uint8_t code[32];
    float d;      // scale
    float m;      // asym_int4 minimum, else 0
    uint32_t hdr; // raw header bits (fp16 d | fp16 m << 16, or fp32 s)
};

template <int QT> __device__ inline float decode(uint32_t c, float d, float m) {
    if constexpr (QT == QT_SYM_INT4) return (float)((int)c - 8) * d;
    else if constexpr (QT == QT_ASYM_INT4) return (float)c * d + m;
    else if constexpr (QT == QT_SYM_INT8) return (float)(int8_t)c * d;
    else if constexpr (QT == QT_NF4) return NF4_CODEBOOK[c] * d;
    else return e4m3_to_f32(c) * d;
}

template <int QT> __device__ inline void hdr_to_scale(uint32_t hdr, float &d, float &m) {
    m = 0.0f;
    if constexpr (QT == QT_FP8_E4M3) d = __builtin_bit_cast(float, hdr);
    else {
        d = h2f((uint16_t)(hdr & 0xffff));
        if constexpr (QT == QT_ASYM_INT4) m = h2f((uint16_t)(hdr >> 16));
    }
}

// ggml layout: row n, sub-block sb of a [N, K] blob.
template <int QT>
__device__ inline void ggml_load_sub(const uint8_t *w, int64_t n, int64_t K, int sb, SubBlock &s) {
    using F = Fmt<QT>;
    constexpr int SPB = F::QK / 32;                  // sub-blocks per block
    const int64_t blk = n * (K / F::QK) + sb / SPB;
    const int part = sb % SPB;
    const uint8_t *b = w + blk * F::TS;
    if constexpr (F::HDR == 2) s.hdr = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
    else s.hdr = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24);
    hdr_to_scale<QT>(s.hdr, s.d, s.m);
    const uint8_t *q = b + F::HDR;
    if constexpr (QT == QT_SYM_INT4 || QT == QT_ASYM_INT4) {
        for (int j = 0; j < 16; j++) { s.code[j] = q[j] & 0xf; s.code[j + 16] = q[j] >> 4; }
    } else if constexpr (QT == QT_NF4) {
        // element e of the 64-block lives in byte e % 32, nibble e / 32
        for (int j = 0; j < 32; j++) {
            const int e = part * 32 + j;
            const uint8_t v = q[e & 31];
            s.code[j] = (e < 32) ? (v & 0xf) : (v >> 4);
        }
    } else {
        for (int j = 0; j < 32; j++) s.code[j] = q[part * 32 + j];
    }
}

// Offsets inside the tiled layout.
template <int QT> __device__ __host__ inline int64_t tile_offset(int64_t n, int64_t K, int sb) {
    return ((n / TILE_ROWS) * (K / TILE_COLS) + sb / 4) * (int64_t)Fmt<QT>::TILE_BYTES;
}

__device__ inline uint32_t pack_nibbles8(const uint8_t *k) {  // columns -> device nibble order
    return (uint32_t)k[0] | ((uint32_t)k[2] << 4) | ((uint32_t)k[4] << 8) | ((uint32_t)k[6] << 12) |
           ((uint32_t)k[1] << 16) | ((uint32_t)k[3] << 20) | ((uint32_t)k[5] << 24) | ((uint32_t)k[7] << 28);
}
__device__ inline void unpack_nibbles8(uint32_t v, uint8_t *k) {
    k[0] = v & 0xf; k[2] = (v >> 4) & 0xf; k[4] = (v >> 8) & 0xf; k[6] = (v >> 12) & 0xf;
    k[1] = (v >> 16) & 0xf; k[3] = (v >> 20) & 0xf; k[5] = (v >> 24) & 0xf; k[7] = (v >> 28) & 0xf;
}

template <int QT> __device__ inline int tile_hdr_offset(int r, int j) {
    using F = Fmt<QT>;
    if constexpr (QT == QT_SYM_INT4 || QT == QT_SYM_INT8) return F::TILE_CODE_BYTES + r * 8 + j * 2;
    else if constexpr (QT == QT_ASYM_INT4) return F::TILE_CODE_BYTES + r * 16 + j * 4;
    else if constexpr (QT == QT_NF4) return F::TILE_CODE_BYTES + r * 4 + (j / 2) * 2;
    else return F::TILE_CODE_BYTES + r * 4;
}

template <int QT>
__device__ inline void tiled_load_sub(const uint8_t *w, int64_t n, int64_t K, int sb, SubBlock &s) {
    using F = Fmt<QT>;
    const uint8_t *t = w + tile_offset<QT>(n, K, sb);
    const int r = (int)(n % TILE_ROWS), j = sb % 4;
    const uint8_t *h = t + tile_hdr_offset<QT>(r, j);
    if constexpr (F::HDR == 2) s.hdr = *(const uint16_t *)h;
    else s.hdr = *(const uint32_t *)h;
    hdr_to_scale<QT>(s.hdr, s.d, s.m);
    for (int c = 0; c < 4; c++) {
        const int lane = c * 16 + r;
        if constexpr (F::BITS == 4) {
            unpack_nibbles8(*(const uint32_t *)(t + lane * 16 + j * 4), s.code + c * 8);
        } else {
            const uint8_t *p = t + (j / 2) * 1024 + lane * 16 + (j % 2) * 8;
            for (int i = 0; i < 8; i++) s.code[c * 8 + i] = p[i];
        }
    }
}

// Stores one sub-block into the tiled layout.  The header is written by the
// caller that owns the first sub-block of a block (see tiled_store_hdr).
template <int QT>
__device__ inline void tiled_store_codes(uint8_t *w, int64_t n, int64_t K, int sb, const uint8_t *code) {
    using F = Fmt<QT>;
    uint8_t *t = w + tile_offset<QT>(n, K, sb);
    const int r = (int)(n % TILE_ROWS), j = sb % 4;
    for (int c = 0; c < 4; c++) {
        const int lane = c * 16 + r;
        if constexpr (F::BITS == 4) {
            *(uint32_t *)(t + lane * 16 + j * 4) = pack_nibbles8(code + c * 8);
        } else {
            uint32_t lo = 0, hi = 0;
            for (int i = 0; i < 4; i++) {
                lo |= (uint32_t)code[c * 8 + i] << (8 * i);
                hi |= (uint32_t)code[c * 8 + 4 + i] << (8 * i);
            }
            uint32_t *p = (uint32_t *)(t + (j / 2) * 1024 + lane * 16 + (j % 2) * 8);
            p[0] = lo;
            p[1] = hi;
        }
    }
}

template <int QT>
__device__ inline void tiled_store_hdr(uint8_t *w, int64_t n, int64_t K, int sb, uint32_t hdr) {
    using F = Fmt<QT>;
    uint8_t *h = w + tile_offset<QT>(n, K, sb) + tile_hdr_offset<QT>((int)(n % TILE_ROWS), sb % 4);
    if constexpr (F::HDR == 2) *(uint16_t *)h = (uint16_t)hdr;
    else *(uint32_t *)h = hdr;
}

// Four consecutive columns (4*part .. 4*part+3, part = 0..7) of sub-block sb of row n, and the raw
// header of their block: what one lane of the dequantizers needs.
template <int QT>
__device__ inline void ggml_load4(const uint8_t *w, int64_t n, int64_t K, int sb, int part, uint32_t (&code)[4],
                                  uint32_t &hdr) {
    using F = Fmt<QT>;
    constexpr int SPB = F::QK / 32;
    const int64_t blk = n * (K / F::QK) + sb / SPB;
    const uint8_t *b = w + blk * F::TS;
    if constexpr (F::HDR == 2) hdr = (uint32_t)b[0] | ((uint32_t)b[1] << 8);
    else hdr = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24);
    // blocks are 18, 20, 34 or 132 bytes long and the codes start 2 or 4 bytes in: every 4-byte
    // group of codes is 2-byte aligned
    const uint8_t *q = b + F::HDR;
    int off, sh = 0;
    if constexpr (QT == QT_SYM_INT4 || QT == QT_ASYM_INT4) {
        off = (part & 3) * 4; sh = (part >> 2) * 4;           // columns 16..31 sit in the high nibbles
    } else if constexpr (QT == QT_NF4) {
        off = part * 4; sh = (sb % SPB) * 4;                  // elements 32..63 sit in the high nibbles
    } else {
        off = (sb % SPB) * 32 + part * 4;
    }
    const uint16_t *q2 = (const uint16_t *)(q + off);
    const uint32_t v = ((uint32_t)q2[0] | ((uint32_t)q2[1] << 16)) >> sh;
    constexpr uint32_t MASK = F::BITS == 4 ? 0xfu : 0xffu;
#pragma unroll
    for (int i = 0; i < 4; i++) code[i] = (v >> (8 * i)) & MASK;
}

template <int QT>
__device__ inline void tiled_load4(const uint8_t *w, int64_t n, int64_t K, int sb, int part, uint32_t (&code)[4],
                                   uint32_t &hdr) {
    using F = Fmt<QT>;
    const uint8_t *t = w + tile_offset<QT>(n, K, sb);
    const int r = (int)(n % TILE_ROWS), j = sb % 4;
    const uint8_t *h = t + tile_hdr_offset<QT>(r, j);
    if constexpr (F::HDR == 2) hdr = *(const uint16_t *)h;
    else hdr = *(const uint32_t *)h;
    const int lane = (part >> 1) * 16 + r, half = part & 1;
    if constexpr (F::BITS == 4) {
        // nibble order 0,2,4,6,1,3,5,7: columns 4*half .. +3 are nibbles 2*half, 2*half+4, 2*half+1, 2*half+5
        const uint32_t v = *(const uint32_t *)(t + lane * 16 + j * 4) >> (8 * half);
        code[0] = v & 0xf; code[1] = (v >> 16) & 0xf; code[2] = (v >> 4) & 0xf; code[3] = (v >> 20) & 0xf;
    } else {
        const uint32_t v = *(const uint32_t *)(t + (j / 2) * 1024 + lane * 16 + (j % 2) * 8 + half * 4);
#pragma unroll
        for (int i = 0; i < 4; i++) code[i] = (v >> (8 * i)) & 0xff;
    }
}

// Stores one sub-block into the ggml layout (codes only for the part it covers;
// the header when it is the first sub-block of its block).
template <int QT>
__device__ inline void ggml_store_sub(uint8_t *w, int64_t n, int64_t K, int sb, const uint8_t *code, uint32_t hdr) {
    using F = Fmt<QT>;
    constexpr int SPB = F::QK / 32;
    const int64_t blk = n * (K / F::QK) + sb / SPB;
    const int part = sb % SPB;
    uint8_t *b = w + blk * F::TS;
    if (part == 0) {
        b[0] = hdr & 0xff;
        b[1] = (hdr >> 8) & 0xff;
        if constexpr (F::HDR == 4) { b[2] = (hdr >> 16) & 0xff; b[3] = (hdr >> 24) & 0xff; }
    }
    uint8_t *q = b + F::HDR;
    if constexpr (QT == QT_SYM_INT4 || QT == QT_ASYM_INT4) {
        for (int j = 0; j < 16; j++) q[j] = code[j] | (code[j + 16] << 4);
    } else if constexpr (QT == QT_NF4) {
        // part 0 owns the low nibbles of bytes 0..31, part 1 the high nibbles: the caller
        // hands over both parts of a block at once through ggml_store_nf4_block instead.
    } else {
        for (int j = 0; j < 32; j++) q[part * 32 + j] = code[j];
    }
}

__device__ inline void ggml_store_nf4_block(uint8_t *w, int64_t blk, const uint8_t *code64, uint32_t hdr) {
    uint8_t *b = w + blk * 34;
    b[0] = hdr & 0xff;
    b[1] = (hdr >> 8) & 0xff;
    for (int j = 0; j < 32; j++) b[2 + j] = code64[j] | (code64[j + 32] << 4);
}

}  // namespace lowbit
