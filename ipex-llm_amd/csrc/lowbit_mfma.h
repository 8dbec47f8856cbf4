// Vector types, MFMA wrappers and per-lane tile registers shared by the GEMV and GEMM kernels.
#pragma once
#include "lowbit_formats.h"

namespace lowbit {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename AT> struct Vec8;
template <> struct Vec8<_Float16> { typedef f16x8 type; };
template <> struct Vec8<__bf16> { typedef bf16x8 type; };

__device__ inline f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
__device__ inline f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }

template <typename AT> __device__ inline AT to_at(float v);
template <> __device__ inline _Float16 to_at<_Float16>(float v) { return (_Float16)v; }
template <> __device__ inline __bf16 to_at<__bf16>(float v) { return (__bf16)v; }

__device__ inline uint32_t and_or(uint32_t a, uint32_t b, uint32_t c) { return (a & b) | c; }

// Raw tile registers of one lane: codes (16 or 32 bytes) and the headers of its row.
template <int QT> struct TileRegs {
    u32x4 q0, q1;
    u32x4 h;
};

// Loads through a pointer that is known to be global memory.  A pointer fetched from a table in
// memory is generic to the compiler and would be read with flat loads, which also count against
// the LDS wait counter.
typedef const __attribute__((address_space(1))) uint8_t *gbytes;
// STREAM: a load of bytes that this launch reads exactly once (the weights of a GEMV), marked nontemporal so
// that they pass through the caches without displacing what is read again (x) - measured on MI355X, sym_int4
// at M = 1: [11008 x 4096] 6.64 -> 6.24 us per launch, [4096 x 4096] 4.12 -> 3.85, [8192 x 8192] 9.10 -> 8.76.
template <typename T, bool STREAM = false> __device__ inline T ld(const uint8_t *p) {
    if constexpr (STREAM) return __builtin_nontemporal_load((const T *)p);
    else return *(const T *)p;
}
template <typename T, bool STREAM = false> __device__ inline T ld(gbytes p) {
    if constexpr (STREAM) return __builtin_nontemporal_load((const __attribute__((address_space(1))) T *)p);
    else return *(const __attribute__((address_space(1))) T *)p;
}

template <int QT, bool STREAM = false, typename P> __device__ inline void load_tile(P tile, int lane, int r, TileRegs<QT> &t) {
    using F = Fmt<QT>;
    t.q0 = ld<u32x4, STREAM>(tile + lane * 16);
    if constexpr (F::BITS == 8) t.q1 = ld<u32x4, STREAM>(tile + 1024 + lane * 16);
    if constexpr (QT == QT_SYM_INT4 || QT == QT_SYM_INT8) {
        const u32x2 h = ld<u32x2, STREAM>(tile + F::TILE_CODE_BYTES + r * 8);
        t.h[0] = h[0]; t.h[1] = h[1];
    } else if constexpr (QT == QT_ASYM_INT4) {
        t.h = ld<u32x4, STREAM>(tile + F::TILE_CODE_BYTES + r * 16);
    } else {
        t.h[0] = ld<uint32_t, STREAM>(tile + F::TILE_CODE_BYTES + r * 4);
    }
}

// scale (and minimum) of sub-block j of the lane's row
template <int QT> __device__ inline void tile_scale(const TileRegs<QT> &t, int j, float &d, float &m) {
    m = 0.0f;
    if constexpr (QT == QT_SYM_INT4 || QT == QT_SYM_INT8) {
        const uint32_t h = t.h[j >> 1];
        d = h2f((j & 1) ? (h >> 16) : (h & 0xffff));
    } else if constexpr (QT == QT_ASYM_INT4) {
        d = h2f(t.h[j] & 0xffff);
        m = h2f(t.h[j] >> 16);
    } else if constexpr (QT == QT_NF4) {
        d = h2f((j >> 1) ? (t.h[0] >> 16) : (t.h[0] & 0xffff));
    } else {
        d = __builtin_bit_cast(float, t.h[0]);
    }
}

}  // namespace lowbit
