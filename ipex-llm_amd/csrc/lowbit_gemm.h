// Pieces shared by the MFMA GEMM kernels: dequantization of tile registers into packed operand pairs,
// the 32x32x16 MFMA with pinned accumulators, wait helpers.
#pragma once
#include <type_traits>
#include "lowbit_mfma.h"

namespace lowbit {

// ---- raw codes of sub-block s of a tile -> 8 *scaled* weights in the activation type ------

// Dequant<QT, AT>::pair(t, s, p): columns 2p, 2p+1 (p = 0..3) of the lane's 8 columns of
// sub-block s, scaled, as one packed 32-bit register.  Pair granularity lets the main loop
// slip a few VALU instructions between consecutive MFMAs.
template <int QT, typename AT> struct Dequant;

// What the dequantizers need besides the tile: the nf4 code book (LDS) and the exponent pattern
// that is OR-ed onto 4-bit codes, held in a vector register.  As a literal it would share the
// instruction's only constant slot with the nibble mask and v_and_or_b32 would fall apart into
// an AND and an OR.
struct DqCtx {
    const void *lut;
    uint32_t magic;
};
template <int QT, typename AT> __device__ inline uint32_t dq_magic() {
    uint32_t r;
    if constexpr (sizeof(AT) == 2 && __is_same(AT, _Float16)) asm("v_mov_b32 %0, 0x64006400" : "=v"(r));
    else asm("v_mov_b32 %0, 0x43004300" : "=v"(r));
    return r;
}

__device__ inline f16x2 h2(uint32_t bits16) {
    const uint32_t p = (bits16 & 0xffffu) | (bits16 << 16);
    return __builtin_bit_cast(f16x2, p);
}
__device__ inline uint32_t pk(f16x2 v) { return __builtin_bit_cast(uint32_t, v); }
__device__ inline uint32_t pk(bf16x2 v) { return __builtin_bit_cast(uint32_t, v); }
template <typename AT> __device__ inline uint32_t pk2(float a, float b);
template <> __device__ inline uint32_t pk2<_Float16>(float a, float b) { return pk(f16x2{(_Float16)a, (_Float16)b}); }
template <> __device__ inline uint32_t pk2<__bf16>(float a, float b) { return pk(bf16x2{(__bf16)a, (__bf16)b}); }

template <> struct Dequant<QT_SYM_INT4, _Float16> {
    __device__ static uint32_t pair(const TileRegs<QT_SYM_INT4> &t, int s, int p, const DqCtx &cx) {
        const uint32_t hb = t.h[s >> 1];
        const f16x2 d2 = h2((s & 1) ? (hb >> 16) : hb);
        const f16x2 k1032 = {(_Float16)1032.0f, (_Float16)1032.0f};
        const f16x2 k16th = {(_Float16)0.0625f, (_Float16)0.0625f};
        const f16x2 k72 = {(_Float16)72.0f, (_Float16)72.0f};
        const uint32_t v = (p & 2) ? (t.q0[s] >> 8) : t.q0[s];
        // exact q - 8 first (0x6400 | q is the half 1024 + q), one rounding in the multiply by d
        if (p & 1)
            return pk(__builtin_elementwise_fma(__builtin_bit_cast(f16x2, and_or(v, 0x00f000f0u, cx.magic)), k16th, -k72) * d2);
        return pk((__builtin_bit_cast(f16x2, and_or(v, 0x000f000fu, cx.magic)) - k1032) * d2);
    }
};

template <> struct Dequant<QT_ASYM_INT4, _Float16> {
    __device__ static uint32_t pair(const TileRegs<QT_ASYM_INT4> &t, int s, int p, const DqCtx &cx) {
        const f16x2 d2 = h2(t.h[s]), m2 = h2(t.h[s] >> 16);
        const f16x2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const f16x2 k16th = {(_Float16)0.0625f, (_Float16)0.0625f};
        const f16x2 k64 = {(_Float16)64.0f, (_Float16)64.0f};
        const uint32_t v = (p & 2) ? (t.q0[s] >> 8) : t.q0[s];
        f16x2 q;
        if (p & 1) q = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, and_or(v, 0x00f000f0u, cx.magic)), k16th, -k64);
        else q = __builtin_bit_cast(f16x2, and_or(v, 0x000f000fu, cx.magic)) - k1024;
        return pk(__builtin_elementwise_fma(q, d2, m2));
    }
};

// 4-bit integer codes with bf16 activations: bf16 has no packed arithmetic on gfx950, so the
// weight is formed in fp32 ((128 + q) comes for free as a bit pattern) and rounded once.
template <int QT> struct DequantInt4Bf16 {
    __device__ static uint32_t pair(const TileRegs<QT> &t, int s, int p, const DqCtx &cx) {
        float d, mn;
        tile_scale<QT>(t, s, d, mn);
        const float off = (QT == QT_SYM_INT4) ? 136.0f : 128.0f;
        const float c = mn - off * d;
        const uint32_t pr = and_or(t.q0[s] >> (4 * p), 0x000f000fu, cx.magic);   // bf16 pair 128+q
        const float lo = __builtin_bit_cast(float, pr << 16);
        const float hi = __builtin_bit_cast(float, pr & 0xffff0000u);
        return pk2<__bf16>(fmaf(lo, d, c), fmaf(hi, d, c));
    }
};
template <> struct Dequant<QT_SYM_INT4, __bf16> : DequantInt4Bf16<QT_SYM_INT4> {};
template <> struct Dequant<QT_ASYM_INT4, __bf16> : DequantInt4Bf16<QT_ASYM_INT4> {};

__device__ inline uint32_t code_word8(const u32x4 &q0, const u32x4 &q1, int s, int p) {
    // 8-bit codes: sub-block s holds two dwords (columns 0..3, 4..7)
    const int w = 2 * (s & 1) + (p >> 1);
    return s < 2 ? q0[w] : q1[w];
}

template <> struct Dequant<QT_SYM_INT8, _Float16> {
    __device__ static uint32_t pair(const TileRegs<QT_SYM_INT8> &t, int s, int p, const DqCtx &cx) {
        const uint32_t hb = t.h[s >> 1];
        const f16x2 d2 = h2((s & 1) ? (hb >> 16) : hb);
        // byte ^ 0x80 = q + 128 (unsigned); 0x6400 | u is the half 1024 + u
        const uint32_t w = code_word8(t.q0, t.q1, s, p) ^ 0x80808080u;
        const f16x2 k1152 = {(_Float16)1152.0f, (_Float16)1152.0f};
        const uint32_t sel = (p & 1) ? 0x04030402u : 0x04010400u;
        return pk((__builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, w, sel)) - k1152) * d2);
    }
};

template <> struct Dequant<QT_SYM_INT8, __bf16> {
    __device__ static uint32_t pair(const TileRegs<QT_SYM_INT8> &t, int s, int p, const DqCtx &cx) {
        float d, mn;
        tile_scale<QT_SYM_INT8>(t, s, d, mn);
        // byte ^ 0x80 = q + 128 as an unsigned byte, converted exactly; (u - 128) * d is one fp32
        // fma, rounded once to bf16
        const uint32_t w = (code_word8(t.q0, t.q1, s, p) ^ 0x80808080u) >> ((p & 1) * 16);
        const float c = -128.0f * d;
        return pk2<__bf16>(fmaf((float)(w & 0xff), d, c), fmaf((float)((w >> 8) & 0xff), d, c));
    }
};

// fp8: exact hardware conversion to fp32, fp32 product with the block scale, one rounding
template <typename AT> struct Dequant<QT_FP8_E4M3, AT> {
    __device__ static uint32_t pair(const TileRegs<QT_FP8_E4M3> &t, int s, int p, const DqCtx &cx) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const float sc = __builtin_bit_cast(float, t.h[0]);
        const uint32_t w = code_word8(t.q0, t.q1, s, p);
        const f32x2 a = (p & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8(w, true) : __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
        return pk2<AT>(a[0] * sc, a[1] * sc);
    }
};

// nf4: fp32 code book in LDS, one rounding after the scale.  Nibble order 0,2,4,6,1,3,5,7:
// columns 2p and 2p+1 sit in nibbles p and p+4.
template <typename AT> struct Dequant<QT_NF4, AT> {
    __device__ static uint32_t pair(const TileRegs<QT_NF4> &t, int s, int p, const DqCtx &cx) {
        const float *lut = (const float *)cx.lut;
        const float d = h2f((s >> 1) ? (t.h[0] >> 16) : (t.h[0] & 0xffff));
        const uint32_t v = t.q0[s] >> (4 * p);
        return pk2<AT>(lut[v & 0xf] * d, lut[(v >> 16) & 0xf] * d);
    }
};

// ------------------------------------------------------------------ kernel

typedef float f32x16 __attribute__((ext_vector_type(16)));

// v_mfma_f32_32x32x16: measured on MI355X at 2.3 PFLOP/s, twice the rate of the 16x16x32 form,
// so the GEMM is built on it.  The accumulator is pinned to accumulation registers, in place,
// through inline assembly: left to the compiler, the 128 accumulators migrate between register
// ranges across the unrolled K steps and get copied back every iteration.
// Waits for every outstanding global load, the LDS-DMA ones included.  Spelled with the builtin
// (s_waitcnt vmcnt(0), other counters untouched) so that the compiler's own wait-count bookkeeping
// sees it: after an opaque inline-asm wait it would still believe the weight loads of the previous
// step to be in flight and wait for them again - in fact for the LDS-DMA loads just issued.
__device__ inline void wait_all_loads() {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}
// Waits until at most N global loads are outstanding (loads retire in order: the N youngest may stay in flight).
template <int N> __device__ inline void wait_loads_but() {
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
    asm volatile("" ::: "memory");
}

// The compiler inserts no wait states for an instruction inside inline assembly: a source register
// written by a VALU instruction within the two instructions ahead of the MFMA (the packed conversion
// that ends a dequantization) needs two wait states before the MFMA may read it.  NOP = false is for
// loops whose operands are ready long before (check_gemm_asm.py verifies that in the generated code):
// with one wave per SIMD every instruction between two MFMAs is issue time the MFMA has to cover.
template <bool NOP = true> __device__ inline void mfma_acc(f32x16 &c, f16x8 a, f16x8 b) {
    if constexpr (NOP) asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
template <bool NOP = true> __device__ inline void mfma_acc(f32x16 &c, bf16x8 a, bf16x8 b) {
    if constexpr (NOP) asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}


}  // namespace lowbit
