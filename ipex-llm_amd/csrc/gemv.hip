// Decode-time product y[M,N] = x[M,K] * dequant(W)[N,K]^T for small M.
//
// Replaces xe_linear.forward_new at M = 1 and xe_batch.batch_forward at small M
// (python/llm/src/ipex_llm/transformers/low_bit_linear.py:657-668).
//
// gemv_mfma_kernel (tiled layout): HBM-bound streaming of the packed weights.
//   One workgroup owns one tile row (16 output columns) and its waves split
//   the 128-column tiles along K.  A lane's 16-byte load of a tile is already
//   its B operand for four v_mfma_f32_16x16x32 (one per 32-column sub-block);
//   codes are turned into exact small numbers in registers (never scaled in
//   half precision), the activations are the A operand (rows = batch index),
//   and the block scale is applied to the fp32 MFMA result.  M <= 16 costs the
//   same weight traffic as M = 1.  Algorithmic bytes per launch:
//   N*K*TS/QK (weights) + M*K*2 (x) + M*N*2 (y).
// gemv_generic_kernel: any layout / any shape fallback, one wave per row.
#include "lowbit_mfma.h"

namespace lowbit {

// ---- codes of one sub-block (8 columns of this lane) -> B operand ----------
//
// The operand holds the *unscaled* code value (q - 8, q, int8, e4m3 value, nf4
// code-book entry); OFFSET<> says what constant is still folded in and has to
// be removed with the row sum of x (0 for every path below except bf16 4-bit).

template <int QT, typename AT> struct Unpack;

// 4-bit integer codes, fp16: 0x6400 | q is the half 1024 + q; 0x6400 | q << 4 is 1024 + 16 q.
template <> struct Unpack<QT_SYM_INT4, _Float16> {
    static constexpr float OFFSET = 0.0f;
    __device__ static f16x8 run(uint32_t v, const void *, uint32_t magic) {
        const f16x2 k1032 = {(_Float16)1032.0f, (_Float16)1032.0f};
        const f16x2 k16th = {(_Float16)0.0625f, (_Float16)0.0625f};
        const f16x2 k72 = {(_Float16)72.0f, (_Float16)72.0f};
        const uint32_t v8 = v >> 8;
        f16x2 t0 = __builtin_bit_cast(f16x2, and_or(v, 0x000f000fu, magic)) - k1032;
        f16x2 t1 = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, and_or(v, 0x00f000f0u, magic)), k16th, -k72);
        f16x2 t2 = __builtin_bit_cast(f16x2, and_or(v8, 0x000f000fu, magic)) - k1032;
        f16x2 t3 = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, and_or(v8, 0x00f000f0u, magic)), k16th, -k72);
        return f16x8{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
    }
};
template <> struct Unpack<QT_ASYM_INT4, _Float16> {
    static constexpr float OFFSET = 0.0f;
    __device__ static f16x8 run(uint32_t v, const void *, uint32_t magic) {
        const f16x2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const f16x2 k16th = {(_Float16)0.0625f, (_Float16)0.0625f};
        const f16x2 k64 = {(_Float16)64.0f, (_Float16)64.0f};
        const uint32_t v8 = v >> 8;
        f16x2 t0 = __builtin_bit_cast(f16x2, and_or(v, 0x000f000fu, magic)) - k1024;
        f16x2 t1 = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, and_or(v, 0x00f000f0u, magic)), k16th, -k64);
        f16x2 t2 = __builtin_bit_cast(f16x2, and_or(v8, 0x000f000fu, magic)) - k1024;
        f16x2 t3 = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, and_or(v8, 0x00f000f0u, magic)), k16th, -k64);
        return f16x8{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
    }
};
// 4-bit integer codes, bf16: 0x4300 | q is the bf16 128 + q (exact); the constant is removed
// afterwards through the row sum of x, which a second MFMA against all-ones provides.
template <int QT> struct UnpackInt4Bf16 {
    static constexpr float OFFSET = (QT == QT_SYM_INT4) ? 136.0f : 128.0f;
    __device__ static bf16x8 run(uint32_t v, const void *, uint32_t magic) {
        u32x4 t;
        t[0] = and_or(v, 0x000f000fu, magic);
        t[1] = and_or(v >> 4, 0x000f000fu, magic);
        t[2] = and_or(v >> 8, 0x000f000fu, magic);
        t[3] = and_or(v >> 12, 0x000f000fu, magic);
        return __builtin_bit_cast(bf16x8, t);
    }
};
template <> struct Unpack<QT_SYM_INT4, __bf16> : UnpackInt4Bf16<QT_SYM_INT4> {};
template <> struct Unpack<QT_ASYM_INT4, __bf16> : UnpackInt4Bf16<QT_ASYM_INT4> {};

// nf4: code-book lookup, two ways.
//   - From a 16-entry table in LDS: eight 2-byte reads and about twelve vector instructions per dword of codes.
//   - In registers: the 16 entries, already in the activation type, lie in two byte planes (low bytes, high bytes)
//     of four registers each; v_perm_b32 looks four codes up at a time in the eight bytes of a register pair -
//     entries 0..7 and 8..15 separately, a third v_perm_b32 picks per byte by the code's bit 3 - and two more
//     interleave the planes into 16-bit values: 21 vector instructions per dword of eight codes, no LDS access.
// Measured on one MI355X on the Llama-3-70B linear set (419 MB of nf4 weights, bf16): at M = 1 from LDS 115.9 us,
// in registers 123.0, half of the sub-blocks each way 117.7; at M = 16, where x takes its share of the LDS pipe,
// 171.4 / 156.7 / 165.6.  So up to four rows of x look up in LDS and more rows in registers.  Either way nf4 stays
// a quarter behind sym_int4 at the same bytes ([28672 x 8192] at M = 1: 31.7 against 25.5 us): the lookups are
// instructions the integer formats do not issue, whichever unit takes them.
struct Nf4Planes {
    uint32_t lo[4], hi[4];        // byte i % 4 of register i / 4 = low / high byte of entry i
    uint32_t k04, k0123;          // 0x04040404 and 0x03020100 in vector registers: as literals the two would need the
                                  // one constant slot of v_and_or_b32 twice
};
// RESID: what rounding the code book to AT dropped (the second term of the fp32-output variants)
template <typename AT, bool RESID> __device__ inline Nf4Planes nf4_planes() {
    Nf4Planes t = {};
#pragma unroll
    for (int i = 0; i < 16; i++) {                      // (constants: folded at compile time)
        const AT main = to_at<AT>(NF4_CODEBOOK[i]);
        const AT v = RESID ? to_at<AT>(NF4_CODEBOOK[i] - (float)main) : main;
        const uint32_t b = __builtin_bit_cast(uint16_t, v);
        t.lo[i / 4] |= (b & 0xffu) << (8 * (i % 4));
        t.hi[i / 4] |= (b >> 8) << (8 * (i % 4));
    }
    asm("v_mov_b32 %0, 0x04040404" : "=v"(t.k04));
    asm("v_mov_b32 %0, 0x03020100" : "=v"(t.k0123));
    return t;
}
template <typename AT> struct Unpack<QT_NF4, AT> {
    static constexpr float OFFSET = 0.0f;
    // four codes, one per byte of `sel` (bits 0..2) and `mrg` (0x03020100 + 4 * bit 3 per byte) -> one byte plane
    __device__ static uint32_t plane4(const uint32_t (&p)[4], uint32_t sel, uint32_t mrg) {
        return __builtin_amdgcn_perm(__builtin_amdgcn_perm(p[3], p[2], sel), __builtin_amdgcn_perm(p[1], p[0], sel), mrg);
    }
    __device__ static typename Vec8<AT>::type run(uint32_t v, const void *planes_, uint32_t) {
        const Nf4Planes &t = *(const Nf4Planes *)planes_;
        // nibbles 0, 2, 4, 6 (columns 0, 4, 1, 5) are the low nibbles of the four bytes, 1, 3, 5, 7 (columns 2, 6,
        // 3, 7) the high ones
        const uint32_t sel_e = v & 0x07070707u, mrg_e = and_or(v >> 1, t.k04, t.k0123);
        const uint32_t sel_o = (v >> 4) & 0x07070707u, mrg_o = and_or(v >> 5, t.k04, t.k0123);
        const uint32_t lo_e = plane4(t.lo, sel_e, mrg_e), hi_e = plane4(t.hi, sel_e, mrg_e);
        const uint32_t lo_o = plane4(t.lo, sel_o, mrg_o), hi_o = plane4(t.hi, sel_o, mrg_o);
        u32x4 r;
        r[0] = __builtin_amdgcn_perm(hi_e, lo_e, 0x06020400u);      // columns 0, 1: bytes 0 and 2 of the even set
        r[1] = __builtin_amdgcn_perm(hi_o, lo_o, 0x06020400u);      // columns 2, 3
        r[2] = __builtin_amdgcn_perm(hi_e, lo_e, 0x07030501u);      // columns 4, 5: bytes 1 and 3
        r[3] = __builtin_amdgcn_perm(hi_o, lo_o, 0x07030501u);      // columns 6, 7
        return __builtin_bit_cast(typename Vec8<AT>::type, r);
    }
    __device__ static typename Vec8<AT>::type run_lds(uint32_t v, const AT *lut) {
        typename Vec8<AT>::type r;
        r[0] = lut[v & 0xf]; r[2] = lut[(v >> 4) & 0xf]; r[4] = lut[(v >> 8) & 0xf]; r[6] = lut[(v >> 12) & 0xf];
        r[1] = lut[(v >> 16) & 0xf]; r[3] = lut[(v >> 20) & 0xf]; r[5] = lut[(v >> 24) & 0xf]; r[7] = lut[v >> 28];
        return r;
    }
};

// 8-bit codes: two dwords (columns 0..3, 4..7).
template <int QT, typename AT> struct Unpack8;
template <> struct Unpack8<QT_SYM_INT8, _Float16> {
    __device__ static f16x8 run(uint32_t lo, uint32_t hi) {
        // byte ^ 0x80 = q + 128 (unsigned); 0x6400 | u is the half 1024 + u
        const f16x2 k1152 = {(_Float16)1152.0f, (_Float16)1152.0f};
        const uint32_t a = lo ^ 0x80808080u, b = hi ^ 0x80808080u;
        const uint32_t c64 = 0x64646464u;
        f16x2 t0 = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(c64, a, 0x04010400u)) - k1152;
        f16x2 t1 = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(c64, a, 0x04030402u)) - k1152;
        f16x2 t2 = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(c64, b, 0x04010400u)) - k1152;
        f16x2 t3 = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(c64, b, 0x04030402u)) - k1152;
        return f16x8{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
    }
};
template <> struct Unpack8<QT_SYM_INT8, __bf16> {
    __device__ static bf16x8 run(uint32_t lo, uint32_t hi) {
        bf16x8 r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r[i] = (__bf16)(float)(int8_t)(lo >> (8 * i));      // |q| <= 128: exact in bf16
            r[4 + i] = (__bf16)(float)(int8_t)(hi >> (8 * i));
        }
        return r;
    }
};
template <> struct Unpack8<QT_FP8_E4M3, _Float16> {
    __device__ static f16x8 run(uint32_t lo, uint32_t hi) {
        f16x2 t0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false);
        f16x2 t1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true);
        f16x2 t2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false);
        f16x2 t3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true);
        return f16x8{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
    }
};
template <> struct Unpack8<QT_FP8_E4M3, __bf16> {
    __device__ static bf16x8 run(uint32_t lo, uint32_t hi) {
        bf16x2 t0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
        bf16x2 t1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
        bf16x2 t2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
        bf16x2 t3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
        return bf16x8{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
    }
};

template <int QT, typename AT> constexpr float code_offset() {
    if constexpr (Fmt<QT>::BITS == 4) return Unpack<QT, AT>::OFFSET;
    else return 0.0f;
}

template <typename AT> __device__ inline typename Vec8<AT>::type ones8() {
    typename Vec8<AT>::type r;
#pragma unroll
    for (int i = 0; i < 8; i++) r[i] = to_at<AT>(1.0f);
    return r;
}

// ------------------------------------------------------------ MFMA GEMV

constexpr int GEMV_MAX_WAVES = 16;

// activation of the gate branch: 0 = SiLU, 1 = GELU in its tanh form (what Gemma uses)
__device__ inline float gate_act(float g, int act) {
    if (act == 0) return g / (1.0f + __expf(-g));
    const float t = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
    return 0.5f * g * (1.0f + t);
}
constexpr int GEMV_LDS_X_BUDGET = 64 * 1024;

// One workgroup = one tile row (16 output columns).  Per round, wave w owns U consecutive
// tiles along K: it first issues every weight load of the round (so the whole slice is in
// flight at once), then copies its slice of x into a wave-private LDS region, then runs
// 4*U MFMAs whose A operand comes from LDS.  Rounds repeat until K is covered.
//
// DUAL: the fused gate/up projection of a gated MLP (xe_linear.mlp_forward_xpu,
// python/llm/src/ipex_llm/transformers/models/common.py:145-158): the workgroup walks the same
// tile row of two weights with one copy of x and writes act(x Wg^T) * (x Wu^T).
//
// MOE: the two launches of a fused mixture-of-experts decode step (xe_linear.moe_forward_vec,
// python/llm/src/ipex_llm/transformers/models/deepseek.py:290-315).  w / w2 are then tables of
// weight pointers in device memory and ids[j] names the expert of routing slot j, so that the host
// never has to read the routing result.
//   MOE == 1 (with DUAL): blockIdx.y = slot j; row j of y = act(x Wg[e]^T) * (x Wu[e]^T).
//   MOE == 2: x is the [slots, K / slots] output of the first launch, read as one long vector;
//             tile g of the K walk belongs to slot g / ge and is scaled by route_w[slot]:
//             y = sum_j route_w[j] * (x_j Wd[e_j]^T).
//
// F32OUT: y is float [M, N] instead of AT (the fp32 path of lowbit_forward_f32: x arrives as two bf16 planes,
// the sums must not be rounded to 8 bits on the way out).
template <int QT, typename AT, int MT, int U, int XN, bool DUAL, int MOE, int R, bool F32OUT>
__global__ __launch_bounds__(1024) void gemv_mfma_kernel(const AT *__restrict__ x, const uint8_t *__restrict__ w,
                                                         const uint8_t *__restrict__ w2, AT *__restrict__ y, int M,
                                                         int N, int K, int act, const int32_t *__restrict__ ids,
                                                         const float *__restrict__ route_w, int ge, int n_exp) {
    using F = Fmt<QT>;
    using V8 = typename Vec8<AT>::type;
    constexpr bool IS4 = (F::BITS == 4);
    constexpr bool ASYM = (QT == QT_ASYM_INT4);
    constexpr float OFFSET = code_offset<QT, AT>();
    constexpr bool NEED_S = ASYM || OFFSET != 0.0f;
    constexpr int SLICE = U * TILE_COLS;                    // columns of x per wave and round
    constexpr bool ZERO_X = XN == 1;                        // how tiles past K are silenced (see the x loads)

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // tile rows walked side by side with one copy of x: the same row of two weights (DUAL) or R
    // consecutive rows of one weight (worth it when M is large and N gives enough workgroups: at
    // M = 16 a workgroup otherwise pulls 3.5 bytes of x out of L2 per byte of weight)
    constexpr int NW = DUAL ? 2 : R;
    static_assert(!(DUAL && R != 1) && XN * 1024 >= NW * MT * 256, "bad GEMV shape parameters");
    // nf4 code book in the activation type (byte planes in registers).  With fp32 output a second table holds what
    // the rounding to AT dropped, and a second MFMA per sub-block adds it: the weights then carry 16 mantissa bits
    // like x does.
    const Nf4Planes lut_planes = (QT == QT_NF4) ? nf4_planes<AT, false>() : Nf4Planes{};
    const Nf4Planes lut_lo_planes = (QT == QT_NF4 && F32OUT) ? nf4_planes<AT, true>() : Nf4Planes{};
    const void *const lut = &lut_planes, *const lut_lo = &lut_lo_planes;
    constexpr bool NF4_IN_LDS = QT == QT_NF4 && MT == 1 && !F32OUT;     // (see Unpack<QT_NF4>)
    __shared__ AT lut_lds[16];
    if constexpr (NF4_IN_LDS) {
        if (threadIdx.x < 16) lut_lds[threadIdx.x] = to_at<AT>(NF4_CODEBOOK[threadIdx.x]);
        __syncthreads();
    }

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, W = blockDim.x >> 6;
    const int G = K / TILE_COLS;
    const int r = lane & 15, c = lane >> 4;
    // A rows: row r carries batch index (r/4)*MT + r%4 when r%4 < MT, so that the C registers
    // i < MT of lane group g hold batch indices g*MT + i and nothing else has to be scaled.
    // Rows with r%4 >= MT (and batch indices >= M) only feed C rows that are never read, so
    // they may hold anything: they re-read a valid row, which LDS serves as a broadcast.
    int m_of_r = (r >> 2) * MT + ((r & 3) < MT ? (r & 3) : MT - 1);
    m_of_r = m_of_r < M ? m_of_r : M - 1;
    gbytes wrow = nullptr, wrow2 = nullptr;
    if constexpr (MOE == 0) {
        wrow = (gbytes)w + (int64_t)blockIdx.x * R * G * F::TILE_BYTES;
        if constexpr (DUAL) wrow2 = (gbytes)w2 + (int64_t)blockIdx.x * G * F::TILE_BYTES;
    } else if constexpr (MOE == 1) {
        // ids come from device memory: clamp, so that a bad id cannot send a load astray
        const int e = min(max(ids[blockIdx.y], 0), n_exp - 1);
        wrow = (gbytes)((const uint8_t *const *)w)[e] + (int64_t)blockIdx.x * G * F::TILE_BYTES;
        wrow2 = (gbytes)((const uint8_t *const *)w2)[e] + (int64_t)blockIdx.x * G * F::TILE_BYTES;
        y += (int64_t)blockIdx.y * N;
    }
    // MOE == 2: tile g -> slot g / ge; its weight row starts at table[ids[slot]] + blockIdx.x * ge tiles
    auto moe_tile = [&](int g, float &rw) -> gbytes {
        const int slot = g / ge;
        rw = route_w[slot];
        return (gbytes)((const uint8_t *const *)w)[min(max(ids[slot], 0), n_exp - 1)] +
               ((int64_t)blockIdx.x * ge + (g - slot * ge)) * F::TILE_BYTES;
    };
    AT *xs = (AT *)smem + (int64_t)wave * (XN * 512);       // [XN*64/(SLICE/8)][SLICE], private to this wave
    const AT *xa = xs + m_of_r * SLICE + 8 * c;

    float acc[NW * MT];
#pragma unroll
    for (int i = 0; i < NW * MT; i++) acc[i] = 0.0f;
    const V8 ones = ones8<AT>();
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    // exponent pattern OR-ed onto 4-bit codes (fp16 1024, bf16 128), held in a vector register: as a
    // literal it would share the instruction's one constant slot with the nibble mask and split every
    // v_and_or_b32 into an AND and an OR
    uint32_t magic;
    if constexpr (sizeof(AT) == 2 && __is_same(AT, _Float16)) asm("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    else asm("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    for (int g0 = 0; g0 < G; g0 += W * U) {
        const int gw = g0 + wave * U;
        // Straight-line loads (addresses clamped instead of branches, so that the compiler can
        // count outstanding loads): x first - it comes from L2 and is needed before any MFMA -
        // then every weight tile of the round.  Loads return in order, so the LDS copy of x
        // waits for the x loads only and each tile is consumed as soon as it lands while the
        // later ones are still in flight.  XN = 16-byte chunks of x per lane (>= M*U/4).
        u32x4 xv[XN];
#pragma unroll
        for (int i = 0; i < XN; i++) {
            const int idx = i * 64 + lane;
            int m = idx / (SLICE / 8);
            const int u = idx % (SLICE / 8);
            int col = gw * TILE_COLS + u * 8;
            m = m < M ? m : M - 1;
            // Columns past K (tiles of the last round that a wave has no work for).  With one chunk of x per lane x
            // reads as zero there - the weights of the tile that stands in, the row's last, are finite - which is
            // one select per round where zeroing the scales is one per sub-block (M = 1: [11008 x 4096] 6.23 ->
            // 6.15 us, [28672 x 8192] 24.8 -> 23.8); with more chunks per lane the same change cost 5-20 %, and
            // those shapes zero the scales (below).
            const bool past = col >= K;
            col = past ? K - 8 : col;
            xv[i] = *(const u32x4 *)(x + (int64_t)m * K + col);
            if constexpr (ZERO_X) xv[i] = past ? u32x4{0u, 0u, 0u, 0u} : xv[i];
        }
        __builtin_amdgcn_sched_barrier(0);                  // keep the x loads ahead of the weight loads
        TileRegs<QT> tr[NW * U];
        float rw[U];
#pragma unroll
        for (int t = 0; t < U; t++) {
            const int g = gw + t < G ? gw + t : G - 1;
            rw[t] = 1.0f;
            if constexpr (MOE == 2) load_tile<QT, true>(moe_tile(g, rw[t]), lane, r, tr[t]);
            else load_tile<QT, true>(wrow + (int64_t)g * F::TILE_BYTES, lane, r, tr[t]);
        }
        if constexpr (DUAL) {
#pragma unroll
            for (int t = 0; t < U; t++) {
                const int g = gw + t;
                load_tile<QT, true>(wrow2 + (int64_t)(g < G ? g : G - 1) * F::TILE_BYTES, lane, r, tr[U + t]);
            }
        }
#pragma unroll
        for (int wi = 1; wi < R; wi++)
#pragma unroll
            for (int t = 0; t < U; t++) {
                const int g = gw + t < G ? gw + t : G - 1;
                load_tile<QT, true>(wrow + ((int64_t)wi * G + g) * F::TILE_BYTES, lane, r, tr[wi * U + t]);
            }

        __builtin_amdgcn_sched_barrier(0);
        // The LDS region is private to the wave and LDS operations of a wave execute in order:
        // a wavefront-scope fence (no hardware wait) is all the synchronization it needs.
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < XN; i++) *(u32x4 *)(xs + (i * 64 + lane) * 8) = xv[i];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();

#pragma unroll
        for (int wi = 0; wi < NW; wi++)
#pragma unroll
            for (int t = 0; t < U; t++) {
                const TileRegs<QT> &tl = tr[wi * U + t];
                const bool live = ZERO_X || gw + t < G;
                V8 a[4];
#pragma unroll
                for (int j = 0; j < 4; j++) a[j] = *(const V8 *)(xa + (t * 4 + j) * 32);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    V8 b;
                    if constexpr (NF4_IN_LDS) b = Unpack<QT, AT>::run_lds(tl.q0[j], lut_lds);
                    else if constexpr (IS4) b = Unpack<QT, AT>::run(tl.q0[j], lut, magic);
                    else if (j < 2) b = Unpack8<QT, AT>::run(tl.q0[2 * j], tl.q0[2 * j + 1]);
                    else b = Unpack8<QT, AT>::run(tl.q1[2 * (j - 2)], tl.q1[2 * (j - 2) + 1]);
                    float d, mn;
                    tile_scale<QT>(tl, j, d, mn);
                    if constexpr (MOE == 2) {
                        d *= rw[t];
                        mn *= rw[t];
                    }
                    if constexpr (!ZERO_X) {
                        d = live ? d : 0.0f;
                        mn = live ? mn : 0.0f;
                    }
                    f32x4 p = mfma16(a[j], b, zero4);
                    if constexpr (QT == QT_NF4 && F32OUT) p = mfma16(a[j], Unpack<QT, AT>::run(tl.q0[j], lut_lo, magic), p);
                    if constexpr (NEED_S) {
                        const f32x4 s = mfma16(a[j], ones, zero4);
                        const float e = mn - OFFSET * d;
#pragma unroll
                        for (int i = 0; i < MT; i++)
                            acc[wi * MT + i] = fmaf(e, s[i], fmaf(d, p[i], acc[wi * MT + i]));
                    } else {
#pragma unroll
                        for (int i = 0; i < MT; i++) acc[wi * MT + i] = fmaf(d, p[i], acc[wi * MT + i]);
                    }
                }
            }
    }

    // sum the K-slices of the waves; wave 0 writes.  C layout: lane = 16*grp + col, register i = row 4*grp + i.
    // The partial sums go to the start of each wave's own x region, which is dead by now.
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    float *red = (float *)smem;
    constexpr int RS = XN * 256;                            // floats per wave region
#pragma unroll
    for (int i = 0; i < NW * MT; i++) red[wave * RS + i * 64 + lane] = acc[i];
    __syncthreads();
    // wave v sums and writes tile row v of the R rows (DUAL: wave 0 combines both weights)
    if (wave < (DUAL ? 1 : R)) {
        const int grp = lane >> 4, col = lane & 15;
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float s = 0.0f;
            for (int ww = 0; ww < W; ww++) s += red[ww * RS + (wave * MT + i) * 64 + lane];
            if constexpr (DUAL) {
                float u = 0.0f;
                for (int ww = 0; ww < W; ww++) u += red[ww * RS + (MT + i) * 64 + lane];
                s = gate_act(s, act) * u;
            }
            const int m = grp * MT + i;
            const int64_t at = (int64_t)m * N + ((int64_t)blockIdx.x * R + wave) * 16 + col;
            if constexpr (F32OUT) {
                if (m < M) ((float *)y)[at] = s;
            } else {
                if (m < M) y[at] = to_at<AT>(s);
            }
        }
    }
}

// --------------------------------------------------------- generic GEMV

template <int QT, int LAYOUT, typename AT, int MC, bool F32OUT>
__global__ __launch_bounds__(256) void gemv_generic_kernel(const AT *__restrict__ x, const uint8_t *__restrict__ w,
                                                           AT *__restrict__ y, int m0, int M, int N, int K) {
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    float acc[MC];
#pragma unroll
    for (int i = 0; i < MC; i++) acc[i] = 0.0f;
    const int sbpr = K / 32;
    for (int sb = lane; sb < sbpr; sb += 64) {
        SubBlock s;
        if constexpr (LAYOUT == LAYOUT_GGML) ggml_load_sub<QT>(w, n, K, sb, s);
        else tiled_load_sub<QT>(w, n, K, sb, s);
        float wv[32];
#pragma unroll
        for (int i = 0; i < 32; i++) wv[i] = decode<QT>(s.code[i], s.d, s.m);
#pragma unroll
        for (int mi = 0; mi < MC; mi++) {
            if (m0 + mi < M) {
                const AT *xp = x + (int64_t)(m0 + mi) * K + sb * 32;
                float a = 0.0f;
#pragma unroll
                for (int i = 0; i < 32; i++) a = fmaf((float)xp[i], wv[i], a);
                acc[mi] += a;
            }
        }
    }
#pragma unroll
    for (int mi = 0; mi < MC; mi++) {
        float v = acc[mi];
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if (lane == 0 && m0 + mi < M) {
            if constexpr (F32OUT) ((float *)y)[(int64_t)(m0 + mi) * N + n] = v;
            else y[(int64_t)(m0 + mi) * N + n] = to_at<AT>(v);
        }
    }
}

// -------------------------------------------------------------- launch

template <int QT, typename AT, int MT, int U, int XN, bool DUAL = false, int MOE = 0, int R = 1, bool F32OUT = false>
static void launch_mfma(const AT *x, const uint8_t *w, AT *y, int M, int N, int K, int waves, hipStream_t st,
                        const uint8_t *w2 = nullptr, int act = 0, const int32_t *ids = nullptr,
                        const float *route_w = nullptr, int ge = 0, int slots = 1, int n_exp = 1) {
    const int G = K / TILE_COLS;
    // waves: enough that one round covers K, within the block size limit and the LDS budget for x
    int wv = (G + U - 1) / U;
    const int lds_cap = GEMV_LDS_X_BUDGET / (XN * 512 * (int)sizeof(AT));
    if (wv > lds_cap) wv = lds_cap;
    if (wv > GEMV_MAX_WAVES) wv = GEMV_MAX_WAVES;
    if (waves > 0 && waves < wv) wv = waves;
    if (wv < 1) wv = 1;
    const size_t lds = (size_t)wv * XN * 512 * sizeof(AT);
    hipLaunchKernelGGL((gemv_mfma_kernel<QT, AT, MT, U, XN, DUAL, MOE, R, F32OUT>), dim3(N / TILE_ROWS / R, MOE == 1 ? slots : 1),
                       dim3(64 * wv), lds, st, x, w, w2, y, M, N, K, act, ids, route_w, ge, n_exp);
}

// y in fp32 (see F32OUT): a handful of shapes of the kernel is enough, the path is not a hot one
template <int QT, typename AT>
static int launch_gemv_f32out(const void *x, const void *w, void *y, int layout, int M, int N, int K, hipStream_t st) {
    const bool tiled_ok = layout == LAYOUT_TILED && (N % TILE_ROWS) == 0 && (K % TILE_COLS) == 0;
    if (layout == LAYOUT_TILED && !tiled_ok) return -5;
    if (tiled_ok) {
        for (int m0 = 0; m0 < M; m0 += 16) {
            const int mc = (M - m0) < 16 ? (M - m0) : 16;
            const AT *xp = (const AT *)x + (int64_t)m0 * K;
            AT *yp = (AT *)((float *)y + (int64_t)m0 * N);
            const uint8_t *wp = (const uint8_t *)w;
            if (mc <= 2) launch_mfma<QT, AT, 1, 2, 1, false, 0, 1, true>(xp, wp, yp, mc, N, K, 0, st);
            else if (mc <= 4) launch_mfma<QT, AT, 1, 2, 2, false, 0, 1, true>(xp, wp, yp, mc, N, K, 0, st);
            else if (mc <= 8) launch_mfma<QT, AT, 2, 1, 2, false, 0, 1, true>(xp, wp, yp, mc, N, K, 0, st);
            else launch_mfma<QT, AT, 4, 2, 8, false, 0, 1, true>(xp, wp, yp, mc, N, K, 0, st);
        }
        return 0;
    }
    for (int m0 = 0; m0 < M; m0 += 4)
        hipLaunchKernelGGL((gemv_generic_kernel<QT, LAYOUT_GGML, AT, 4, true>), dim3((N + 3) / 4), dim3(256), 0, st,
                           (const AT *)x, (const uint8_t *)w, (AT *)y, m0, M, N, K);
    return 0;
}

template <int QT, typename AT>
static int launch_gemv_t(const void *x, const void *w, void *y, int layout, int M, int N, int K, int waves,
                         hipStream_t st) {
    const bool tiled_ok = layout == LAYOUT_TILED && (N % TILE_ROWS) == 0 && (K % TILE_COLS) == 0;
    if (layout == LAYOUT_TILED && !tiled_ok) return -5;
    if (tiled_ok) {
        for (int m0 = 0; m0 < M; m0 += 16) {
            const int mc = (M - m0) < 16 ? (M - m0) : 16;
            const AT *xp = (const AT *)x + (int64_t)m0 * K;
            AT *yp = (AT *)y + (int64_t)m0 * N;
            // Tiles per wave and round (U), measured on MI355X: 4 when K fits one round of 8 waves and
            // there are many tile rows to spread over the CUs, else 2 with up to 16 waves and as many
            // rounds as K needs.  XN = 16-byte chunks of x per lane = ceil(M * U / 4).
            const bool u4 = (K / TILE_COLS) <= 32 && N >= 8192;
            const uint8_t *wp = (const uint8_t *)w;
            if (mc <= 4) {
                if (u4) {
                    if (mc == 1) launch_mfma<QT, AT, 1, 4, 1>(xp, wp, yp, mc, N, K, waves, st);
                    else if (mc == 2) launch_mfma<QT, AT, 1, 4, 2>(xp, wp, yp, mc, N, K, waves, st);
                    else launch_mfma<QT, AT, 1, 4, 4>(xp, wp, yp, mc, N, K, waves, st);
                } else {
                    if (mc <= 2) launch_mfma<QT, AT, 1, 2, 1>(xp, wp, yp, mc, N, K, waves, st);
                    else launch_mfma<QT, AT, 1, 2, 2>(xp, wp, yp, mc, N, K, waves, st);
                }
            }
            // 5 .. 8 rows: one tile per wave and round with up to 16 waves keeps the x slice of a wave (and with
            // it the workgroup's LDS footprint) small; two tile rows share x where N leaves enough workgroups
            // (measured on MI355X, sym_int4: 5-7 % on the Llama-2-7B shapes, 15-20 % on [28672 x 8192] and
            // [8192 x 28672] against four tiles per wave)
            else if (mc <= 8 && (N / TILE_ROWS) % 2 == 0 && N >= 8192)
                launch_mfma<QT, AT, 2, 1, 2, false, 0, 2>(xp, wp, yp, mc, N, K, waves, st);
            else if (mc <= 8) launch_mfma<QT, AT, 2, 1, 2>(xp, wp, yp, mc, N, K, waves, st);
            // 9 .. 16 rows of x: share x between 4 or 2 tile rows where N still gives enough workgroups
            // (measured on MI355X: +25 .. 70 % on [28672 x 8192], +8 .. 24 % on [8192 x 8192])
            else if ((N / TILE_ROWS) % 4 == 0 && N >= 16384)
                launch_mfma<QT, AT, 4, 1, 4, false, 0, 4>(xp, wp, yp, mc, N, K, waves, st);
            else if ((N / TILE_ROWS) % 2 == 0 && N >= 8192 && K >= 8192)
                launch_mfma<QT, AT, 4, 1, 4, false, 0, 2>(xp, wp, yp, mc, N, K, waves, st);
            else if ((N / TILE_ROWS) % 2 == 0 && N >= 8192)
                launch_mfma<QT, AT, 4, 2, 8, false, 0, 2>(xp, wp, yp, mc, N, K, waves, st);
            else launch_mfma<QT, AT, 4, 2, 8>(xp, wp, yp, mc, N, K, waves, st);
        }
        return 0;
    }
    for (int m0 = 0; m0 < M; m0 += 4)
        hipLaunchKernelGGL((gemv_generic_kernel<QT, LAYOUT_GGML, AT, 4, false>), dim3((N + 3) / 4), dim3(256), 0, st,
                           (const AT *)x, (const uint8_t *)w, (AT *)y, m0, M, N, K);
    return 0;
}

template <int QT>
static int launch_gemv_q(const void *x, const void *w, void *y, int layout, int dt, int M, int N, int K, int waves,
                         hipStream_t st) {
    if (dt == DT_F16) return launch_gemv_t<QT, _Float16>(x, w, y, layout, M, N, K, waves, st);
    if (dt == DT_BF16) return launch_gemv_t<QT, __bf16>(x, w, y, layout, M, N, K, waves, st);
    return -4;
}

template <int QT, typename AT>
static int launch_mlp_t(const void *x, const void *wg, const void *wu, void *y, int M, int N, int K, int act,
                        hipStream_t st) {
    // Two tiles of each weight per wave and round, at most 8 waves: the registers of four tiles in flight
    // keep the kernel below 80 vector registers, so that a CU holds three workgroups and the 688 workgroups
    // of a [11008 x 4096] pair all run side by side.  With four tiles of each weight the kernel takes 120
    // registers and a third of the workgroups has to wait for a free slot.
    const uint8_t *g = (const uint8_t *)wg, *u = (const uint8_t *)wu;
    for (int m0 = 0; m0 < M; m0 += 16) {             // one pass over both weights per 16 rows
        const int mc = (M - m0) < 16 ? (M - m0) : 16;
        const AT *xp = (const AT *)x + (int64_t)m0 * K;
        AT *yp = (AT *)y + (int64_t)m0 * N;
        if (mc <= 2) launch_mfma<QT, AT, 1, 2, 1, true>(xp, g, yp, mc, N, K, 8, st, u, act);
        else if (mc <= 4) launch_mfma<QT, AT, 1, 2, 2, true>(xp, g, yp, mc, N, K, 8, st, u, act);
        // 5 .. 16 rows: one tile of each weight per wave and round with up to 16 waves, as the plain product's
        // kernels that share x between two tile rows
        else if (mc <= 8) launch_mfma<QT, AT, 2, 1, 2, true>(xp, g, yp, mc, N, K, 0, st, u, act);
        else launch_mfma<QT, AT, 4, 1, 4, true>(xp, g, yp, mc, N, K, 0, st, u, act);
    }
    return 0;
}

template <int QT>
static int launch_mlp_q(const void *x, const void *wg, const void *wu, void *y, int dt, int M, int N, int K, int act,
                        hipStream_t st) {
    if (dt == DT_F16) return launch_mlp_t<QT, _Float16>(x, wg, wu, y, M, N, K, act, st);
    if (dt == DT_BF16) return launch_mlp_t<QT, __bf16>(x, wg, wu, y, M, N, K, act, st);
    return -4;
}

// y[M, N] = act(x Wg^T) * (x Wu^T) in passes of 16 rows, both weights tiled [N, K]
int launch_mlp_gemv(const void *x, const void *wg, const void *wu, void *y, int qtype, int act_dtype, int M, int N,
                    int K, int act, hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    switch (qtype) {
    case QT_SYM_INT4: return launch_mlp_q<QT_SYM_INT4>(x, wg, wu, y, act_dtype, M, N, K, act, st);
    case QT_ASYM_INT4: return launch_mlp_q<QT_ASYM_INT4>(x, wg, wu, y, act_dtype, M, N, K, act, st);
    case QT_SYM_INT8: return launch_mlp_q<QT_SYM_INT8>(x, wg, wu, y, act_dtype, M, N, K, act, st);
    case QT_NF4: return launch_mlp_q<QT_NF4>(x, wg, wu, y, act_dtype, M, N, K, act, st);
    case QT_FP8_E4M3: return launch_mlp_q<QT_FP8_E4M3>(x, wg, wu, y, act_dtype, M, N, K, act, st);
    default: return -2;
    }
}

template <int QT, typename AT>
static int launch_moe_t(const void *x, const int32_t *ids, const float *route_w, int slots, int n_exp, const void *gates,
                        const void *ups, const void *downs, void *h, void *y, int hidden, int inter, int act,
                        hipStream_t st) {
    // h[slots, inter] = act(x Wg[e]^T) * (x Wu[e]^T), then y[hidden] = sum_j route_w[j] * h[j] Wd[e_j]^T
    launch_mfma<QT, AT, 1, 4, 1, true, 1>((const AT *)x, (const uint8_t *)gates, (AT *)h, 1, inter, hidden, 0, st,
                                          (const uint8_t *)ups, act, ids, nullptr, 0, slots, n_exp);
    launch_mfma<QT, AT, 1, 4, 1, false, 2>((const AT *)h, (const uint8_t *)downs, (AT *)y, 1, hidden, slots * inter, 0,
                                           st, nullptr, 0, ids, route_w, inter / TILE_COLS, slots, n_exp);
    return 0;
}

template <int QT>
static int launch_moe_q(const void *x, const int32_t *ids, const float *route_w, int slots, int n_exp, const void *gates,
                        const void *ups, const void *downs, void *h, void *y, int dt, int hidden, int inter, int act,
                        hipStream_t st) {
    if (dt == DT_F16) return launch_moe_t<QT, _Float16>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, hidden, inter, act, st);
    if (dt == DT_BF16) return launch_moe_t<QT, __bf16>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, hidden, inter, act, st);
    return -4;
}

int launch_moe_gemv(const void *x, const int32_t *ids, const float *route_w, int slots, int n_exp, const void *gates,
                    const void *ups, const void *downs, void *h, void *y, int qtype, int act_dtype, int hidden,
                    int inter, int act, hipStream_t st) {
    switch (qtype) {
    case QT_SYM_INT4: return launch_moe_q<QT_SYM_INT4>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, act_dtype, hidden, inter, act, st);
    case QT_ASYM_INT4: return launch_moe_q<QT_ASYM_INT4>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, act_dtype, hidden, inter, act, st);
    case QT_SYM_INT8: return launch_moe_q<QT_SYM_INT8>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, act_dtype, hidden, inter, act, st);
    case QT_NF4: return launch_moe_q<QT_NF4>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, act_dtype, hidden, inter, act, st);
    case QT_FP8_E4M3: return launch_moe_q<QT_FP8_E4M3>(x, ids, route_w, slots, n_exp, gates, ups, downs, h, y, act_dtype, hidden, inter, act, st);
    default: return -2;
    }
}

// x: bf16 [M, K]; y: float [M, N]
int launch_gemv_bf16_f32out(const void *x, const void *w, void *y, int qtype, int layout, int M, int N, int K,
                            hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    switch (qtype) {
    case QT_SYM_INT4: return launch_gemv_f32out<QT_SYM_INT4, __bf16>(x, w, y, layout, M, N, K, st);
    case QT_ASYM_INT4: return launch_gemv_f32out<QT_ASYM_INT4, __bf16>(x, w, y, layout, M, N, K, st);
    case QT_SYM_INT8: return launch_gemv_f32out<QT_SYM_INT8, __bf16>(x, w, y, layout, M, N, K, st);
    case QT_NF4: return launch_gemv_f32out<QT_NF4, __bf16>(x, w, y, layout, M, N, K, st);
    case QT_FP8_E4M3: return launch_gemv_f32out<QT_FP8_E4M3, __bf16>(x, w, y, layout, M, N, K, st);
    default: return -2;
    }
}

int launch_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                int waves, hipStream_t st) {
    if (M == 0 || N == 0) return 0;
    switch (qtype) {
    case QT_SYM_INT4: return launch_gemv_q<QT_SYM_INT4>(x, w, y, layout, act_dtype, M, N, K, waves, st);
    case QT_ASYM_INT4: return launch_gemv_q<QT_ASYM_INT4>(x, w, y, layout, act_dtype, M, N, K, waves, st);
    case QT_SYM_INT8: return launch_gemv_q<QT_SYM_INT8>(x, w, y, layout, act_dtype, M, N, K, waves, st);
    case QT_NF4: return launch_gemv_q<QT_NF4>(x, w, y, layout, act_dtype, M, N, K, waves, st);
    case QT_FP8_E4M3: return launch_gemv_q<QT_FP8_E4M3>(x, w, y, layout, act_dtype, M, N, K, waves, st);
    default: return -2;
    }
}

}  // namespace lowbit
