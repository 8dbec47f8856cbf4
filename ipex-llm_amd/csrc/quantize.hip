// Block quantizers: fp32 [N, K] -> packed low-bit blob, in either layout.
//
// Replaces ggml_quantize_tensor (python/llm/src/ipex_llm/ggml/model/llama/
// llama_cpp.py:946-967, called from low_bit_linear.py:162).  Output bytes are
// identical to the ggml reference quantizers; the arithmetic that decides a
// bit (1/d, x*id + 8.5, the fp16 rounding of d) is written with explicit
// round-to-nearest intrinsics so that no contraction into FMA can happen, and
// the file is compiled with -ffp-contract=off and correctly rounded division.
//
// Work split: QK/4 adjacent lanes own one block, each lane one float4 of it,
// so a wave reads 1 KiB of contiguous fp32 per load.  HBM-bound: 4 B read and
// TS/QK B written per weight.
#include "lowbit_formats.h"

namespace lowbit {

template <int W> __device__ inline float group_max(float v) {
#pragma unroll
    for (int o = W / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, W));
    return v;
}
template <int W> __device__ inline float group_min(float v) {
#pragma unroll
    for (int o = W / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, W));
    return v;
}

// Signed value of the FIRST element with the largest magnitude in the block.
// four floats of the source, which is read once: a nontemporal load
__device__ inline float4 stream4(const float *p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 v = __builtin_nontemporal_load((const f4 *)p);
    return make_float4(v[0], v[1], v[2], v[3]);
}

template <int W> __device__ inline float group_first_absmax_signed(const float4 &v, int lane_in_block) {
    float amax = 0.0f, mx = 0.0f;
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (amax < fabsf(e[i])) { amax = fabsf(e[i]); mx = e[i]; }
    int who = lane_in_block;
#pragma unroll
    for (int o = W / 2; o > 0; o >>= 1) {
        const float oa = __shfl_xor(amax, o, W);
        const float om = __shfl_xor(mx, o, W);
        const int ow = __shfl_xor(who, o, W);
        if (oa > amax || (oa == amax && ow < who)) { amax = oa; mx = om; who = ow; }
    }
    return mx;
}

// Index of the code-book entry nearest to v (ties to the smaller index) = number of midpoints
// below v.  The 15 midpoints (fp32 sums halved, as the reference computes them) sit in LDS and are
// searched by bisection: 4 compares per element instead of 15.
__device__ inline void nf4_fill_mids(float *mids) {
    if (threadIdx.x < 15)
        mids[threadIdx.x] = __fmul_rn(__fadd_rn(NF4_CODEBOOK[threadIdx.x], NF4_CODEBOOK[threadIdx.x + 1]), 0.5f);
    __syncthreads();
}
__device__ inline uint32_t nf4_index(float v, const float *mids) {
    uint32_t idx = 0;
#pragma unroll
    for (int step = 8; step > 0; step >>= 1) idx += (v > mids[idx + step - 1]) ? step : 0;
    return idx;
}

// Header bits and the four codes (one per byte) of this lane's float4; the LPB lanes of a block
// cooperate through shuffles.
template <int QT>
__device__ inline void block_codes(const float4 &v, int lib, uint32_t &hdr, uint32_t &mine, const float *mids) {
    using F = Fmt<QT>;
    constexpr int LPB = F::QK / 4;
    const float e[4] = {v.x, v.y, v.z, v.w};
    hdr = 0;
    mine = 0;                                            // byte i = code of element 4*lib + i
    if constexpr (QT == QT_SYM_INT4) {
        const float mx = group_first_absmax_signed<LPB>(v, lib);
        const float d = __fdiv_rn(mx, -8.0f);
        const float id = (d != 0.0f) ? __fdiv_rn(1.0f, d) : 0.0f;
        hdr = f2h(d);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int q = (int)(int8_t)__fadd_rn(__fmul_rn(e[i], id), 8.5f);
            q = q > 15 ? 15 : q;
            mine |= (uint32_t)(q & 0xff) << (8 * i);
        }
    } else if constexpr (QT == QT_ASYM_INT4) {
        const float mn = group_min<LPB>(fminf(fminf(e[0], e[1]), fminf(e[2], e[3])));
        const float mx = group_max<LPB>(fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3])));
        const float d = __fdiv_rn(__fsub_rn(mx, mn), 15.0f);
        const float id = (d != 0.0f) ? __fdiv_rn(1.0f, d) : 0.0f;
        hdr = (uint32_t)f2h(d) | ((uint32_t)f2h(mn) << 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int q = (int)(int8_t)__fadd_rn(__fmul_rn(__fsub_rn(e[i], mn), id), 0.5f);
            q = q > 15 ? 15 : q;
            mine |= (uint32_t)(q & 0xff) << (8 * i);
        }
    } else if constexpr (QT == QT_SYM_INT8) {
        const float amax = group_max<LPB>(fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3]))));
        const float d = __fdiv_rn(amax, 127.0f);
        const float id = (d != 0.0f) ? __fdiv_rn(1.0f, d) : 0.0f;
        hdr = f2h(d);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int q = (int)(int8_t)roundf(__fmul_rn(e[i], id));
            mine |= (uint32_t)(q & 0xff) << (8 * i);
        }
    } else if constexpr (QT == QT_NF4) {
        const float amax = group_max<LPB>(fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3]))));
        const float id = (amax != 0.0f) ? __fdiv_rn(1.0f, amax) : 0.0f;
        hdr = f2h(amax);
#pragma unroll
        for (int i = 0; i < 4; i++) mine |= nf4_index(__fmul_rn(e[i], id), mids) << (8 * i);
    } else {
        const float amax = group_max<LPB>(fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3]))));
        const float s = __fdiv_rn(amax, 448.0f);
        const float is = (s != 0.0f) ? __fdiv_rn(1.0f, s) : 0.0f;
        hdr = __builtin_bit_cast(uint32_t, s);
#pragma unroll
        for (int i = 0; i < 4; i++) mine |= f32_to_e4m3(__fmul_rn(e[i], is)) << (8 * i);
    }
}

// ggml layout: one thread group per block, written where the block lives.
template <int QT>
__global__ __launch_bounds__(256) void quantize_kernel(const float *__restrict__ src, uint8_t *__restrict__ dst,
                                                       int64_t n_blocks) {
    using F = Fmt<QT>;
    constexpr int LPB = F::QK / 4;                       // lanes per block
    __shared__ float mids[16];
    if constexpr (QT == QT_NF4) nf4_fill_mids(mids);
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t blk = t / LPB;
    const int lib = (int)(t % LPB);
    if (blk >= n_blocks) return;                         // whole LPB-groups leave together
    const float4 v = stream4(src + blk * F::QK + lib * 4);

    uint32_t hdr, mine;
    block_codes<QT>(v, lib, hdr, mine, mids);

    uint8_t *b = dst + blk * F::TS;
    if (lib == 0) {
        *(uint16_t *)b = (uint16_t)hdr;              // every block starts on an even address
        if constexpr (F::HDR == 4) *(uint16_t *)(b + 2) = (uint16_t)(hdr >> 16);
    }
    if constexpr (F::BITS == 4) {
        // byte j = code[j] | code[j + QK/2] << 4: lane i packs its own codes with lane i + LPB/2's
        const uint32_t other = __shfl_down(mine, LPB / 2, LPB);
        if (lib < LPB / 2) {
            const uint32_t out = (mine & 0x0f0f0f0fu) | ((other & 0x0f0f0f0fu) << 4);
            uint16_t *p = (uint16_t *)(b + F::HDR + lib * 4);
            p[0] = (uint16_t)out;
            p[1] = (uint16_t)(out >> 16);
        }
    } else {
        uint16_t *p = (uint16_t *)(b + F::HDR + lib * 4);
        p[0] = (uint16_t)mine;
        p[1] = (uint16_t)(mine >> 16);
    }
}

// Tiled layout, assembled in LDS.  A workgroup owns one tile row (16 rows of W) by QTW tiles
// (QTW * 128 columns): wave w reads rows 4w .. 4w+3, 1 or 2 KiB of contiguous fp32 each, the
// codes are placed into an LDS image of the tiles, and the image goes out with contiguous
// 16-byte stores.  (Writing the 4-byte pieces straight to HBM costs about twice the bytes, since
// the 16 rows of a tile would arrive from different workgroups at different times.)
constexpr int QTW = 4;

template <int QT>
__global__ __launch_bounds__(256) void quantize_tiled_kernel(const float *__restrict__ src, uint8_t *__restrict__ dst,
                                                             int64_t K) {
    using F = Fmt<QT>;
    constexpr int LPB = F::QK / 4;
    __shared__ __attribute__((aligned(16))) uint8_t img[QTW * F::TILE_BYTES];
    __shared__ float mids[16];
    if constexpr (QT == QT_NF4) nf4_fill_mids(mids);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tiles_k = (int)(K / TILE_COLS);
    const int t0 = blockIdx.x * QTW;                                 // first tile of this strip
    const int nt = tiles_k - t0 < QTW ? tiles_k - t0 : QTW;          // tiles in this strip
    const int64_t row0 = (int64_t)blockIdx.y * TILE_ROWS;
    constexpr int PASSES = QTW * TILE_COLS / 256;                    // 256 columns per wave-wide load

    float4 v[4][PASSES];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            int col = ps * 256 + lane * 4;
            col = col < nt * TILE_COLS ? col : 0;                    // past the strip: a valid re-read, not stored
            v[i][ps] = stream4(src + (row0 + wave * 4 + i) * K + (int64_t)t0 * TILE_COLS + col);
        }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            const int r = wave * 4 + i;
            const int col = ps * 256 + lane * 4;
            const int lib = lane % LPB;
            uint32_t hdr, mine;
            block_codes<QT>(v[i][ps], lib, hdr, mine, mids);
            if (col >= nt * TILE_COLS) continue;                      // whole blocks leave together
            uint8_t *tile = img + (col / TILE_COLS) * F::TILE_BYTES;
            const int j = (col % TILE_COLS) / 32;                     // sub-block in the tile
            const int c = (col % 32) / 8;                             // lane group of 8 columns
            if (lib == 0) {
                uint8_t *h = tile + tile_hdr_offset<QT>(r, j);
                if constexpr (F::HDR == 2) *(uint16_t *)h = (uint16_t)hdr;
                else *(uint32_t *)h = hdr;
            }
            if constexpr (F::BITS == 4) {
                const uint32_t other = __shfl_down(mine, 1, LPB);
                if ((lane & 1) == 0) {
                    // mine = columns 0..3 (bytes 0..3), other = columns 4..7; nibble order 0,2,4,6,1,3,5,7
                    const uint32_t out = (mine & 0xf) | (((mine >> 16) & 0xf) << 4) | ((other & 0xf) << 8) |
                                         (((other >> 16) & 0xf) << 12) | (((mine >> 8) & 0xf) << 16) |
                                         (((mine >> 24) & 0xf) << 20) | (((other >> 8) & 0xf) << 24) |
                                         (((other >> 24) & 0xf) << 28);
                    *(uint32_t *)(tile + (c * 16 + r) * 16 + j * 4) = out;
                }
            } else {
                *(uint32_t *)(tile + (j / 2) * 1024 + (c * 16 + r) * 16 + (j % 2) * 8 + (lane & 1) * 4) = mine;
            }
        }
    __syncthreads();
    uint8_t *out = dst + ((int64_t)blockIdx.y * tiles_k + t0) * F::TILE_BYTES;
    const int bytes = nt * F::TILE_BYTES;                             // a multiple of 16
    for (int o = threadIdx.x * 16; o < bytes; o += 256 * 16) *(uint4 *)(out + o) = *(const uint4 *)(img + o);
}

template <int QT> static int launch_q(const float *src, void *dst, int64_t N, int64_t K, int layout, hipStream_t st) {
    using F = Fmt<QT>;
    const int64_t n_blocks = N * K / F::QK;
    const int64_t threads = n_blocks * (F::QK / 4);
    if (threads == 0) return 0;
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7fffffff) return -3;
    if (layout == LAYOUT_GGML)
        hipLaunchKernelGGL((quantize_kernel<QT>), dim3((unsigned)grid), dim3(256), 0, st, src, (uint8_t *)dst, n_blocks);
    else {
        const int64_t strips = (K / TILE_COLS + QTW - 1) / QTW, tile_rows = N / TILE_ROWS;
        if (tile_rows > 65535) return -3;
        hipLaunchKernelGGL((quantize_tiled_kernel<QT>), dim3((unsigned)strips, (unsigned)tile_rows), dim3(256), 0, st, src,
                           (uint8_t *)dst, K);
    }
    return 0;
}

int launch_quantize(const float *src, void *dst, int qtype, int64_t N, int64_t K, int layout, hipStream_t st) {
    switch (qtype) {
    case QT_SYM_INT4: return launch_q<QT_SYM_INT4>(src, dst, N, K, layout, st);
    case QT_ASYM_INT4: return launch_q<QT_ASYM_INT4>(src, dst, N, K, layout, st);
    case QT_SYM_INT8: return launch_q<QT_SYM_INT8>(src, dst, N, K, layout, st);
    case QT_NF4: return launch_q<QT_NF4>(src, dst, N, K, layout, st);
    case QT_FP8_E4M3: return launch_q<QT_FP8_E4M3>(src, dst, N, K, layout, st);
    default: return -2;
    }
}

}  // namespace lowbit
