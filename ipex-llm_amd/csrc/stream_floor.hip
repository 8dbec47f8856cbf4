// What a launch that only READS n bytes costs on this machine: the floor that the decode GEMV (gemv.hip) is
// measured against.  Not part of the product library: bench.py --floor-only loads libstream_floor.so, chains
// launches over distinct buffers in a HIP graph exactly as it does for the GEMV's roofline figure, and reports the
// empty launch and the fastest and slowest of these access patterns.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum { FLOOR_NT = 1, FLOOR_INTERLEAVE = 2 };

// WAVES waves per workgroup, each wave reads U KiB in U instructions of 64 lanes x 16 bytes, all issued before the
// first use.  Plain: a wave's U KiB are contiguous; interleaved: instruction i of wave w reads KiB i * WAVES + w of
// the workgroup's block.
template <int WAVES, int U, int FLAGS>
__global__ __launch_bounds__(64 * WAVES) void floor_read_kernel(const u32x4 *__restrict__ src, uint32_t *out, size_t n16) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t wg_base = (size_t)blockIdx.x * WAVES * U * 64;
    u32x4 v[U];
#pragma unroll
    for (int i = 0; i < U; i++) {
        size_t idx = (FLAGS & FLOOR_INTERLEAVE) ? wg_base + ((size_t)i * WAVES + wave) * 64 + lane
                                                : wg_base + ((size_t)wave * U + i) * 64 + lane;
        idx = idx < n16 ? idx : n16 - 1;
        if constexpr (FLAGS & FLOOR_NT) v[i] = __builtin_nontemporal_load(src + idx);
        else v[i] = src[idx];
    }
    // (left alone the compiler issues two loads, consumes the first and only then issues the next: the wave
    // then has two loads in flight instead of U)
    __builtin_amdgcn_sched_barrier(0);
    uint32_t a = 0;
#pragma unroll
    for (int i = 0; i < U; i++) a ^= v[i][0] ^ v[i][1] ^ v[i][2] ^ v[i][3];
    if (a == 0x12345678u) out[0] = a;              // (keeps the loads alive; the buffers never hold this value)
}

// The weight access pattern of the grouped GEMM (lowbit_gemm_kernel.h): a workgroup of four waves owns 16 tile rows
// (256 weight rows), a wave walks its four tile rows side by side, one tile of each per K step (the first two KiB
// of a tile: the codes of an 8-bit format).  tiles_per_row tiles of tile_bytes bytes per tile row.
__global__ __launch_bounds__(256) void floor_read_tiles_kernel(const uint8_t *const *__restrict__ weights, uint32_t *out,
                                                               int tile_rows, int tiles_per_row, int tile_bytes) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t *w = weights[blockIdx.y];                   // one weight per blockIdx.y, as one expert's
    const int64_t r0 = ((int64_t)blockIdx.x * 4 + wave) * 4;
    if (r0 + 4 > tile_rows) return;
    u32x4 acc = {0, 0, 0, 0};
#pragma unroll 2
    for (int s = 0; s < tiles_per_row; s++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint8_t *t = w + ((r0 + r) * tiles_per_row + s) * (int64_t)tile_bytes;
            acc ^= *(const u32x4 *)(t + lane * 16);
            acc ^= *(const u32x4 *)(t + 1024 + lane * 16);
        }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[0] = 1;
}

__global__ void floor_empty_kernel(uint32_t *out) {
    if (out == nullptr) __builtin_trap();          // never: a kernel with no work at all
}

template <int WAVES, int U, int FLAGS>
static int launch_read(const void *buf, size_t bytes, uint32_t *out, hipStream_t st) {
    const size_t n16 = bytes / 16, per_wg = (size_t)WAVES * U * 64;
    hipLaunchKernelGGL((floor_read_kernel<WAVES, U, FLAGS>), dim3((unsigned)((n16 + per_wg - 1) / per_wg)), dim3(64 * WAVES), 0,
                       st, (const u32x4 *)buf, out, n16);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

extern "C" {

int stream_floor_patterns(void) { return 12; }

// Name of pattern p: "<waves per workgroup>x<KiB per wave>[ interleaved][ nontemporal]"
const char *stream_floor_pattern_name(int p) {
    static const char *names[] = {"4x4", "4x8", "8x4", "8x8", "16x2", "16x4", "8x4 interleaved", "16x4 interleaved",
                                  "8x4 nontemporal", "8x8 nontemporal", "16x4 nontemporal", "16x8"};
    return p >= 0 && p < 12 ? names[p] : "";
}

// One launch that reads bytes (a multiple of 16) from buf with pattern p; out: 4 bytes of device memory.
int stream_floor_read(const void *buf, size_t bytes, int p, void *out, void *stream) {
    hipStream_t st = (hipStream_t)stream;
    uint32_t *o = (uint32_t *)out;
    if (!buf || !out || (bytes & 15) || bytes == 0) return -1;
    switch (p) {
    case 0: return launch_read<4, 4, 0>(buf, bytes, o, st);
    case 1: return launch_read<4, 8, 0>(buf, bytes, o, st);
    case 2: return launch_read<8, 4, 0>(buf, bytes, o, st);
    case 3: return launch_read<8, 8, 0>(buf, bytes, o, st);
    case 4: return launch_read<16, 2, 0>(buf, bytes, o, st);
    case 5: return launch_read<16, 4, 0>(buf, bytes, o, st);
    case 6: return launch_read<8, 4, FLOOR_INTERLEAVE>(buf, bytes, o, st);
    case 7: return launch_read<16, 4, FLOOR_INTERLEAVE>(buf, bytes, o, st);
    case 8: return launch_read<8, 4, FLOOR_NT>(buf, bytes, o, st);
    case 9: return launch_read<8, 8, FLOOR_NT>(buf, bytes, o, st);
    case 10: return launch_read<16, 4, FLOOR_NT>(buf, bytes, o, st);
    case 11: return launch_read<16, 8, 0>(buf, bytes, o, st);
    default: return -1;
    }
}

// One launch that reads n_weights tiled weights (a table of device pointers in device memory; each tile_rows rows
// of tiles_per_row tiles, tile_bytes >= 2048 each, tile_rows a multiple of 16) the way the grouped GEMM walks them.
int stream_floor_read_tiles(const void *const *weights, int n_weights, int tile_rows, int tiles_per_row, int tile_bytes,
                            void *out, void *stream) {
    if (!weights || !out || n_weights <= 0 || n_weights > 65535 || tile_rows <= 0 || (tile_rows % 16) || tiles_per_row <= 0 ||
        tile_bytes < 2048 || (tile_bytes % 16))
        return -1;
    hipLaunchKernelGGL(floor_read_tiles_kernel, dim3(tile_rows / 16, n_weights), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t *const *)weights, (uint32_t *)out, tile_rows, tiles_per_row, tile_bytes);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int stream_floor_empty(void *out, void *stream) {
    hipLaunchKernelGGL(floor_empty_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (uint32_t *)out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // extern "C"
