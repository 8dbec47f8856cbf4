// Prefill product (large M).  Placeholder dispatch until the MFMA GEMM lands:
// runs the streaming kernel over 16-row slices of x.
#include "lowbit_formats.h"

namespace lowbit {
int launch_gemv(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                int waves, hipStream_t st);

int launch_gemm(const void *x, const void *w, void *y, int qtype, int layout, int act_dtype, int M, int N, int K,
                hipStream_t st) {
    return launch_gemv(x, w, y, qtype, layout, act_dtype, M, N, K, 0, st);
}
}  // namespace lowbit
