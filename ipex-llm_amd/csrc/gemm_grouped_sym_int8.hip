// The grouped GEMM kernels (lowbit_gemm_grouped.h) for sym_int8 weights.
#include "lowbit_gemm_grouped.h"

namespace lowbit {

template int launch_grouped_q<QT_SYM_INT8>(const void *, const void *const *, const void *const *, void *, const int32_t *, int, int,
                                    int, int, int, int, const GroupedPlan &, float *, hipStream_t);

template int launch_mlp_gemm_q<QT_SYM_INT8>(const void *, const void *, const void *, void *, int, int, int, int, int, int, bool, hipStream_t);

}  // namespace lowbit
