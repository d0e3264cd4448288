// Prefill GEMM (M > 1) on MFMA -- placeholder until the tiled kernel lands: reports
// "unsupported" so that mi_linear runs the batched GEMV for every M.
#include "common.h"

namespace mi {

bool gemm_supported(WeightKind, int, int, int) { return false; }

bool launch_gemm(hipStream_t, WeightKind, int, int, int, const void*, const void*, const void*, void*) {
    MI_ERROR_FMT("gemm: not built");
    return false;
}

}  // namespace mi
