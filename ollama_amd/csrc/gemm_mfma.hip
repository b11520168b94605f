// Kernel 3: int8-MFMA prefill GEMM (placeholder until the tiled kernel lands; reports "unsupported"
// so the dispatcher keeps batches on the streaming GEMV in column groups).
#include "internal.h"

namespace miqmm {

bool gemm_supports(int, int64_t, int64_t) { return false; }

hipError_t launch_gemm(const DevWeight &, const DevAct &, float *, int64_t, int, hipStream_t) {
    return hipErrorNotSupported;
}

}  // namespace miqmm
