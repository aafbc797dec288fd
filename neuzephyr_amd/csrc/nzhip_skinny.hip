// Bandwidth-bound GEMM kernels for very few output rows (M <= 8): GEMV-shaped products such
// as a single sample through Model::Linear or the M = 1 case of TensorCoreGEMMParallel
// (src/OperationKernels.cu:914-1026), where an MFMA tile would be 97 % padding.
#include <hip/hip_runtime.h>

#include "nzhip_internal.h"

namespace nzhip {

bool gemm_skinny_applicable(const nzhip_gemm_desc&) { return false; }

int gemm_skinny_dispatch(const nzhip_gemm_desc&, hipStream_t) {
    return set_error(NZHIP_E_UNSUPPORTED, "skinny GEMM path not built");
}

}  // namespace nzhip
