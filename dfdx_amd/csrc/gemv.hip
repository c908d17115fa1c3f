// Bandwidth-bound vector products (M = 1 or N = 1).
#include "gemm_internal.h"

namespace dfdx_rocm {

bool gemv_supported(const GemmProblem &) { return false; }
hipError_t launch_gemv(const GemmProblem &, hipStream_t) { return hipErrorInvalidValue; }

}  // namespace dfdx_rocm
