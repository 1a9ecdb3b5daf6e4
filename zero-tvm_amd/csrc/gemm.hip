#include "internal.h"
namespace ztvm {
bool gemm_supports(const MatmulArgs&) { return false; }
hipError_t launch_gemm(const MatmulArgs&, const Tune&, hipStream_t) { return hipErrorNotSupported; }
}  // namespace ztvm
