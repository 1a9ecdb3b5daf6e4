#include "internal.h"
namespace ztvm {
bool skinny_supports(const MatmulArgs&) { return false; }
hipError_t launch_skinny(const MatmulArgs&, const Tune&, hipStream_t) { return hipErrorNotSupported; }
}  // namespace ztvm
