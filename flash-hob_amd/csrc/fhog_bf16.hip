// bf16 MFMA kernels (placeholder while the fast path is being brought up).
#include "fhog_common.h"
namespace fhog {
bool bf16_shape_supported(int64_t, int64_t, int64_t, int) { return false; }
hipError_t launch_bf16_pass(const Params&, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace fhog
