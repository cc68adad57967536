// Placeholder until the MFMA kernels land: no shape is claimed.
#include "kernels_common.hip.h"

namespace mgn {
bool mfma_supported(const LaunchArgs&) { return false; }
int launch_matmul_mfma(ihipStream_t*, const LaunchArgs&) { return (int)hipErrorNotSupported; }
}  // namespace mgn
