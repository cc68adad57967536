// Placeholder until the tiled MFMA GEMM lands: no shape is claimed.
#include "kernels_common.hip.h"

namespace mgn {
bool gemm_mfma_supported(const LaunchArgs&) { return false; }
int launch_matmul_gemm_mfma(ihipStream_t*, const LaunchArgs&) { return (int)hipErrorNotSupported; }
}  // namespace mgn
