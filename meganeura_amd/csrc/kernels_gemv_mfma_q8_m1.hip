// MFMA GEMV kernels for Q8 weights and one activation row.
#include "kernels_gemv_mfma.hip.h"

namespace mgn {
int launch_gemv_mfma_q8_m1(ihipStream_t* s, const LaunchArgs& x) { return launch_t<MGN_FMT_Q8, 1>(s, x); }
}  // namespace mgn
