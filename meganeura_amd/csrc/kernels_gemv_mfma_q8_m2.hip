// MFMA GEMV kernels for Q8 weights and 2 activation rows.
#include "kernels_gemv_mfma.hip.h"

namespace mgn {
int launch_gemv_mfma_q8_m2(ihipStream_t* s, const LaunchArgs& x) { return launch_t<MGN_FMT_Q8, 2>(s, x); }
}  // namespace mgn
