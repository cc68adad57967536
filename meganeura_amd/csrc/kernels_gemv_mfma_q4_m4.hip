// MFMA GEMV kernels for Q4 weights and 4 activation rows.
#include "kernels_gemv_mfma.hip.h"

namespace mgn {
int launch_gemv_mfma_q4_m4(ihipStream_t* s, const LaunchArgs& x) { return launch_t<MGN_FMT_Q4, 4>(s, x); }
}  // namespace mgn
