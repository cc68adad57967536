// The MFMA GEMV route: shape check and dispatch to the per-(format, rows) translation units.
// The kernel template lives in kernels_gemv_mfma.hip.h; each kernels_gemv_mfma_<fmt>_m<rows>.hip
// instantiates it for one weight format and one row count so that they compile in parallel.
#include "kernels_gemv_mfma.hip.h"

namespace mgn {

int launch_gemv_mfma_q4_m1(ihipStream_t* s, const LaunchArgs& x);
int launch_gemv_mfma_q4_m2(ihipStream_t* s, const LaunchArgs& x);
int launch_gemv_mfma_q4_m4(ihipStream_t* s, const LaunchArgs& x);
int launch_gemv_mfma_q8_m1(ihipStream_t* s, const LaunchArgs& x);
int launch_gemv_mfma_q8_m2(ihipStream_t* s, const LaunchArgs& x);
int launch_gemv_mfma_q8_m4(ihipStream_t* s, const LaunchArgs& x);

bool gemv_mfma_supported(const LaunchArgs& x) {
  if (x.m == 0 || x.m > 4) return false;
  if (x.a_is_f16 && x.pro_kind != kProNone) return false;  // fp16 activations: the plain matmul only
  MfmaGemvPlan p;
  for (int j = 0; j < x.n_more; j++)
    if (x.more[j].w.k != x.w.k || x.more[j].w.fmt != x.w.fmt) return false;
  if (x.n_more < 0 || x.n_more > kMaxBatch - 1) return false;
  return plan_mfma_gemv(x, x.m <= 2 ? x.m : 4, &p);
}

bool describe_gemv_mfma(const LaunchArgs& x, mgn_plan_info* out) {
  if (!gemv_mfma_supported(x)) return false;
  const uint32_t mrows = x.m <= 2 ? x.m : 4;
  MfmaGemvPlan p;
  if (!plan_mfma_gemv(x, mrows, &p)) return false;
  out->route = MGN_ROUTE_GEMV_MFMA;
  out->grid[0] = p.grid, out->grid[1] = p.kparts, out->grid[2] = 1;
  out->threads = 64 * p.ksc * p.wnc;
  out->lds_bytes = (uint32_t)p.lds;
  out->waves_n = p.wnc, out->k_splits = p.ksc, out->k_parts = p.kparts, out->steps = p.steps;
  out->quads_per_wave = p.qpw, out->full_steps = p.exact ? 1 : 0, out->tail_blocks = p.tail;
  out->workspace_bytes = (uint64_t)(p.kparts - 1) * mrows * x.w.n * sizeof(float);
  return true;
}

int launch_matmul_gemv_mfma(ihipStream_t* s, const LaunchArgs& x) {
  if (x.w.fmt == MGN_FMT_Q4)
    return x.m == 1 ? launch_gemv_mfma_q4_m1(s, x) : x.m == 2 ? launch_gemv_mfma_q4_m2(s, x) : launch_gemv_mfma_q4_m4(s, x);
  return x.m == 1 ? launch_gemv_mfma_q8_m1(s, x) : x.m == 2 ? launch_gemv_mfma_q8_m2(s, x) : launch_gemv_mfma_q8_m4(s, x);
}

}  // namespace mgn
