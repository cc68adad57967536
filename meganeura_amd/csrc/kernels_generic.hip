// Scalar fallback: C[M,N] = A[M,K] x dequant(W) (+ D), any M, any N, K % 32 == 0.
//
// Same arithmetic as the reference's tiled shader with dequant on B-load
// (src/shaders/matmul.wgsl, src/codegen.rs:748-805): every weight is
// dequantized to its exact f32 value and multiplied in f32.  It exists so that
// every shape has a correct route and so the fast kernels have a second GPU
// implementation to be compared with; it is not tuned.
//
// Work split: a workgroup owns 64 output columns x TM rows.  Lane = column,
// the 4 waves split K by block (kb = wave, wave+4, ...), partial sums meet in
// LDS.  A is read straight from global memory: all lanes of a wave read the
// same address, which the cache broadcasts.
#include "kernels_common.hip.h"

namespace mgn {
namespace {

constexpr int TM = 8;

template <int FMT>
__device__ __forceinline__ void load_block(const WeightView& w, size_t b, float (&wv)[32]) {
  if constexpr (FMT == MGN_FMT_Q4) {
    const uint32_t dm = ((const uint32_t*)w.meta)[b];
    const float d = half_bits_to_float(dm & 0xFFFFu), m = half_bits_to_float(dm >> 16);
    const uint4 q = ((const uint4*)w.quants)[b];
    const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int j = 0; j < 8; j++) wv[t * 8 + j] = __fmaf_rn((float)((words[t] >> (4 * j)) & 0xFu), d, m);
  } else {
    const float s = half_bits_to_float(((const uint16_t*)w.meta)[b]);
    const uint4* qp = (const uint4*)w.quants + b * 2;
    const uint4 q0 = qp[0], q1 = qp[1];
    const uint32_t words[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
      for (int j = 0; j < 4; j++) wv[t * 4 + j] = (float)(int8_t)(words[t] >> (8 * j)) * s;
  }
}

template <int FMT, typename AT>
__global__ __launch_bounds__(256) void generic_kernel(WeightView w, const AT* __restrict__ a,
                                                      const float* __restrict__ d, float* __restrict__ c,
                                                      uint32_t m, uint32_t epilogue) {
  __shared__ float red[4][TM][64];
  const uint32_t lane = threadIdx.x & 63, ks = threadIdx.x >> 6;
  const uint32_t n = blockIdx.x * 64 + lane;
  const uint32_t m0 = blockIdx.y * TM;
  const uint32_t bpc = w.k / 32;
  float acc[TM];
#pragma unroll
  for (int r = 0; r < TM; r++) acc[r] = 0.0f;
  if (n < w.n) {
    for (uint32_t kb = ks; kb < bpc; kb += 4) {
      float wv[32];
      load_block<FMT>(w, (size_t)n * bpc + kb, wv);
#pragma unroll
      for (int r = 0; r < TM; r++) {
        if (m0 + r < m) {
          const AT* ar = a + (size_t)(m0 + r) * w.k + kb * 32;
#pragma unroll
          for (int i = 0; i < 32; i++) acc[r] = __fmaf_rn((float)ar[i], wv[i], acc[r]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < TM; r++) red[ks][r][lane] = acc[r];
  __syncthreads();
  if (ks == 0 && n < w.n) {
#pragma unroll
    for (int r = 0; r < TM; r++) {
      if (m0 + r < m) {
        float v = (red[0][r][lane] + red[1][r][lane]) + (red[2][r][lane] + red[3][r][lane]);
        const size_t idx = (size_t)(m0 + r) * w.n + n;
        if (d) v += d[idx];
        c[idx] = apply_epilogue(v, epilogue);
      }
    }
  }
}

}  // namespace

int launch_matmul_generic(ihipStream_t* s, const LaunchArgs& x) {
  dim3 grid((x.w.n + 63) / 64, (x.m + TM - 1) / TM);
  dim3 block(256);
#define MGN_GENERIC(FMT, AT) \
  hipLaunchKernelGGL((generic_kernel<FMT, AT>), grid, block, 0, s, x.w, (const AT*)x.a, x.d, x.c, x.m, x.epilogue)
  if (x.w.fmt == MGN_FMT_Q4) {
    if (x.a_is_f16) MGN_GENERIC(MGN_FMT_Q4, _Float16); else MGN_GENERIC(MGN_FMT_Q4, float);
  } else {
    if (x.a_is_f16) MGN_GENERIC(MGN_FMT_Q8, _Float16); else MGN_GENERIC(MGN_FMT_Q8, float);
  }
#undef MGN_GENERIC
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace mgn
