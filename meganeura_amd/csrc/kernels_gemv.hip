// Streaming dequant-GEMV for small M (decode): C[M,N] = A[M,K] x W (+ D), M <= 4.
//
// The reference has no quantized GEMV: at M = 1 its compiler emits
// ShaderEntry::MatMulGemv (src/compile.rs:1390-1406) but codegen falls back to
// the f32 GEMV shader for quantized weights (src/codegen.rs:1065-1074), which
// then reads packed bytes as floats.  This kernel computes what that route is
// meant to: per column sum_k a[k] * dequant(W)[k,n], the definition the
// reference's own test uses as ground truth (tests/gpu_smoke.rs:2726-2741),
// with the residual added once at the end as matmul_gemv_add.wgsl:49 does.
//
// Mapping (wave64).  A wave owns KBW consecutive blocks along K (one lane = one
// 32-element block, so one lane = one 128-bit load of nibbles plus one 32-bit
// load of scale|min) times NW = 64/KBW adjacent columns, and walks down the
// columns.  Because a lane's K position never changes, its 32 activations per
// row live in registers for the whole kernel; the inner loop touches no LDS.
// Consecutive lanes read consecutive blocks, so every wave load is one
// contiguous 1 KiB (nibbles) + 256 B (scale|min) run per column.
// Per block:  sum_i w_i x_i = d * sum_i nib_i x_i + m * sum_i x_i, with the
// second sum hoisted out of the loop.  Lane partials are added across the KBW
// lanes with DPP, across the K groups of a workgroup through LDS.
//
// HBM traffic per call is the packed weight once (20 B or 34 B per block) plus
// M*K*4 of activations per workgroup from L2, and M*N*4 of output.
#include "kernels_common.hip.h"

namespace mgn {
namespace {

template <int MR>
struct XRegs {
  float x[MR][32];  // Q4: odd elements pre-scaled by 1/16 (their nibble arrives as 16*nib)
  float sx[MR];     // plain sum of the 32 activations
};

// Activations reach the lanes through LDS: the workgroup copies the M rows of A
// with coalesced 128-bit loads into rows of 36 floats per 32-element block (the
// 4-float pad makes the per-lane 128-bit reads below conflict-free: lane l
// starts at dword 36*l, and 36*l mod 64 hits each multiple of 4 once per 16
// lanes), then every lane lifts its own block into registers.
constexpr int kXStride = 36;

template <int MR>
__device__ __forceinline__ void stage_x(float* __restrict__ xs, const float* __restrict__ a, uint32_t m,
                                        uint32_t k) {
  const uint32_t bpc = k / 32;
  for (uint32_t r = 0; r < (uint32_t)MR && r < m; r++) {
    const float4* src = (const float4*)(a + (size_t)r * k);
    float* dst = xs + (size_t)r * bpc * kXStride;
    for (uint32_t i = threadIdx.x; i < k / 4; i += blockDim.x)
      *(float4*)(dst + (i >> 3) * kXStride + (i & 7) * 4) = src[i];
  }
}

template <int FMT, int MR>
__device__ __forceinline__ void load_x(XRegs<MR>& xr, const float* __restrict__ xs, uint32_t m, uint32_t k,
                                       uint32_t kb, bool ok) {
  const uint32_t bpc = k / 32;
#pragma unroll
  for (int r = 0; r < MR; r++) {
    float s = 0.0f;
    if (ok && (uint32_t)r < m) {
      const float4* p = (const float4*)(xs + ((size_t)r * bpc + kb) * kXStride);
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const float4 v = p[j];
        xr.x[r][4 * j + 0] = v.x;
        xr.x[r][4 * j + 1] = v.y;
        xr.x[r][4 * j + 2] = v.z;
        xr.x[r][4 * j + 3] = v.w;
        s += (v.x + v.y) + (v.z + v.w);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 32; i++) xr.x[r][i] = 0.0f;
    }
    xr.sx[r] = s;
    if constexpr (FMT == MGN_FMT_Q4) {
#pragma unroll
      for (int i = 1; i < 32; i += 2) xr.x[r][i] *= 0.0625f;
    }
  }
}

// Raw block as loaded: Q4 = 4 words of nibbles + (d|m); Q8 = 8 words of int8 + scale.
template <int FMT>
struct RawBlock;
template <>
struct RawBlock<MGN_FMT_Q4> {
  uint4 q;
  uint32_t dm;
  __device__ __forceinline__ void load(const WeightView& w, size_t b) {
    q = stream_load_u128((const uint4*)w.quants + b);
    dm = stream_load_u32((const uint32_t*)w.meta + b);
  }
};
template <>
struct RawBlock<MGN_FMT_Q8> {
  uint4 q0, q1;
  uint16_t s;
  __device__ __forceinline__ void load(const WeightView& w, size_t b) {
    q0 = stream_load_u128((const uint4*)w.quants + b * 2);
    q1 = stream_load_u128((const uint4*)w.quants + b * 2 + 1);
    s = stream_load_u16((const uint16_t*)w.meta + b);
  }
};

template <int MR>
__device__ __forceinline__ void block_dot(const RawBlock<MGN_FMT_Q4>& blk, const XRegs<MR>& xr,
                                          float (&out)[MR]) {
  const uint32_t words[4] = {blk.q.x, blk.q.y, blk.q.z, blk.q.w};
  float acc0[MR], acc1[MR];
#pragma unroll
  for (int r = 0; r < MR; r++) acc0[r] = acc1[r] = 0.0f;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    // byte j of `lo` is element 8t+2j; byte j of `hi` is 16 * element 8t+2j+1
    const uint32_t lo = words[t] & 0x0F0F0F0Fu, hi = words[t] & 0xF0F0F0F0u;
    const float e[8] = {ubyte0(lo), ubyte0(hi), ubyte1(lo), ubyte1(hi),
                        ubyte2(lo), ubyte2(hi), ubyte3(lo), ubyte3(hi)};
#pragma unroll
    for (int r = 0; r < MR; r++) {
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        acc0[r] = __fmaf_rn(e[j], xr.x[r][8 * t + j], acc0[r]);
        acc1[r] = __fmaf_rn(e[j + 1], xr.x[r][8 * t + j + 1], acc1[r]);
      }
    }
  }
  const float d = half_bits_to_float(blk.dm & 0xFFFFu), m = half_bits_to_float(blk.dm >> 16);
#pragma unroll
  for (int r = 0; r < MR; r++) out[r] = __fmaf_rn(d, acc0[r] + acc1[r], m * xr.sx[r]);
}

template <int MR>
__device__ __forceinline__ void block_dot(const RawBlock<MGN_FMT_Q8>& blk, const XRegs<MR>& xr,
                                          float (&out)[MR]) {
  const uint32_t words[8] = {blk.q0.x, blk.q0.y, blk.q0.z, blk.q0.w, blk.q1.x, blk.q1.y, blk.q1.z, blk.q1.w};
  float acc0[MR], acc1[MR];
#pragma unroll
  for (int r = 0; r < MR; r++) acc0[r] = acc1[r] = 0.0f;
#pragma unroll
  for (int t = 0; t < 8; t++) {
    // flip the sign bits: bytes become q + 128 in 0..255, converted without sign handling
    const uint32_t u = words[t] ^ 0x80808080u;
    const float e[4] = {ubyte0(u), ubyte1(u), ubyte2(u), ubyte3(u)};
#pragma unroll
    for (int r = 0; r < MR; r++) {
      acc0[r] = __fmaf_rn(e[0], xr.x[r][4 * t + 0], acc0[r]);
      acc1[r] = __fmaf_rn(e[1], xr.x[r][4 * t + 1], acc1[r]);
      acc0[r] = __fmaf_rn(e[2], xr.x[r][4 * t + 2], acc0[r]);
      acc1[r] = __fmaf_rn(e[3], xr.x[r][4 * t + 3], acc1[r]);
    }
  }
  const float s = half_bits_to_float(blk.s);
#pragma unroll
  for (int r = 0; r < MR; r++) out[r] = s * __fmaf_rn(-128.0f, xr.sx[r], acc0[r] + acc1[r]);
}

// grid.x workgroups; blockDim.x = 64 * kgc * wnc.  Wave w: K group kg = w % kgc,
// column strip wn = w / kgc.  `steps` column steps per wave (a multiple of U).
template <int MR>
constexpr int max_waves() { return MR >= 4 ? 4 : 8; }

template <int FMT, int KBW, int MR, int U>
__global__ __launch_bounds__(64 * max_waves<MR>()) void gemv_kernel(WeightView w, const float* __restrict__ a, const float* __restrict__ d,
                            float* __restrict__ c, uint32_t m, uint32_t steps, uint32_t kgc, uint32_t epilogue) {
  extern __shared__ float lds[];
  const uint32_t x_floats = MR * (w.k / 32) * kXStride;
  float* xs = lds;               // [MR][bpc][36] staged activations
  float* red = lds + x_floats;   // [kgc][MR][cols_per_wg], used when kgc > 1
  constexpr int NW = 64 / KBW;
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t kg = wave % kgc, wn = wave / kgc, wnc = (blockDim.x >> 6) / kgc;
  const uint32_t cols_per_wave = steps * NW, cols_per_wg = cols_per_wave * wnc;
  const uint32_t kbl = lane % KBW, nsub = lane / KBW;
  const uint32_t bpc = w.k / 32;
  const uint32_t kb = kg * KBW + kbl;
  const bool kb_ok = kb < bpc;
  const uint32_t col0 = wn * cols_per_wave + nsub;            // column within the workgroup
  const uint32_t n0 = blockIdx.x * cols_per_wg + col0;        // global column of step 0

  RawBlock<FMT> blk[U];
  auto issue = [&](uint32_t step) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t n = n0 + (step + u) * NW;
      const bool ok = kb_ok && n < w.n;
      blk[u].load(w, ok ? (size_t)n * bpc + kb : 0);  // block 0 always exists
    }
  };
  issue(0);  // weights first: they are in flight while the activations are staged
  stage_x<MR>(xs, a, m, w.k);
  lds_barrier();
  XRegs<MR> xr;
  load_x<FMT, MR>(xr, xs, m, w.k, kb, kb_ok);

  for (uint32_t step = 0; step < steps; step += U) {
    RawBlock<FMT> cur[U];
#pragma unroll
    for (int u = 0; u < U; u++) cur[u] = blk[u];
    if (step + U < steps) issue(step + U);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t n = n0 + (step + u) * NW;
      float part[MR];
      block_dot<MR>(cur[u], xr, part);
#pragma unroll
      for (int r = 0; r < MR; r++) {
        float v = group_sum<KBW>((kb_ok && n < w.n) ? part[r] : 0.0f);
        if (kbl == 0) {
          if (kgc == 1) {
            if (n < w.n && (uint32_t)r < m) {
              const size_t idx = (size_t)r * w.n + n;
              c[idx] = apply_epilogue(d ? v + d[idx] : v, epilogue);
            }
          } else {
            red[(kg * MR + r) * cols_per_wg + col0 + (step + u) * NW] = v;
          }
        }
      }
    }
  }
  if (kgc > 1) {
    lds_barrier();
    for (uint32_t idx = threadIdx.x; idx < MR * cols_per_wg; idx += blockDim.x) {
      const uint32_t r = idx / cols_per_wg, col = idx % cols_per_wg;
      const uint32_t n = blockIdx.x * cols_per_wg + col;
      if (r < m && n < w.n) {
        float v = 0.0f;
        for (uint32_t g = 0; g < kgc; g++) v += red[(g * MR + r) * cols_per_wg + col];
        const size_t o = (size_t)r * w.n + n;
        c[o] = apply_epilogue(d ? v + d[o] : v, epilogue);
      }
    }
  }
}

struct GemvPlan {
  int kbw;
  uint32_t kgc, wnc, steps, grid;
};

constexpr int kUnroll = 4;

GemvPlan plan_gemv(uint32_t k, uint32_t n, int num_cus, uint32_t max_waves) {
  const uint32_t bpc = k / 32;
  GemvPlan p{};
  // widest K span per wave that keeps at least 3/4 of the lanes on real blocks
  int best = 8;
  double best_eff = 0.0;
  for (int kbw = 64; kbw >= 8; kbw /= 2) {
    const double eff = (double)bpc / (double)(((bpc + kbw - 1) / kbw) * kbw);
    if (eff >= 0.75) {
      best = kbw;
      break;
    }
    if (eff > best_eff) {
      best_eff = eff;
      best = kbw;
    }
  }
  p.kbw = best;
  p.kgc = (bpc + best - 1) / best;
  p.wnc = p.kgc >= max_waves ? 1 : max_waves / p.kgc;
  const uint32_t nw = 64 / best;
  const uint32_t col_steps = (n + nw - 1) / nw;
  // aim at ~16 waves per CU so that the whole weight is in flight early
  uint32_t n_waves = std::max<uint32_t>(1, (uint32_t)num_cus * 16 / p.kgc);
  uint32_t steps = (col_steps + n_waves - 1) / n_waves;
  steps = std::max<uint32_t>(kUnroll, (steps + kUnroll - 1) / kUnroll * kUnroll);
  p.steps = steps;
  const uint32_t cols_per_wg = steps * nw * p.wnc;
  p.grid = (n + cols_per_wg - 1) / cols_per_wg;
  return p;
}

template <int FMT, int MR>
int launch_gemv_t(ihipStream_t* s, const LaunchArgs& x) {
  const GemvPlan p = plan_gemv(x.w.k, x.w.n, x.num_cus, max_waves<MR>());
  const dim3 grid(p.grid), block(64 * p.kgc * p.wnc);
  const uint32_t nw = 64 / p.kbw;
  const size_t lds = ((size_t)MR * (x.w.k / 32) * kXStride +
                      (p.kgc > 1 ? (size_t)p.kgc * MR * p.steps * nw * p.wnc : 0)) * sizeof(float);
  // more than 64 KiB of dynamic LDS has to be allowed per kernel and device, once
#define MGN_GEMV(KBW)                                                                                   \
  do {                                                                                                  \
    auto kern = gemv_kernel<FMT, KBW, MR, kUnroll>;                                                     \
    static std::atomic<uint64_t> big_lds_done{0};                                                       \
    if (lds > 64 * 1024)                                                                                \
      if (int e = enable_big_lds(kern, x.device, big_lds_done)) return e;                               \
    hipLaunchKernelGGL(kern, grid, block, lds, s, x.w, (const float*)x.a, x.d, x.c, x.m, p.steps, p.kgc, x.epilogue); \
  } while (0)
  switch (p.kbw) {
    case 64: MGN_GEMV(64); break;
    case 32: MGN_GEMV(32); break;
    case 16: MGN_GEMV(16); break;
    default: MGN_GEMV(8); break;
  }
#undef MGN_GEMV
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace

bool gemv_supported(const LaunchArgs& x) {
  if (x.a_is_f16 || x.m == 0 || x.m > 4) return false;
  const uint32_t mw = x.m > 2 ? max_waves<4>() : max_waves<1>();
  const GemvPlan p = plan_gemv(x.w.k, x.w.n, x.num_cus, mw);
  const size_t x_bytes = (size_t)(x.m > 2 ? 4 : x.m) * (x.w.k / 32) * kXStride * sizeof(float);
  // all K groups of a column must fit in one workgroup, the staged activations in LDS
  return p.kgc <= mw && x_bytes <= 128 * 1024;
}

int launch_matmul_gemv(ihipStream_t* s, const LaunchArgs& x) {
  const int mr = x.m == 1 ? 1 : (x.m == 2 ? 2 : 4);
  if (x.w.fmt == MGN_FMT_Q4) {
    if (mr == 1) return launch_gemv_t<MGN_FMT_Q4, 1>(s, x);
    if (mr == 2) return launch_gemv_t<MGN_FMT_Q4, 2>(s, x);
    return launch_gemv_t<MGN_FMT_Q4, 4>(s, x);
  }
  if (mr == 1) return launch_gemv_t<MGN_FMT_Q8, 1>(s, x);
  if (mr == 2) return launch_gemv_t<MGN_FMT_Q8, 2>(s, x);
  return launch_gemv_t<MGN_FMT_Q8, 4>(s, x);
}

}  // namespace mgn
