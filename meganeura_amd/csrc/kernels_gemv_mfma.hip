// Dequant-GEMV on the matrix cores for M <= 2 (decode): C[M,N] = A[M,K] x W (+ D).
//
// Why MFMA for a matrix-vector product: streaming a 4-bit weight at HBM speed
// leaves about one vector instruction per four weights per lane; converting
// every nibble to f32 and multiplying it on the vector ALU costs three times
// that and makes the kernel ALU-bound.  Here the vector ALU only masks nibbles
// into place (5 instructions per 8 weights); the multiply-adds run on
// v_mfma_f32_4x4x4_16B_f16, whose 16 independent 4x4 blocks fit the problem:
//   lane (b, i), b = lane/4, i = lane%4, supplies "row i" of block b's A:
//     four weights of quant block (column 4q+i, K block kb0+b);
//   lane (b, j) supplies "column j" of block b's B: four activations of K block
//     kb0+b, j = 2*row for the high half of an fp16 split, 2*row+1 for the low;
//   lane (b, j) receives D[i][j], i = 0..3: the four columns' partial sums.
// Eight such MFMAs cover one 32-element quant block per lane.
//
// Exactness.  A nibble n masked to bits 0-3 (or 4-7) of an fp16 is the
// subnormal n * 2^-24 (n * 2^-20): exact, and the matrix cores do not flush
// fp16 subnormals.  Activations are split x = hi + lo into two fp16 after
// scaling the row by a power of two (|x| < 2^12), so products are exact in f32
// and only the f32 accumulation rounds: the result carries ~21 bits of x, not
// 11.  Per block the identity used is
//   sum_k (n_k d + m) x_k = d * (sum_k n_k x_k - 8 sum_k x_k) + (m + 8 d) * sum_k x_k :
// the nibbles are centred (n - 8) so that neither term is large against the
// result, and the "- 8 sum x" enters as the MFMA chain's initial accumulator,
// i.e. before anything is scaled or summed across blocks; accumulating
// d * sum(n x) and m * sum(x) separately down a column would cancel
// catastrophically.  Q8 bytes are biased to unsigned (q + 128) and the bias
// leaves the same way (- 128 sum x as the initial accumulator).
//
// A wave owns four adjacent columns and walks K sixteen blocks at a time, so
// its four accumulators stay in registers down the whole column; cross-lane
// sums happen once per column quad.  The activations' B operands are prepared
// once per workgroup in LDS, laid out so that consecutive lanes read
// consecutive 16-byte chunks.
#include "kernels_common.hip.h"

namespace mgn {
namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr float kTwoPow24 = 16777216.0f;
constexpr int kMaxTasks = 2;  // activation chunks a thread prepares, per row

__device__ __forceinline__ uint32_t pack_half2(float lo, float hi) {
  const uint32_t a = __builtin_bit_cast(uint16_t, (_Float16)lo);
  const uint32_t b = __builtin_bit_cast(uint16_t, (_Float16)hi);
  return a | (b << 16);
}

__device__ __forceinline__ float half_residual(float v) { return v - (float)(_Float16)v; }

__device__ __forceinline__ half4 as_half4(uint32_t lo, uint32_t hi) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  const u32x2 v = {lo, hi};
  return __builtin_bit_cast(half4, v);
}

constexpr int kQuadBcast[4] = {0x00, 0x55, 0xAA, 0xFF};  // quad_perm:[i,i,i,i]
constexpr int kRowRor4 = 0x124, kRowRor8 = 0x128;        // rotate right within a row of 16

// sum over the 16 lanes sharing lane%4 (every such lane ends with the total)
__device__ __forceinline__ float sum_over_blocks(float v) {
  v += dpp_move<kRowRor4>(v);
  v += dpp_move<kRowRor8>(v);
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

template <int FMT>
struct Raw;
template <>
struct Raw<MGN_FMT_Q4> {
  uint4 q;
  uint32_t meta;
  __device__ __forceinline__ void load(const WeightView& w, size_t b) {
    q = stream_load_u128((const uint4*)w.quants + b);
    meta = stream_load_u32((const uint32_t*)w.meta + b);
  }
};
template <>
struct Raw<MGN_FMT_Q8> {
  uint4 q0, q1;
  uint32_t meta;
  __device__ __forceinline__ void load(const WeightView& w, size_t b) {
    q0 = stream_load_u128((const uint4*)w.quants + b * 2);
    q1 = stream_load_u128((const uint4*)w.quants + b * 2 + 1);
    meta = stream_load_u16((const uint16_t*)w.meta + b);
  }
};

// LDS image of the activations, per workgroup:
//   chunk planes  xb[c][kb * NJ + j]  (uint4), c = 0..3: the B operands of the two MFMAs
//                 that consume elements 8c..8c+7 of K block kb, B column j;
//   sx24[r][kb]   2^-24 * sum of the (scaled) activations of K block kb, row r.
// Q4 pairs nibble k with k+4 in one fp16x2 mask, and odd nibbles sit 4 bits higher
// (2^-20 instead of 2^-24), so the chunk is (x0,x4,x2,x6 | x1,x5,x3,x7 / 16).
// Q8 bytes come out in natural order: (x0,x1,x2,x3 | x4,x5,x6,x7).
// *s_hi / *s_lo get sum_k of the value nibble/byte k is multiplied with in the hi / lo
// column (for Q4's odd elements that is 16 * fp16(x/16)), in f32.
template <int FMT>
__device__ __forceinline__ void make_chunks(const float (&x)[8], uint4& hi, uint4& lo, float* s_hi, float* s_lo) {
  float p[8];
  if constexpr (FMT == MGN_FMT_Q4) {
    const float o = 0.0625f;
    p[0] = x[0], p[1] = x[4], p[2] = x[2], p[3] = x[6];
    p[4] = x[1] * o, p[5] = x[5] * o, p[6] = x[3] * o, p[7] = x[7] * o;
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) p[i] = x[i];
  }
  hi = make_uint4(pack_half2(p[0], p[1]), pack_half2(p[2], p[3]), pack_half2(p[4], p[5]), pack_half2(p[6], p[7]));
  float r[8];
#pragma unroll
  for (int i = 0; i < 8; i++) r[i] = half_residual(p[i]);
  lo = make_uint4(pack_half2(r[0], r[1]), pack_half2(r[2], r[3]), pack_half2(r[4], r[5]), pack_half2(r[6], r[7]));
  float h[8], l[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    h[i] = (float)(_Float16)p[i];
    l[i] = (float)(_Float16)r[i];
  }
  const float sc = FMT == MGN_FMT_Q4 ? 16.0f : 1.0f;  // second half of a Q4 chunk is x/16
  *s_hi = ((h[0] + h[1]) + (h[2] + h[3])) + sc * ((h[4] + h[5]) + (h[6] + h[7]));
  *s_lo = ((l[0] + l[1]) + (l[2] + l[3])) + sc * ((l[4] + l[5]) + (l[6] + l[7]));
}

// Power of two that brings the row's largest magnitude below 2^12 (1 if the row
// is all zero or not finite).  Returns the scale; *inv gets its reciprocal.
__device__ __forceinline__ float row_scale(float amax, float* inv) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, amax);
  const int e = (int)(bits >> 23) - 127;  // floor(log2(amax)) for normal values
  if (bits == 0 || e >= 128 || e <= -100) {
    *inv = 1.0f;
    return 1.0f;
  }
  const int sh = 11 - e;  // amax * 2^sh in [2^11, 2^12)
  *inv = __builtin_bit_cast(float, (uint32_t)(127 - sh) << 23);
  return __builtin_bit_cast(float, (uint32_t)(127 + sh) << 23);
}

// blockDim.x = 64 * ksc * wnc.  Wave w: K split ks = w % ksc, quad lane wn = w / ksc.
// The workgroup owns quads [blockIdx.x * qpw, +qpw); wave (ks, wn) takes quads wn, wn+wnc, ...
// and K blocks [ks * spk * 16, (ks+1) * spk * 16).
template <int FMT, int MROWS, int U>
__global__ __launch_bounds__(1024) void gemv_mfma_kernel(WeightView w, const float* __restrict__ a,
                                                         const float* __restrict__ dres, float* __restrict__ c,
                                                         uint32_t m, uint32_t qpw, uint32_t ksc, uint32_t spk) {
  constexpr int NJ = 2 * MROWS;
  extern __shared__ uint4 lds4[];
  const uint32_t bpc = w.k / 32;
  const uint32_t bpc_pad = (bpc + 15) & ~15u;
  const uint32_t plane = bpc_pad * NJ;
  uint4* xb = lds4;                                  // [4][plane]
  float* sx24 = (float*)(lds4 + 4 * plane);          // [MROWS][bpc_pad]
  float* cinit = sx24 + MROWS * bpc_pad;             // [bpc_pad][NJ]: -bias * 2^-24 * sum of column j's operands
  float* red = cinit + plane;                        // [qpw][ksc][MROWS][4]
  float* scratch = red + qpw * ksc * MROWS * 4;      // [16 waves][MROWS] row maxima, then [MROWS] scales

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  // everything derived from the wave index is wave-uniform: keep it in scalar registers
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t nwaves = blockDim.x >> 6;
  const uint32_t ks = wave % ksc, wn = wave / ksc, wnc = nwaves / ksc;
  const uint32_t b = lane >> 2, i = lane & 3;        // MFMA block, row (A) / column (B) within it
  const uint32_t quad0 = blockIdx.x * qpw;
  const uint32_t nquads = (w.n + 3) / 4;

  // This wave's work, linearised: quads first, first + wnc, ... below q_end, each walked
  // in my_steps steps of 16 K blocks.  A producer cursor (pq, pst) runs U steps ahead of
  // the consumer cursor (cq, cst) and keeps a ring of U raw blocks in flight per lane.
  const uint32_t steps_total = bpc_pad / 16;
  const uint32_t step_begin = ks * spk;
  const uint32_t my_steps = step_begin >= steps_total ? 0u : min(spk, steps_total - step_begin);
  const uint32_t first = quad0 + wn;
  const uint32_t q_end = my_steps == 0 ? 0u : min(quad0 + qpw, nquads);
  const uint32_t kb_first = step_begin * 16 + b;      // this lane's K block at step 0
  const uint32_t zero_block = bpc * w.n;              // an all-zero block behind the last real one
  Raw<FMT> ring[U];
  uint32_t pq = first, pst = 0;
  uint32_t pblk = 0;  // block index the producer loads next (valid while pn_ok)
  bool pn_ok = false;
  auto produce = [&](int u) {
    if (pq < q_end) {  // wave-uniform
      if (pst == 0) {
        const uint32_t n = pq * 4 + i;
        pn_ok = n < w.n;
        pblk = n * bpc + kb_first;
      }
      const bool ok = pn_ok && kb_first + pst * 16 < bpc;
      ring[u].load(w, ok ? pblk : zero_block);
      pblk += 16;
      if (++pst == my_steps) {
        pst = 0;
        pq += wnc;
      }
    }
  };
  // Memory returns a wave's loads in issue order, so the (small, cache-resident)
  // activation loads go first and the weight ring right behind them: the activation
  // prep below then waits for its own data only, while the weights stream in.
  // One task = 8 consecutive activations of one row = one B chunk; the 4 tasks of a K
  // block sit in one lane quad.  A thread holds at most kMaxTasks tasks in registers.
  float4 xraw[kMaxTasks][MROWS][2];
#pragma unroll
  for (int tt = 0; tt < kMaxTasks; tt++) {
    const uint32_t t = tid + tt * blockDim.x, kb = t >> 2, ch = t & 3;
#pragma unroll
    for (int r = 0; r < MROWS; r++) {
      if (kb < bpc && (uint32_t)r < m) {
        const float4* src = (const float4*)(a + (size_t)r * w.k + (size_t)kb * 32 + ch * 8);
        xraw[tt][r][0] = src[0];
        xraw[tt][r][1] = src[1];
      } else {
        xraw[tt][r][0] = xraw[tt][r][1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < U; u++) produce(u);
  for (uint32_t t = tid; t < qpw * ksc * MROWS * 4; t += blockDim.x) red[t] = 0.0f;

  // ---- activations -> LDS (once per workgroup) ----
  float inv_scale[MROWS];
  {
    float scale[MROWS];
#pragma unroll
    for (int r = 0; r < MROWS; r++) {
      float am = 0.0f;
#pragma unroll
      for (int tt = 0; tt < kMaxTasks; tt++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const float4 v = xraw[tt][r][h];
          am = fmaxf(am, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
      // NaN never wins fmaxf; infinities do and switch scaling off in row_scale
      am = fmaxf(am, dpp_move<kDppQuadXor1>(am));
      am = fmaxf(am, dpp_move<kDppQuadXor2>(am));
      am = fmaxf(am, dpp_move<kDppRowHalfMirror>(am));
      am = fmaxf(am, dpp_move<kDppRowMirror>(am));
      am = fmaxf(am, __shfl_xor(am, 16, 64));
      am = fmaxf(am, __shfl_xor(am, 32, 64));
      if (lane == 0) scratch[(tid >> 6) * MROWS + r] = am;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < MROWS; r++) {
      float v = 0.0f;
      for (uint32_t wv = 0; wv < nwaves; wv++) v = fmaxf(v, scratch[wv * MROWS + r]);
      scale[r] = row_scale(v, &inv_scale[r]);
    }
#pragma unroll
    for (int tt = 0; tt < kMaxTasks; tt++) {
      const uint32_t t = tid + tt * blockDim.x, kb = t >> 2, ch = t & 3;
      if (t < bpc_pad * 4) {  // whole waves take this branch together (bpc_pad * 4 is a multiple of 64)
#pragma unroll
        for (int r = 0; r < MROWS; r++) {
          const float4 v0 = xraw[tt][r][0], v1 = xraw[tt][r][1];
          const float x[8] = {v0.x * scale[r], v0.y * scale[r], v0.z * scale[r], v0.w * scale[r],
                              v1.x * scale[r], v1.y * scale[r], v1.z * scale[r], v1.w * scale[r]};
          uint4 hi, lo;
          float s_hi, s_lo;
          make_chunks<FMT>(x, hi, lo, &s_hi, &s_lo);
          xb[ch * plane + kb * NJ + 2 * r] = hi;
          xb[ch * plane + kb * NJ + 2 * r + 1] = lo;
          s_hi += dpp_move<kDppQuadXor1>(s_hi);
          s_hi += dpp_move<kDppQuadXor2>(s_hi);
          s_lo += dpp_move<kDppQuadXor1>(s_lo);
          s_lo += dpp_move<kDppQuadXor2>(s_lo);
          if (ch == 0) {
            constexpr float bias = FMT == MGN_FMT_Q4 ? 8.0f : 128.0f;
            // the m-term uses the same split values the MFMAs see, so the result is the
            // exact dot product with hi + lo up to f32 rounding
            sx24[r * bpc_pad + kb] = (s_hi + s_lo) * (1.0f / kTwoPow24);
            cinit[kb * NJ + 2 * r] = s_hi * (-bias / kTwoPow24);
            cinit[kb * NJ + 2 * r + 1] = s_lo * (-bias / kTwoPow24);
          }
        }
      }
    }
  }
  __syncthreads();

  // ---- main loop ----
  // Lanes i >= NJ have no B column of their own; they re-read column i % NJ (a broadcast in
  // LDS) and their sums are never looked at.  Byte offsets into the chunk planes / sx24:
  const uint32_t x_lane = ((kb_first * NJ) + (i % NJ)) * 16;
  const uint32_t sx_lane = kb_first * 4;
  const uint32_t ci_lane = (kb_first * NJ + (i % NJ)) * 4;
  const char* xb_bytes = (const char*)xb;
  const char* sx_bytes = (const char*)sx24;
  const char* ci_bytes = (const char*)cinit;
  floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};  // lane (b, j): sum over K of d * D[i][j], i = 0..3
  float macc[MROWS];                       // lane (b, i): sum over K of m * sum(x) for column 4q+i
#pragma unroll
  for (int r = 0; r < MROWS; r++) macc[r] = 0.0f;
  uint32_t cq = first, cst = 0;
  while (cq < q_end) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (cq < q_end) {  // wave-uniform
        const Raw<FMT> cur = ring[u];
        produce(u);
        // B operands: 4 chunks of 16 bytes, consecutive lanes -> consecutive chunks
        const uint32_t x_off = x_lane + cst * (16 * NJ * 16);
        uint4 bx[4];
#pragma unroll
        for (int ch = 0; ch < 4; ch++) bx[ch] = *(const uint4*)(xb_bytes + x_off + ch * plane * 16);
        float sxv[MROWS];
#pragma unroll
        for (int r = 0; r < MROWS; r++) sxv[r] = *(const float*)(sx_bytes + sx_lane + cst * 64 + r * bpc_pad * 4);
        const float ci = *(const float*)(ci_bytes + ci_lane + cst * (16 * NJ * 4));
        floatx4 dsum = {ci, ci, ci, ci};  // the centring term rides in as the chain's start value
        float dscale, mterm;
        if constexpr (FMT == MGN_FMT_Q4) {
          const uint32_t words[4] = {cur.q.x, cur.q.y, cur.q.z, cur.q.w};
#pragma unroll
          for (int ch = 0; ch < 4; ch++) {
            const uint32_t wd = words[ch], w8 = wd >> 8;
            const uint32_t e0 = wd & 0x000F000Fu, o0 = wd & 0x00F000F0u;  // (n0,n4) 2^-24, (n1,n5) 2^-20
            const uint32_t e1 = w8 & 0x000F000Fu, o1 = w8 & 0x00F000F0u;  // (n2,n6),       (n3,n7)
            dsum = __builtin_amdgcn_mfma_f32_4x4x4f16(as_half4(e0, e1), as_half4(bx[ch].x, bx[ch].y), dsum, 0, 0, 0);
            dsum = __builtin_amdgcn_mfma_f32_4x4x4f16(as_half4(o0, o1), as_half4(bx[ch].z, bx[ch].w), dsum, 0, 0, 0);
          }
          dscale = half_bits_to_float(cur.meta & 0xFFFFu);
          mterm = __fmaf_rn(8.0f, dscale, half_bits_to_float(cur.meta >> 16));  // m + 8 d
        } else {
          const uint32_t words[8] = {cur.q0.x, cur.q0.y, cur.q0.z, cur.q0.w, cur.q1.x, cur.q1.y, cur.q1.z, cur.q1.w};
#pragma unroll
          for (int ch = 0; ch < 4; ch++) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
              const uint32_t u8 = words[2 * ch + h] ^ 0x80808080u;  // q + 128 in every byte
              const uint32_t lo2 = __builtin_amdgcn_perm(0u, u8, 0x0c010c00u);  // (b0, b1) as fp16 mantissas
              const uint32_t hi2 = __builtin_amdgcn_perm(0u, u8, 0x0c030c02u);  // (b2, b3)
              const half4 bop = h == 0 ? as_half4(bx[ch].x, bx[ch].y) : as_half4(bx[ch].z, bx[ch].w);
              dsum = __builtin_amdgcn_mfma_f32_4x4x4f16(as_half4(lo2, hi2), bop, dsum, 0, 0, 0);
            }
          }
          dscale = half_bits_to_float(cur.meta & 0xFFFFu);
          mterm = 0.0f;  // symmetric format: nothing besides the centred sum
        }
        // acc[i] += d(column i of this block) * D[i]: d sits in lane (b, i), a quad broadcast away
        acc[0] = __fmaf_rn(dpp_move<kQuadBcast[0]>(dscale), dsum[0], acc[0]);
        acc[1] = __fmaf_rn(dpp_move<kQuadBcast[1]>(dscale), dsum[1], acc[1]);
        acc[2] = __fmaf_rn(dpp_move<kQuadBcast[2]>(dscale), dsum[2], acc[2]);
        acc[3] = __fmaf_rn(dpp_move<kQuadBcast[3]>(dscale), dsum[3], acc[3]);
#pragma unroll
        for (int r = 0; r < MROWS; r++)
          if constexpr (FMT == MGN_FMT_Q4) macc[r] = __fmaf_rn(mterm, sxv[r], macc[r]);

        if (cst + 1 == my_steps) {
          // ---- end of a column quad: the one cross-lane reduction ----
          // acc[col] in lane (b, j): add the hi/lo pair (j ^ 1), then all 16 blocks b
          float tot[4];
#pragma unroll
          for (int col = 0; col < 4; col++) {
            float v = acc[col];
            v += dpp_move<kDppQuadXor1>(v);
            tot[col] = sum_over_blocks(v);  // lanes j = 2r, 2r+1: row r's sum for column `col`
            acc[col] = 0.0f;
          }
#pragma unroll
          for (int r = 0; r < MROWS; r++) {
            const float mt = sum_over_blocks(macc[r]);  // lane (., i): column i's m-term, row r
            macc[r] = 0.0f;
            const float m0 = dpp_move<kQuadBcast[0]>(mt), m1 = dpp_move<kQuadBcast[1]>(mt);
            const float m2 = dpp_move<kQuadBcast[2]>(mt), m3 = dpp_move<kQuadBcast[3]>(mt);
            if (lane == (uint32_t)(2 * r)) {
              const float os = kTwoPow24 * inv_scale[r];
              float* dst = red + (((cq - quad0) * ksc + ks) * MROWS + r) * 4;
              dst[0] = (tot[0] + m0) * os;
              dst[1] = (tot[1] + m1) * os;
              dst[2] = (tot[2] + m2) * os;
              dst[3] = (tot[3] + m3) * os;
            }
          }
        }
        if (++cst == my_steps) {
          cst = 0;
          cq += wnc;
        }
      }
    }
  }
  __syncthreads();
  // ---- combine the K splits, add the residual, store ----
  for (uint32_t t = tid; t < qpw * MROWS * 4; t += blockDim.x) {
    const uint32_t col = t & 3, r = (t >> 2) % MROWS, ql = t / (4 * MROWS);
    const uint32_t n = (quad0 + ql) * 4 + col;
    if (r < m && n < w.n) {
      float v = 0.0f;
      for (uint32_t s = 0; s < ksc; s++) v += red[((ql * ksc + s) * MROWS + r) * 4 + col];
      const size_t o = (size_t)r * w.n + n;
      c[o] = dres ? v + dres[o] : v;
    }
  }
}

struct MfmaGemvPlan {
  uint32_t ksc, wnc, qpw, spk, grid;
  size_t lds;
};

// raw blocks in flight per lane: 8 x 20 B for Q4, 6 x 34 B for Q8
template <int FMT>
constexpr int ring_depth() { return FMT == MGN_FMT_Q4 ? 8 : 6; }

bool plan_mfma_gemv(uint32_t k, uint32_t n, uint32_t mrows, int num_cus, MfmaGemvPlan* out) {
  const uint32_t bpc = k / 32, bpc_pad = (bpc + 15) & ~15u;
  const uint32_t steps_total = bpc_pad / 16;
  const uint32_t nquads = (n + 3) / 4;
  MfmaGemvPlan p{};
  // quads per workgroup: spread the quads evenly over the CUs (one workgroup per CU when
  // there is enough work), so the activations are prepared as few times as possible
  p.qpw = std::max<uint32_t>(1, (nquads + num_cus - 1) / num_cus);
  // K splits: keep at least ~12 waves per workgroup busy when a workgroup has few quads,
  // but leave every wave a few steps of its own
  uint32_t ksc = 1;
  while (p.qpw * ksc < 12 && ksc * 2 <= 16 && steps_total / (ksc * 2) >= 2) ksc *= 2;
  p.ksc = ksc;
  p.spk = (steps_total + ksc - 1) / ksc;
  p.wnc = std::max<uint32_t>(1, std::min<uint32_t>(p.qpw, 16 / ksc));
  // enough threads to prepare the activations (waves beyond the quads only help there)
  const uint32_t prep_waves = (bpc_pad * 4 + kMaxTasks * 64 - 1) / (kMaxTasks * 64);
  p.wnc = std::min<uint32_t>(16 / ksc, std::max<uint32_t>(p.wnc, (prep_waves + ksc - 1) / ksc));
  p.grid = (nquads + p.qpw - 1) / p.qpw;
  const size_t nj = 2 * mrows;
  p.lds = (size_t)4 * bpc_pad * nj * 16 + (size_t)mrows * bpc_pad * 4 + (size_t)bpc_pad * nj * 4 +
          (size_t)p.qpw * ksc * mrows * 16 + (size_t)16 * mrows * 4 + 64;
  if (p.lds > 150 * 1024) return false;
  // every thread prepares at most kMaxTasks activation chunks per row
  if ((size_t)bpc_pad * 4 > (size_t)kMaxTasks * 64 * p.ksc * p.wnc) return false;
  *out = p;
  return true;
}

template <int FMT, int MROWS>
int launch_t(ihipStream_t* s, const LaunchArgs& x) {
  MfmaGemvPlan p;
  if (!plan_mfma_gemv(x.w.k, x.w.n, MROWS, x.num_cus, &p)) return (int)hipErrorInvalidValue;
  auto kern = gemv_mfma_kernel<FMT, MROWS, ring_depth<FMT>()>;
  static bool big_lds_enabled = false;
  if (p.lds > 64 * 1024 && !big_lds_enabled) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return (int)e;
    big_lds_enabled = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.grid), dim3(64 * p.ksc * p.wnc), p.lds, s, x.w, (const float*)x.a, x.d, x.c, x.m,
                     p.qpw, p.ksc, p.spk);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace

bool gemv_mfma_supported(const LaunchArgs& x) {
  if (x.a_is_f16 || x.m == 0 || x.m > 2) return false;
  MfmaGemvPlan p;
  return plan_mfma_gemv(x.w.k, x.w.n, x.m, x.num_cus, &p);
}

int launch_matmul_gemv_mfma(ihipStream_t* s, const LaunchArgs& x) {
  if (x.w.fmt == MGN_FMT_Q4) return x.m == 1 ? launch_t<MGN_FMT_Q4, 1>(s, x) : launch_t<MGN_FMT_Q4, 2>(s, x);
  return x.m == 1 ? launch_t<MGN_FMT_Q8, 1>(s, x) : launch_t<MGN_FMT_Q8, 2>(s, x);
}

}  // namespace mgn
