// Dequant-GEMV on the matrix cores for M <= 4 (decode): C[M,N] = A[M,K] x W (+ D).
//
// Why MFMA for a matrix-vector product: streaming a 4-bit weight at HBM speed
// leaves about one vector instruction per four weights per lane; converting
// every nibble to f32 and multiplying it on the vector ALU costs three times
// that and makes the kernel ALU-bound.  Here the vector ALU only masks nibbles
// into place (5 instructions per 8 weights); the multiply-adds run on
// v_mfma_f32_4x4x4_16B_f16, whose 16 independent 4x4 blocks fit the problem.
// With b = lane/4 the MFMA block and i, j = lane%4:
//   lane (b, j) supplies column j of block b's B operand: four weights of ITS OWN
//     quant block (output column 4q+j, K block kb0+b);
//   lane (b, i) supplies row i of block b's A operand: four activations of K block
//     kb0+b; row 0/1 = high/low half of an fp16 split of activation row 0, row
//     2/3 the same for activation row 1;
//   lane (b, j) receives D[i][j], i = 0..3: the dot products of its own weights
//     with the four activation rows, so scaling by the block's d stays in-lane.
// Eight such MFMAs cover one 32-element quant block per lane.
//
// Exactness.  A nibble n masked to bits 4-7 of an fp16 is the subnormal
// n * 2^-20, and the matrix cores do not flush fp16 subnormals.  (Bits 0-3,
// n * 2^-24, would save the shifts but is measurably worse: the MFMA datapath
// aligns products by the operands' nominal exponents and drops low bits of
// mantissas with many leading zeros.  Q8 bytes, q + 128 in bits 0-7, have few
// leading zeros and are fine.)  Activations are split x = hi + lo into two fp16 after
// scaling each 32-element K block by its own power of two (|x| < 2^12; the
// scale needs only the block's four preparing lanes, no workgroup-wide
// reduction), so products are exact in f32
// and only the f32 accumulation rounds: the result carries ~21 bits of x, not
// 11.  Per block the identity used is
//   sum_k (n_k d + m) x_k = d * (sum_k n_k x_k - 8 S) + (m + 8 d) * S,  S = sum_k x_k :
// the nibbles are centred (n - 8) so that neither term is large against the
// result, and "- 8 S" enters as the MFMA chain's initial accumulator, i.e.
// before anything is scaled or summed across blocks; accumulating
// d * sum(n x) and m * sum(x) separately down a column would cancel
// catastrophically.  Q8 bytes are biased to unsigned (q + 128) and the bias
// leaves the same way (- 128 S as the initial accumulator).
//
// A wave owns four adjacent columns and walks K sixteen blocks at a time, so a
// lane's accumulator stays in a register down the whole column; the 16 lanes
// of a column are summed once per column quad.  The activations' A operands
// are prepared once per workgroup in LDS, laid out so that consecutive lanes
// read consecutive 16-byte chunks.
#pragma once
#include "kernels_common.hip.h"
#include "kernels_gemv_prep.hip.h"

namespace mgn {
namespace {

// Up to three weights that share K, the format and the activations, served by one launch
// (the q, k and v projections of a decode layer): their column quads are numbered one
// after the other and every wave looks up which weight its quad belongs to.
constexpr int kMaxBatch = 3;
struct GemvBatch {
  WeightView w[kMaxBatch];
  const float* d[kMaxBatch];
  float* c[kMaxBatch];
  uint32_t first_quad[kMaxBatch];  // [0] = 0; unused entries 0xFFFFFFFF
};
// K split over workgroups (KSPLIT): blockIdx.y is the K part; `kdim` is then one part's K.
struct GemvSplit {
  uint32_t k_full;     // the weight's K: column stride of its blocks, row stride of the activations
  uint32_t kparts;
  float* handover;     // [kparts - 1][MROWS][n] partial sums of all parts but the last; kHandoverEmpty between launches
  uint32_t spin_limit; // polls after which the adding workgroup stops waiting for a partial sum
  uint32_t* fault_flag;  // set when it did
  uint32_t epilogue;   // unary operations on the output (apply_epilogue); needed with or without K parts
};
template <typename T>
__device__ __forceinline__ T pick3(uint32_t idx, T a0, T a1, T a2) {
  return idx == 0 ? a0 : idx == 1 ? a1 : a2;
}

struct GemvPrologue {
  const float* norm_weight;  // [K], kProRmsNorm
  float eps;
};

template <int FMT>
struct Raw;
template <>
struct Raw<MGN_FMT_Q4> {
  uint4 q;
  uint32_t meta;
  __device__ __forceinline__ void load_at(const char* pq, const char* pm) {
    q = stream_load_u128(pq);
    meta = stream_load_u32(pm);
  }
};
// Q8: a lane does not fetch "its" 32-byte block with two 16-byte loads (each load instruction
// would then touch only half of every cache line it brings in, and the line is fetched from
// L2 twice).  Instead the 16 lanes of a column read 16 consecutive 16-byte pieces per load:
// lane b gets half (b & 1) of K block kb0 + b/2 from the first load and the same half of
// block kb0 + 8 + b/2 from the second.  Each half block carries its own scale and its own
// MFMA chain; the A operands are read from LDS to match.
template <>
struct Raw<MGN_FMT_Q8> {
  uint4 q0, q1;
  uint32_t meta;  // scale of block kb0 + b: the scales of the two half blocks come from lanes b/2 and 8 + b/2
  // pq: this lane's half of block kb0 + b/2 (the partner block is 8 blocks further on); pm: scale of block kb0 + b
  __device__ __forceinline__ void load_at(const char* pq, const char* pm) {
    q0 = stream_load_u128(pq);
    q1 = stream_load_u128(pq + 8 * 32);
    meta = stream_load_u16(pm);
  }
};

// LDS entries of the chain constants per K block: one for a Q4 block, one per half for Q8
template <int FMT>
constexpr uint32_t cinit_per_block() { return FMT == MGN_FMT_Q8 ? 2u : 1u; }
// Padding (in 16-byte units) behind every chunk plane.  Q8 lanes of one LDS access read from
// two planes at once (chunks 2h and 2h+1 of half h); the padding moves those onto different banks.
template <int FMT>
constexpr uint32_t plane_pad(uint32_t nj) { return FMT == MGN_FMT_Q8 ? (nj == 4 ? 4u : 2u) : 0u; }

// LDS image of the activations, per workgroup:
//   chunk planes  xa[c][kb * NJ + j]  (uint4), c = 0..3: the A-operand rows of the two
//                 MFMAs that consume elements 8c..8c+7 of K block kb; j = 2*row (high
//                 halves) or 2*row + 1 (low halves);
//   cinit[kb][row] = { -bias / operand_scale * S(kb, row), the chain's initial accumulator;
//                      operand_scale / block scale, which undoes both scalings afterwards }
//                 (Q8: cinit[kb][half][row], S over the 16 elements of that half).
// Q4 pairs nibble k with k+4 in one fp16x2 mask, so the chunk is (x0,x4,x2,x6 | x1,x5,x3,x7).
// Q8 bytes come out in natural order: (x0,x1,x2,x3 | x4,x5,x6,x7).
template <int FMT>
__device__ __forceinline__ void make_chunks(const float (&x)[8], uint4& hi, uint4& lo) {
  float p[8];
  if constexpr (FMT == MGN_FMT_Q4) {
    p[0] = x[0], p[1] = x[4], p[2] = x[2], p[3] = x[6];
    p[4] = x[1], p[5] = x[5], p[6] = x[3], p[7] = x[7];
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) p[i] = x[i];
  }
  hi = make_uint4(pack_rtz(p[0], p[1]), pack_rtz(p[2], p[3]), pack_rtz(p[4], p[5]), pack_rtz(p[6], p[7]));
  const uint32_t h[4] = {hi.x, hi.y, hi.z, hi.w};
  uint32_t l[4];
#pragma unroll
  for (int i = 0; i < 4; i++) l[i] = pack_rtz(p[2 * i] - half_lo(h[i]), p[2 * i + 1] - half_hi(h[i]));
  lo = make_uint4(l[0], l[1], l[2], l[3]);
}

// blockDim.x = 64 * ksc * wnc.  Wave w: K split ks = w % ksc, quad slot wn = w / ksc.
// The workgroup owns quads [blockIdx.x * wnc, +wnc); wave (ks, wn) takes quad wn and the
// K steps [ks * STEPS, (ks+1) * STEPS) of 16 blocks each (the last split's window is moved back
// when the steps do not divide evenly).  A wave keeps two or three block loads ahead of the
// step it works on and runs straight-line code: with no branch around a load the compiler's
// wait counts are exact, so step s starts as soon as its own block has arrived while the
// later ones are still in flight.
// QPW > 1 (short K, many columns): a wave takes QPW consecutive quads, so that it still has
// QPW * STEPS block loads to keep in flight and the workgroup count stays near the CU count.
// PRO: what the activations go through on their way into LDS, in place of a kernel of its own:
//   kProNone     a[m, K] as is;
//   kProRmsNorm  a[m, K] * rsqrt(mean(a^2) + eps) * norm_weight[K]   (src/shaders/rms_norm.wgsl:1-57);
//   kProSwiglu   a[m, 2K] = gate | up  ->  gate * sigmoid(gate) * up  (src/shaders/swiglu_concat.wgsl:20-32).
// TASKS: activation chunks per thread (1 when the workgroup has a thread for every chunk; the
// prologue in front of the first weight load is then half as long).
// EXACT: K is a multiple of 512 and the K splits share the steps evenly, so every step of every
// wave is a full one and nothing needs masking.
// KSPLIT (one weight, no fused prologue, QPW = 1, steps masked as without EXACT): the activations
// of all of K would not fit in LDS (M = 4 with K > ~9000) or need more threads to prepare than a
// workgroup has (K > 16384), so grid.y workgroups share a quad group, each with a part of K
// that is a whole number of steps (the last part may reach past the end of K).  Their partial
// sums meet in the hand-over workspace, whose words all hold kHandoverEmpty between launches: every
// part but the last stores its sums there and is done; the last part (dispatched last, when the
// others are running or done; grid.x is a multiple of 8, so a quad group's parts share an XCD and
// its L2) polls each word it needs until it is no longer empty, adds the parts in part order, its
// own last (bit-identical from run to run), puts the empty pattern back and writes C.  No counter,
// no barrier, one trip to the L2 per poll; the wait is bounded (spin_limit polls, then the
// context's fault word is set and the next synchronising call reports it).
template <int FMT, int MROWS, int STEPS, int QPW, int PRO, int TASKS, bool EXACT, bool KSPLIT, bool TAIL = false>
__global__ __launch_bounds__(1024) void gemv_mfma_kernel(
    // The leading scalar arguments are what a wave needs before it can issue its first loads;
    // they are declared first (and not inside a struct) so that the dispatcher can hand them
    // over in registers (kernel-argument preload) instead of the wave fetching them from memory.
    // (three pointers and eight 32-bit values: the 14 dwords that can be preloaded)
    const float* __restrict__ a, const void* __restrict__ meta0, const void* __restrict__ quants0,
    uint32_t m_flags,  // rows in bits 0-7; bit 31: the activations are fp16 (kProNone only)
    uint32_t ksc, uint32_t wnc, uint32_t kdim, uint32_t n0, uint32_t first_quad1, uint32_t first_quad2,
    uint32_t ksc_recip,  // ceil(4096 / ksc): wave / ksc == (wave * ksc_recip) >> 12 for the 16 waves there can be
    const float* __restrict__ norm_weight, float eps, GemvBatch bt, GemvSplit sp) {
  if (KSPLIT && blockIdx.x * wnc >= (n0 + 3) / 4) return;  // padding of the grid to a multiple of 8 quad groups
  const uint32_t m = m_flags & 0xFFu;
  const bool a_f16 = PRO == kProNone && (m_flags >> 31) != 0;
  const GemvPrologue pro{norm_weight, eps};
  // one activation row of a Q4 weight: integer digits, int8 matrix instruction (see above).  (Q8 has the
  // code path too but measured 3 % slower with it, 12.35 against 12.0 us on 4096 x 14336: its bytes
  // need no unpacking in either form, so there is little vector-ALU work to save.)
  constexpr bool I8 = MROWS == 1 && FMT == MGN_FMT_Q4;
  constexpr int NJ = 2 * MROWS;       // A rows in LDS: hi and lo of every activation row
  constexpr int NG = (MROWS + 1) / 2;  // groups of four A rows = MFMA chains per weight chunk
  extern __shared__ uint4 lds4[];
  // this wave's weight: the one whose quad range holds the wave's (first) quad
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t nthreads = 64 * ksc * wnc;  // = blockDim.x, without reading it from memory
  const uint32_t gquad_u = (blockIdx.x * wnc + ((wave_u * ksc_recip) >> 12)) * QPW;
  const uint32_t widx = (gquad_u >= first_quad1 ? 1u : 0u) + (gquad_u >= first_quad2 ? 1u : 0u);
  WeightView w;
  w.meta = meta0;
  w.quants = quants0;
  w.n = n0;
  if (widx != 0) {  // a later weight of a batch: its view comes from the argument block in memory
    asm volatile("" ::: "memory");  // keep these loads (and the wait for them) inside the branch
    w.meta = widx == 1 ? bt.w[1].meta : bt.w[2].meta;
    w.quants = widx == 1 ? bt.w[1].quants : bt.w[2].quants;
    w.n = widx == 1 ? bt.w[1].n : bt.w[2].n;
  }
  w.k = kdim;
  w.fmt = FMT;
  const uint32_t quad_base = pick3(widx, 0u, first_quad1, first_quad2);  // first quad of that weight
  const uint32_t bpc = w.k / 32;
  static_assert(!KSPLIT || (!EXACT && PRO == kProNone && QPW == 1), "K parts come with masked steps, one quad per wave and no prologue");
  static_assert(!TAIL || (FMT == MGN_FMT_Q4 && QPW > 1 && EXACT && !KSPLIT && PRO == kProNone),
                "the shared tail step: Q4, several quads per wave, full regular steps, one K part, no prologue");
  const uint32_t kpart = KSPLIT ? blockIdx.y : 0u;
  const uint32_t bpc_full = KSPLIT ? sp.k_full / 32 : bpc;  // blocks per column of the weight
  const uint32_t kb_part = kpart * bpc;                     // this workgroup's first K block
  const uint32_t bpc_live = KSPLIT ? min(bpc, bpc_full - kb_part) : bpc;  // blocks of this part that exist
  const uint32_t bpc_pad = (bpc + 15) & ~15u;
  constexpr uint32_t CPB = cinit_per_block<FMT>();
  const uint32_t plane = bpc_pad * NJ + plane_pad<FMT>(NJ);
  const uint32_t nwaves = ksc * wnc;
  uint4* xa = lds4;                                   // [4][plane]
  float2* cinit = (float2*)(lds4 + 4 * plane);        // [bpc_pad][CPB][MROWS]
  float* red = (float*)(cinit + bpc_pad * CPB * MROWS);  // [wnc][ksc][MROWS][4]
  float* nrm = red + wnc * ksc * MROWS * 4;           // [16 waves][MROWS] sums of squares (kProRmsNorm)

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  // everything derived from the wave index is wave-uniform: keep it in scalar registers
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wn = (wave * ksc_recip) >> 12, ks = wave - wn * ksc;
  const uint32_t b = lane >> 2, i = lane & 3;
  const uint32_t quad0 = blockIdx.x * wnc * QPW;  // first quad of the workgroup, numbered over the whole batch
  const uint32_t nquads = (w.n + 3) / 4;
  const uint32_t quad = quad0 + wn * QPW - quad_base;  // first of this wave's QPW quads, within its weight
  const uint32_t steps_total = bpc_pad / 16;
  // The wave's window of STEPS steps.  When the K splits do not share the steps evenly the
  // last split's window is moved back to end with the last step; the steps it then has in
  // common with its neighbour count for nothing (their scales are read as zero).
  uint32_t step_begin = ks * STEPS, first_own = 0;
  if (!EXACT && step_begin + STEPS > steps_total) {
    first_own = step_begin + STEPS - steps_total;
    step_begin = steps_total - STEPS;
  }
  const bool wave_live = quad < nquads;  // a wave without a quad only helps to prepare the activations
  const uint32_t kb_first = step_begin * 16 + b;  // this lane's K block at step 0

  // Memory returns a wave's loads in issue order, so the (small, cache-resident)
  // activation loads go first and the weight loads right behind them: the activation
  // prep below then waits for its own data only, while the weights stream in.
  // One task = 8 consecutive activations of one row = one A chunk; the 4 tasks of a K
  // block sit in one lane quad.  A thread holds TASKS tasks in registers.
  float4 xraw[TASKS][MROWS][2];
  float4 xup[PRO == kProSwiglu ? TASKS : 1][MROWS][2];   // the "up" halves
  float4 gw[PRO == kProRmsNorm ? TASKS : 1][2];          // norm weights of the task's 8 columns
  const uint32_t a_stride = KSPLIT ? sp.k_full : PRO == kProSwiglu ? 2 * w.k : w.k;
#pragma unroll
  for (int tt = 0; tt < TASKS; tt++) {
    const uint32_t t = tid + tt * nthreads, kb = t >> 2, ch = t & 3;
    const bool live = kb < bpc_live;
#pragma unroll
    for (int r = 0; r < MROWS; r++) {
      // always load (from element 0 when there is nothing to load) and zero afterwards
      const bool ok = live && (uint32_t)r < m;
      const size_t off = ok ? (size_t)r * a_stride + (size_t)(kb_part + kb) * 32 + ch * 8 : (size_t)0;
      if (a_f16) {  // eight halves in one 16-byte load; widened once the weight loads are on their way
        xraw[tt][r][0] = *(const float4*)((const _Float16*)(const void*)a + off);
        xraw[tt][r][1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      } else {
        const float4* src = (const float4*)(a + off);
        xraw[tt][r][0] = src[0];
        xraw[tt][r][1] = src[1];
      }
      if constexpr (PRO == kProSwiglu) {
        const float4* up = (const float4*)(a + (ok ? (size_t)r * a_stride + w.k + (size_t)kb * 32 + ch * 8 : (size_t)0));
        xup[tt][r][0] = up[0];
        xup[tt][r][1] = up[1];
      }
    }
    if constexpr (PRO == kProRmsNorm) {
      const float4* gp = (const float4*)(pro.norm_weight + (live ? (size_t)kb * 32 + ch * 8 : (size_t)0));
      gw[tt][0] = gp[0];
      gw[tt][1] = gp[1];
    }
  }
  // Weight blocks: kDepth loads run ahead of the step that consumes them.  That is enough
  // to keep the memory system busy; issuing every load up front would only park the wave
  // in the load queue (which drains at HBM speed) before it could prepare any activations.
  // load t = q * STEPS + s: K step s of the wave's quad q
  constexpr int TS = STEPS * QPW;
  // One row with the shared tail step (short K, e.g. 576 x 49152: four one-step quads and the tail
  // make five loads per wave): all five go out before the activations are prepared, which is little
  // work at such a K, so none of them pays a second trip to memory behind the barrier (5.94 -> 5.54
  // us; 640 x 32768 5.06 -> 4.74; with more rows the prologue is longer and the deeper queue loses).
  // (One row of Q4 with four ahead instead of three gains 0.15 us on 4096 x 14336 on three boxes of
  // five and loses 0.26 us there and 0.55 us on 14336 x 4096 on a fourth: three it stays, 7.68-7.73
  // us on all five.)
  // Three or four rows of Q4: two ahead (the rows' operands and sums leave fewer registers for loads
  // in flight; 4096 x 14336 at M = 4 11.7 -> 11.35 us, 14336 x 4096 13.7 -> 13.45; one ahead is slower again).
  constexpr int kDepth = (TAIL && MROWS == 1) ? 5 : (MROWS > 2 && FMT == MGN_FMT_Q4) ? 2 : prefetch_depth<FMT>();
  // TAIL: K is STEPS full steps plus 1, 2 or 4 leftover blocks per column.  Instead of a second,
  // nearly empty step for every quad, one more step takes the leftovers of all QPW quads at once:
  // the MFMA's 16 blocks are independent, so slot b serves quad b / T, K block 16 * STEPS + b % T.
  constexpr int TS_ALL = TS + (TAIL ? 1 : 0);
  Raw<FMT> blk[TS_ALL];
  // Q8: first block of this lane's pair, see Raw<MGN_FMT_Q8>
  const uint32_t kb8_first = step_begin * 16 + (b >> 1);
  // A lane's loads are its base pointer plus a constant: no address arithmetic or range
  // checks per step.  The column index is clamped (a last quad with fewer than four columns,
  // a wave without a quad); lanes of the last step that lie past the end of K read the
  // blocks that follow in memory (the next column's, or the padding behind the last
  // column) against all-zero activations, and their scales are read as zero.
  constexpr uint32_t QB = FMT == MGN_FMT_Q8 ? 32 : 16, MB = FMT == MGN_FMT_Q8 ? 2 : 4;  // bytes per block
  const char* pq[QPW];
  const char* pm[QPW];
#pragma unroll
  for (int q = 0; q < QPW; q++) {
    const uint32_t col = min((quad + q) * 4 + i, w.n - 1);
    const uint32_t at0 = col * bpc_full + kb_part;
    pq[q] = (const char*)w.quants + (size_t)(at0 + (FMT == MGN_FMT_Q8 ? kb8_first : kb_first)) * QB +
            (FMT == MGN_FMT_Q8 ? (b & 1) * 16 : 0);
    pm[q] = (const char*)w.meta + (size_t)(at0 + kb_first) * MB;
  }
  uint32_t tail_q = 0, tail_kb = 0;  // this lane's quad (within the wave) and K block in the tail step
  const char* pq_tail = nullptr;
  const char* pm_tail = nullptr;
  if constexpr (TAIL) {
    const uint32_t tcount = bpc - 16 * STEPS;  // 1, 2 or 4, and QPW * tcount <= 16 (the planner sees to both)
    const uint32_t tshift = (uint32_t)__builtin_ctz(tcount);
    tail_q = b >> tshift;  // slots with tail_q >= QPW serve nobody: their results are never selected
    tail_kb = 16 * STEPS + (b & (tcount - 1));
    const uint32_t col = min((quad + min(tail_q, (uint32_t)QPW - 1)) * 4 + i, w.n - 1);
    pq_tail = (const char*)w.quants + ((size_t)col * bpc_full + tail_kb) * QB;
    pm_tail = (const char*)w.meta + ((size_t)col * bpc_full + tail_kb) * MB;
  }
  auto fetch = [&](int t) {
    if (TAIL && t == TS) {
      blk[t].load_at(pq_tail, pm_tail);
      return;
    }
    const int q = t / STEPS, s = t % STEPS;
    blk[t].load_at(pq[q] + s * (16 * QB), pm[q] + s * (16 * MB));
  };
  // (a wave without a quad issues these too, from the last column's blocks, and skips the
  // walk; a branch around the loads would make every wave wait for them at the join)
#pragma unroll
  for (int t = 0; t < TS_ALL && t < kDepth; t++) {
    fetch(t);
    __builtin_amdgcn_sched_barrier(0);  // in this order: step 0 waits for its own block only
  }
  for (uint32_t t = tid; t < wnc * ksc * MROWS * 4; t += nthreads) red[t] = 0.0f;

  if (a_f16) {
#pragma unroll
    for (int tt = 0; tt < TASKS; tt++)
#pragma unroll
      for (int r = 0; r < MROWS; r++) {
        const float4 h = xraw[tt][r][0];
        const uint32_t h0 = __builtin_bit_cast(uint32_t, h.x), h1 = __builtin_bit_cast(uint32_t, h.y);
        const uint32_t h2 = __builtin_bit_cast(uint32_t, h.z), h3 = __builtin_bit_cast(uint32_t, h.w);
        xraw[tt][r][0] = make_float4(half_lo(h0), half_hi(h0), half_lo(h1), half_hi(h1));
        xraw[tt][r][1] = make_float4(half_lo(h2), half_hi(h2), half_lo(h3), half_hi(h3));
      }
  }
  // ---- fused prologue: turn the raw loads into the matmul's activations ----
  if constexpr (PRO == kProSwiglu) {
#pragma unroll
    for (int tt = 0; tt < TASKS; tt++)
#pragma unroll
      for (int r = 0; r < MROWS; r++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const float4 g4 = xraw[tt][r][h], u4 = xup[tt][r][h];
          xraw[tt][r][h] = make_float4(swiglu_act(g4.x, u4.x), swiglu_act(g4.y, u4.y), swiglu_act(g4.z, u4.z),
                                       swiglu_act(g4.w, u4.w));
        }
  }
  if constexpr (PRO == kProRmsNorm) {
    // x * rstd * g is staged as x * g: the row's rstd is one factor for all of K, so it is applied
    // to the finished sums instead (rms_rstd below) and nothing waits for the row's sum of squares
    // before the staging.  The sums of squares go to LDS per wave; the barrier behind the staging
    // publishes them.
#pragma unroll
    for (int r = 0; r < MROWS; r++) {
      float ss = 0.0f;
#pragma unroll
      for (int tt = 0; tt < TASKS; tt++) {
        const uint32_t kb = (tid + tt * nthreads) >> 2;
        if (kb < bpc_live && (uint32_t)r < m) {
#pragma unroll
          for (int h = 0; h < 2; h++) {
            const float4 v = xraw[tt][r][h];
            ss = __fmaf_rn(v.x, v.x, ss);
            ss = __fmaf_rn(v.y, v.y, ss);
            ss = __fmaf_rn(v.z, v.z, ss);
            ss = __fmaf_rn(v.w, v.w, ss);
          }
        }
      }
      ss = group_sum<64>(ss);
      if (lane == 0) nrm[wave * MROWS + r] = ss;
#pragma unroll
      for (int tt = 0; tt < TASKS; tt++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const float4 v = xraw[tt][r][h], g4 = gw[tt][h];
          xraw[tt][r][h] = make_float4(v.x * g4.x, v.y * g4.y, v.z * g4.z, v.w * g4.w);
        }
    }
  }
  // kProRmsNorm: 1 / sqrt(mean(x^2) + eps) of row r, from the waves' sums (valid behind the staging barrier)
  auto rms_rstd = [&](uint32_t r) {
    const float tot = group_sum<16>((lane & 15u) < nwaves ? nrm[(lane & 15u) * MROWS + r] : 0.0f);
    return 1.0f / sqrtf(tot / (float)w.k + pro.eps);
  };

  // ---- activations -> LDS (once per workgroup) ----
#pragma unroll
  for (int tt = 0; tt < TASKS; tt++) {
    const uint32_t t = tid + tt * nthreads, kb = t >> 2, ch = t & 3;
    if (t < bpc_pad * 4) {  // whole waves take this branch together (bpc_pad * 4 is a multiple of 64)
#pragma unroll
      for (int r = 0; r < MROWS; r++) {
        float4 v0 = xraw[tt][r][0], v1 = xraw[tt][r][1];
        if (!(kb < bpc_live && (uint32_t)r < m)) v0 = v1 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        // block maximum over the quad's 32 values; NaN never wins fmaxf, an infinity
        // does and switches scaling off
        float am = fmaxf(fmaxf(fmaxf(fabsf(v0.x), fabsf(v0.y)), fmaxf(fabsf(v0.z), fabsf(v0.w))),
                         fmaxf(fmaxf(fabsf(v1.x), fabsf(v1.y)), fmaxf(fabsf(v1.z), fabsf(v1.w))));
        if constexpr (I8) {
          // integers cannot carry a NaN along: a block that holds one (or an infinity, or values
          // beyond 2^100, which are not rescaled) is given a NaN factor, so its column sums come
          // out non-finite as the reference's would
          const bool has_nan = __builtin_isunordered(v0.x, v0.y) || __builtin_isunordered(v0.z, v0.w) ||
                               __builtin_isunordered(v1.x, v1.y) || __builtin_isunordered(v1.z, v1.w);
          am = has_nan ? __builtin_inff() : am;
        }
        am = fmaxf(am, dpp_move<kDppQuadXor1>(am));
        am = fmaxf(am, dpp_move<kDppQuadXor2>(am));
        float inv;
        float scale = block_scale(am, &inv);
        if constexpr (I8) {
          // |x| * scale < 2^20 (block_scale leaves 2^12), so that rounding cannot reach 2^21 and the top
          // digit stays within int8.  Blocks that block_scale leaves alone take the factor too: all
          // zero stays zero, below 2^-100 rounds to zero, beyond 2^100 gets the NaN factor below.
          scale *= 256.0f, inv *= 0.00390625f;
          if (!(am < 1.0e30f)) inv = __builtin_nanf("");
          const float x[8] = {v0.x * scale, v0.y * scale, v0.z * scale, v0.w * scale,
                              v1.x * scale, v1.y * scale, v1.z * scale, v1.w * scale};
          uint32_t dlo[3], dhi[3];
          int isum;
          uint32_t* const xw = (uint32_t*)xa;
          if constexpr (FMT == MGN_FMT_Q4) {
            const int order[8] = {0, 2, 4, 6, 1, 3, 5, 7};
            make_digits(x, order, dlo, dhi, &isum);
#pragma unroll
            for (int pl = 0; pl < 3; pl++) *(uint2*)(xw + kb * 32 + pl * 8 + 2 * ch) = make_uint2(dlo[pl], dhi[pl]);
            isum += __builtin_amdgcn_update_dpp(0, isum, kDppQuadXor1, 0xF, 0xF, true);
            isum += __builtin_amdgcn_update_dpp(0, isum, kDppQuadXor2, 0xF, 0xF, true);
            if (ch == 0) cinit[kb * MROWS + r] = make_float2(-8.0f * (float)isum, inv);
          } else {
            const int order[8] = {0, 1, 2, 3, 4, 5, 6, 7};
            make_digits(x, order, dlo, dhi, &isum);
            // half ch / 2 of the block, MFMAs 2 (ch % 2) and 2 (ch % 2) + 1 of that half
#pragma unroll
            for (int pl = 0; pl < 3; pl++) *(uint2*)(xw + kb * 32 + (ch >> 1) * 16 + pl * 4 + 2 * (ch & 1)) = make_uint2(dlo[pl], dhi[pl]);
            if ((ch & 1) == 0) cinit[(kb * 2 + (ch >> 1)) * MROWS + r] = make_float2(0.0f, inv);
          }
        } else {
        const float x[8] = {v0.x * scale, v0.y * scale, v0.z * scale, v0.w * scale,
                            v1.x * scale, v1.y * scale, v1.z * scale, v1.w * scale};
        uint4 hi, lo;
        make_chunks<FMT>(x, hi, lo);
        xa[ch * plane + kb * NJ + 2 * r] = hi;
        xa[ch * plane + kb * NJ + 2 * r + 1] = lo;
        float s = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
        s += dpp_move<kDppQuadXor1>(s);
        constexpr float bias = FMT == MGN_FMT_Q4 ? 8.0f : 128.0f;
        if constexpr (FMT == MGN_FMT_Q8) {
          // chunks 0,1 and 2,3 are the two halves of the block
          if ((ch & 1) == 0)
            cinit[(kb * 2 + (ch >> 1)) * MROWS + r] = make_float2(s * (-bias / operand_scale<FMT>()), inv * operand_scale<FMT>());
        } else {
          s += dpp_move<kDppQuadXor2>(s);
          if (ch == 0) cinit[kb * MROWS + r] = make_float2(s * (-bias / operand_scale<FMT>()), inv * operand_scale<FMT>());
        }
        }
      }
    }
  }
  lds_barrier();

  // ---- the K walk: STEPS blocks per lane, straight-line ----
  // Lanes i >= NJ have no activation row of their own; they re-read row i % NJ (a broadcast
  // in LDS) and the D entries they produce are never looked at.
  const uint32_t jrow = NJ < 4 ? i % NJ : i;
  const uint32_t scale_lane = (((b >> 1) << 2) | i) * 4;  // Q8: byte address of lane (b / 2, i) for ds_bpermute
  // Q4: K block kb_first + 16 s.  Q8: half (b & 1) of blocks kb8_first + 16 s and + 8, i.e. chunks
  // 2 (b & 1) and 2 (b & 1) + 1 of those blocks.
  const char* xa_lane = I8 ? (FMT == MGN_FMT_Q8 ? (const char*)xa + (size_t)kb8_first * 128 + (b & 1) * 64 + i * 16
                                                : (const char*)xa + (size_t)kb_first * 128 + i * 32)
                        : FMT == MGN_FMT_Q8
                            ? (const char*)xa + ((size_t)kb8_first * NJ + jrow + (size_t)2 * (b & 1) * plane) * 16
                            : (const char*)xa + ((size_t)kb_first * NJ + jrow) * 16;
  const char* ci_lane = FMT == MGN_FMT_Q8 ? (const char*)cinit + (size_t)(kb8_first * 2 + (b & 1)) * MROWS * 8
                                          : (const char*)cinit + (size_t)kb_first * MROWS * 8;
  float acc[QPW][MROWS];  // lane (b, j): sum over this lane's K blocks for column 4*(quad+q)+j, per row
#pragma unroll
  for (int q = 0; q < QPW; q++)
#pragma unroll
    for (int r = 0; r < MROWS; r++) acc[q][r] = 0.0f;
  if (wave_live) {
#pragma unroll
  for (int t = 0; t < TS_ALL; t++) {
    const int s = t % STEPS, q = t / STEPS;
    if (t + kDepth < TS_ALL) {
      // keep the load where it is written: one step's loads per step, kDepth steps ahead (with
      // constant offsets the scheduler would otherwise gather the loads of several steps)
      __builtin_amdgcn_sched_barrier(0);
      fetch(t + kDepth);
      __builtin_amdgcn_sched_barrier(0);
    }
    Raw<FMT> cur = blk[t];
    // not every step is a full one: a block past the end of K or in a step that belongs to the
    // neighbouring K split gets scale (and minimum) zero
    if constexpr (!EXACT) cur.meta = ((uint32_t)s >= first_own && kb_first + s * 16 < bpc_live) ? cur.meta : 0u;
    if constexpr (I8 && FMT == MGN_FMT_Q4) {
      typedef int intx4 __attribute__((ext_vector_type(4)));
      const bool tail_step = TAIL && t == TS;
      const char* const xa_step = tail_step ? (const char*)xa + (size_t)tail_kb * 128 + i * 32 : xa_lane + s * (16 * 128);
      const char* const ci_step = tail_step ? (const char*)cinit + (size_t)tail_kb * MROWS * 8 : ci_lane + s * (16 * MROWS * 8);
      const uint4 a0 = *(const uint4*)xa_step, a1 = *(const uint4*)(xa_step + 16);  // this lane's digit plane, 8 MFMAs
      const float2 ci0 = *(const float2*)ci_step;  // {-8 * sum of the block's integers, factor that undoes the block scale}
      const uint32_t aw[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
      const uint32_t words[4] = {cur.q.x, cur.q.y, cur.q.z, cur.q.w};
      intx4 dsum = {0, 0, 0, 0};
#pragma unroll
      for (int ch = 0; ch < 4; ch++) {
        const uint32_t wd = words[ch];
        const uint32_t even = wd & 0x0F0F0F0Fu, odd = (wd >> 4) & 0x0F0F0F0Fu;  // (n0,n2,n4,n6), (n1,n3,n5,n7)
        dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)aw[2 * ch], (int)even, dsum, 0, 0, 0);
        dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)aw[2 * ch + 1], (int)odd, dsum, 0, 0, 0);
      }
      const int tot = (((dsum[2] << 7) + dsum[1]) << 7) + dsum[0];  // digits back together: sum n * x
      const float dscale = half_bits_to_float(cur.meta & 0xFFFFu);
      const float mneg = __fmaf_rn(-0.125f, half_bits_to_float(cur.meta >> 16), -dscale);  // (m + 8 d) S = mneg * (-8 S)
      float v = dscale * ((float)tot + ci0.x);
      v = __fmaf_rn(mneg, ci0.x, v);
      if (tail_step) {
#pragma unroll
        for (int qq = 0; qq < QPW; qq++) {
          const float sum = __fmaf_rn(v, ci0.y, acc[qq][0]);
          acc[qq][0] = tail_q == (uint32_t)qq ? sum : acc[qq][0];
        }
      } else {
        constexpr int QMAX = QPW - 1;
        const int qa = q < QPW ? q : QMAX;
        acc[qa][0] = __fmaf_rn(v, ci0.y, acc[qa][0]);
      }
    } else if constexpr (I8) {
      typedef int intx4 __attribute__((ext_vector_type(4)));
      // Q8: two half blocks per step; the weight bytes are the B operand as they are
      const int dscale_own = __builtin_bit_cast(int, half_bits_to_float(cur.meta));
      const float dscales[2] = {__builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)scale_lane, dscale_own)),
                                __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)scale_lane + 8 * 4 * 4, dscale_own))};
#pragma unroll
      for (int hb = 0; hb < 2; hb++) {
        const uint4 qw = hb == 0 ? cur.q0 : cur.q1;
        const uint4 a4 = *(const uint4*)(xa_lane + s * (16 * 128) + hb * (8 * 128));
        const float2 ci0 = *(const float2*)(ci_lane + s * (16 * 2 * MROWS * 8) + hb * (8 * 2 * MROWS * 8));
        intx4 dsum = {0, 0, 0, 0};
        dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)a4.x, (int)qw.x, dsum, 0, 0, 0);
        dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)a4.y, (int)qw.y, dsum, 0, 0, 0);
        dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)a4.z, (int)qw.z, dsum, 0, 0, 0);
        dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)a4.w, (int)qw.w, dsum, 0, 0, 0);
        const int tot = (((dsum[2] << 7) + dsum[1]) << 7) + dsum[0];
        acc[q][0] = __fmaf_rn(dscales[hb] * (float)tot, ci0.y, acc[q][0]);
      }
    } else if constexpr (FMT == MGN_FMT_Q4) {
      const bool tail_step = TAIL && t == TS;
      // the step's activations and block constants: K block kb_first + 16 s, or the lane's tail block
      const char* const xa_step = tail_step ? (const char*)xa + ((size_t)tail_kb * NJ + jrow) * 16 : xa_lane + s * (16 * NJ * 16);
      const char* const ci_step = tail_step ? (const char*)cinit + (size_t)tail_kb * MROWS * 8 : ci_lane + s * (16 * MROWS * 8);
      // A operands: 4 chunks of 16 bytes, consecutive lanes -> consecutive chunks; with more than
      // two activation rows a second group of four A rows (rows 2 and 3, hi and lo) follows
      uint4 ax[NG][4];
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int ch = 0; ch < 4; ch++)
          ax[g][ch] = *(const uint4*)(xa_step + ch * plane * 16 + g * 64);
      float2 ci[MROWS];  // {chain start value, factor that undoes the operand and block scales}
#pragma unroll
      for (int r = 0; r < MROWS; r++) ci[r] = *(const float2*)(ci_step + r * 8);
      // the centring term rides in as the chain's start value (rows 2r and 2r+1 add up later)
      floatx4 dsum[NG];
#pragma unroll
      for (int g = 0; g < NG; g++) dsum[g] = floatx4{ci[2 * g].x, 0.0f, 2 * g + 1 < MROWS ? ci[2 * g + 1 < MROWS ? 2 * g + 1 : 0].x : 0.0f, 0.0f};
      const uint32_t words[4] = {cur.q.x, cur.q.y, cur.q.z, cur.q.w};
#pragma unroll
      for (int ch = 0; ch < 4; ch++) {
        // every nibble pair goes to bits 4-7 / 20-23: n * 2^-20 in each fp16 half
        const uint32_t wd = words[ch];
        const uint32_t e0 = (wd << 4) & 0x00F000F0u, o0 = wd & 0x00F000F0u;         // (n0,n4), (n1,n5)
        const uint32_t e1 = (wd >> 4) & 0x00F000F0u, o1 = (wd >> 8) & 0x00F000F0u;  // (n2,n6), (n3,n7)
#pragma unroll
        for (int g = 0; g < NG; g++) {
          dsum[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_half4(ax[g][ch].x, ax[g][ch].y), as_half4(e0, e1), dsum[g], 0, 0, 0);
          dsum[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(as_half4(ax[g][ch].z, ax[g][ch].w), as_half4(o0, o1), dsum[g], 0, 0, 0);
        }
      }
      const float dscale = half_bits_to_float(cur.meta & 0xFFFFu);
      // (m + 8 d) * S with S = -ci * operand_scale / 8: fold the -1/8 into the block constant
      const float mneg = __fmaf_rn(-0.125f, half_bits_to_float(cur.meta >> 16), -dscale);
#pragma unroll
      for (int r = 0; r < MROWS; r++) {
        float v = dscale * (dsum[r / 2][2 * (r % 2)] + dsum[r / 2][2 * (r % 2) + 1]);
        v = __fmaf_rn(mneg, ci[r].x, v);
        if (tail_step) {
          // the slot's quad differs from lane to lane: every accumulator takes what is its own
#pragma unroll
          for (int qq = 0; qq < QPW; qq++) {
            const float sum = __fmaf_rn(v, ci[r].y, acc[qq][r]);
            acc[qq][r] = tail_q == (uint32_t)qq ? sum : acc[qq][r];
          }
        } else {
          constexpr int QMAX = QPW - 1;
          const int qa = q < QPW ? q : QMAX;  // (q == QPW only in the tail step, which does not come here)
          acc[qa][r] = __fmaf_rn(v, ci[r].y, acc[qa][r]);
        }
      }
    } else {
      // two half blocks per step, each with its own chain of four MFMAs and its own scale
      // the half blocks' scales sit in lanes (b / 2, i) and (8 + b / 2, i); fetched first so that
      // the answers are back when the chains end
      const int dscale_own = __builtin_bit_cast(int, half_bits_to_float(cur.meta));
      const float dscales[2] = {__builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)scale_lane, dscale_own)),
                          __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)scale_lane + 8 * 4 * 4, dscale_own))};
#pragma unroll
      for (int hb = 0; hb < 2; hb++) {
        const uint4 qw = hb == 0 ? cur.q0 : cur.q1;
        uint4 ax[NG][2];
#pragma unroll
        for (int g = 0; g < NG; g++)
#pragma unroll
          for (int c2 = 0; c2 < 2; c2++)
            ax[g][c2] = *(const uint4*)(xa_lane + s * (16 * NJ * 16) + hb * (8 * NJ * 16) + c2 * plane * 16 + g * 64);
        float2 ci[MROWS];
#pragma unroll
        for (int r = 0; r < MROWS; r++)
          ci[r] = *(const float2*)(ci_lane + s * (16 * 2 * MROWS * 8) + hb * (8 * 2 * MROWS * 8) + r * 8);
        floatx4 dsum[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) dsum[g] = floatx4{ci[2 * g].x, 0.0f, 2 * g + 1 < MROWS ? ci[2 * g + 1 < MROWS ? 2 * g + 1 : 0].x : 0.0f, 0.0f};
        const uint32_t words[4] = {qw.x, qw.y, qw.z, qw.w};
#pragma unroll
        for (int wi = 0; wi < 4; wi++) {
          const uint32_t u8 = words[wi] ^ 0x80808080u;  // q + 128 in every byte
          const uint32_t lo2 = __builtin_amdgcn_perm(0u, u8, 0x0c010c00u);  // (b0, b1) as fp16 mantissas
          const uint32_t hi2 = __builtin_amdgcn_perm(0u, u8, 0x0c030c02u);  // (b2, b3)
#pragma unroll
          for (int g = 0; g < NG; g++) {
            const uint4 a8 = ax[g][wi >> 1];
            const half4 aop = (wi & 1) == 0 ? as_half4(a8.x, a8.y) : as_half4(a8.z, a8.w);
            dsum[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(aop, as_half4(lo2, hi2), dsum[g], 0, 0, 0);
          }
        }
        const float dscale = dscales[hb];
#pragma unroll
        for (int r = 0; r < MROWS; r++) {
          const float v = dscale * (dsum[r / 2][2 * (r % 2)] + dsum[r / 2][2 * (r % 2) + 1]);
          acc[q][r] = __fmaf_rn(v, ci[r].y, acc[q][r]);
        }
      }
    }
  }
  }
  // ---- sum the 16 lanes of each column ----
  if (!KSPLIT && (QPW > 1 || ksc == 1)) {
    // no K split (always the case with QPW > 1): lanes 0..3 hold the four finished columns of a quad
#pragma unroll
    for (int q = 0; q < QPW; q++) {
      uint32_t r;
      bool writer;
      const float tot = sum_rows_over_blocks<MROWS>(acc[q], lane, &r, &writer);
      const uint32_t n = (quad + q) * 4 + (lane & 3u);
      float tot_r = tot;
      if constexpr (PRO == kProRmsNorm) tot_r *= rms_rstd(min(r, (uint32_t)MROWS - 1));
      if (writer && wave_live && r < m && n < w.n) {
        const size_t o = (size_t)r * w.n + n;
        const float* const dres = pick3(widx, bt.d[0], bt.d[1], bt.d[2]);
        float* const c = pick3(widx, bt.c[0], bt.c[1], bt.c[2]);
        c[o] = apply_epilogue(dres ? tot_r + dres[o] : tot_r, sp.epilogue);
      }
    }
    return;
  }
  {
    uint32_t r;
    bool writer;
    const float tot = sum_rows_over_blocks<MROWS>(acc[0], lane, &r, &writer);
    if (writer && wave_live && r < (uint32_t)MROWS) red[((wn * ksc + ks) * MROWS + r) * 4 + (lane & 3u)] = tot;
  }
  lds_barrier();
  // ---- combine the K splits, then the K parts, add the residual, store ----
  float rstd_row[MROWS];
#pragma unroll
  for (int r = 0; r < MROWS; r++) rstd_row[r] = PRO == kProRmsNorm ? rms_rstd(r) : 1.0f;
  for (uint32_t t = tid; t < wnc * MROWS * 4; t += nthreads) {
    const uint32_t col = t & 3, r = (t >> 2) % MROWS, ql = t / (4 * MROWS);
    // the quads of a workgroup may belong to different weights of the batch
    const uint32_t gq = quad0 + ql;
    const uint32_t wi = (gq >= first_quad1 ? 1u : 0u) + (gq >= first_quad2 ? 1u : 0u);
    const uint32_t wn_cols = pick3(wi, n0, bt.w[1].n, bt.w[2].n);
    const uint32_t n = (gq - pick3(wi, 0u, first_quad1, first_quad2)) * 4 + col;
    if (r < m && n < wn_cols) {
      float v = 0.0f;
      for (uint32_t s = 0; s < ksc; s++) v += red[((ql * ksc + s) * MROWS + r) * 4 + col];
      if constexpr (PRO == kProRmsNorm) {
        float f = rstd_row[0];
#pragma unroll
        for (int rr = 1; rr < MROWS; rr++) f = r == (uint32_t)rr ? rstd_row[rr] : f;
        v *= f;
      }
      if constexpr (KSPLIT) {
        float* const slot0 = sp.handover + (size_t)r * wn_cols + n;  // part p's word: slot0 + p * MROWS * wn_cols
        const size_t pstride = (size_t)MROWS * wn_cols;
        if (kpart + 1 < sp.kparts) {
          const uint32_t bits = __builtin_bit_cast(uint32_t, v);
          __hip_atomic_store(slot0 + kpart * pstride, __builtin_bit_cast(float, bits == kHandoverEmpty ? 0x7FC00000u : bits),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          continue;
        }
        float acc = 0.0f;
        bool gave_up = false;
        for (uint32_t p = 0; p + 1 < sp.kparts; p++) {
          float x = __builtin_bit_cast(float, kHandoverEmpty);
          for (uint32_t polls = 0;; polls++) {
            if (polls >= sp.spin_limit) {  // (a limit of 0 looks at nothing: the give-up path, for tests)
              gave_up = true;
              break;
            }
            x = __hip_atomic_load(slot0 + p * pstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (__builtin_bit_cast(uint32_t, x) != kHandoverEmpty) break;
            __builtin_amdgcn_s_sleep(1);
          }
          acc += x;
          __hip_atomic_store(slot0 + p * pstride, __builtin_bit_cast(float, kHandoverEmpty), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        v = acc + v;
        if (gave_up && sp.fault_flag) *sp.fault_flag = 1u;
      }
      const size_t o = (size_t)r * wn_cols + n;
      const float* const dd = pick3(wi, bt.d[0], bt.d[1], bt.d[2]);
      pick3(wi, bt.c[0], bt.c[1], bt.c[2])[o] = apply_epilogue(dd ? v + dd[o] : v, sp.epilogue);
    }
  }
}

struct MfmaGemvPlan {
  uint32_t ksc, wnc, steps, qpw, tasks, grid;
  uint32_t kparts;  // workgroups sharing a quad group (1: no split over workgroups)
  uint32_t part_k;  // K of one part when kparts > 1: a whole number of 16-block steps
  bool exact;  // every step of every K split is a full one
  uint32_t tail;  // 0, or the leftover blocks per column (1, 2, 4) that all quads of a wave share one more step for
  size_t lds;
};

constexpr uint32_t kMaxSteps = 8;  // blocks a lane holds in flight: 8 x 20 B (Q4) or 8 x 34 B (Q8)

// `nquads`: column quads over all weights of the launch; `one_quad_per_wave`: fused prologues
// and batches of several weights come with QPW = 1 only.
bool plan_one_part(int fmt, uint32_t k, uint32_t nquads, uint32_t mrows, int num_cus, bool one_quad_per_wave, MfmaGemvPlan* out) {
  const uint32_t bpc = k / 32, bpc_pad = (bpc + 15) & ~15u;
  const uint32_t steps_total = bpc_pad / 16;
  MfmaGemvPlan p{};
  p.kparts = 1;
  // K splits: at least enough that a wave's share fits in its registers; more when there
  // are too few column quads to give every CU a handful of waves
  uint32_t ksc = (steps_total + kMaxSteps - 1) / kMaxSteps;
  if (ksc > 16) return false;
  const uint32_t want_waves = (uint32_t)num_cus * 8;
  while (ksc < 16 && nquads * ksc < want_waves && (steps_total + ksc) / (ksc + 1) >= 2) ksc++;
  p.steps = (steps_total + ksc - 1) / ksc;
  p.ksc = (steps_total + p.steps - 1) / p.steps;  // drop splits that would get no step
  // quads per wave: with a short K and very many columns a wave takes several quads, as
  // long as that leaves at least 8 waves per CU
  p.qpw = 1;
  if (p.ksc == 1 && !one_quad_per_wave)
    while (p.qpw < 4 && p.steps * p.qpw * 2 <= kMaxSteps && nquads / (p.qpw * 2) >= (uint32_t)num_cus * 8) p.qpw *= 2;
  // waves per workgroup: spread the quads evenly over the CUs (one workgroup per CU when
  // there is enough work), so the activations are prepared as few times as possible
  const uint32_t max_wnc = 16 / p.ksc;
  const uint32_t wave_quads = (nquads + p.qpw - 1) / p.qpw;  // quad groups = waves with work
  uint32_t per_cu = (wave_quads + num_cus - 1) / num_cus;
  if (per_cu > max_wnc) {
    // Several rounds of workgroups.  With the largest workgroups the last round may be nearly
    // empty (296 workgroups of 16 waves: 216 CUs idle while 40 work through a second one);
    // when that wastes more than an eighth of the time, as many workgroups go to every CU, each
    // as small as that allows.  (Smaller workgroups prepare the activations more often, so a
    // better filled last round is left alone: 8192 x 28672, an eighth exactly, lost 10-13 % to
    // this, while 5120 x 13824, 80 CUs idle in the second of two rounds, gains 3 %.)
    const uint32_t grid_max = (wave_quads + max_wnc - 1) / max_wnc;
    const uint32_t rounds = (grid_max + num_cus - 1) / num_cus;
    const uint32_t last = grid_max - (rounds - 1) * num_cus;  // workgroups in the last round
    if ((num_cus - last) * 8 > (uint32_t)num_cus * rounds) per_cu = (wave_quads + num_cus * rounds - 1) / (num_cus * rounds);
  }
  p.wnc = std::max<uint32_t>(1, std::min<uint32_t>(max_wnc, per_cu));
  // enough threads to prepare the activations (waves without a quad only help there)
  const uint32_t prep_waves = (bpc_pad * 4 + kMaxTasks * 64 - 1) / (kMaxTasks * 64);
  p.wnc = std::max<uint32_t>(p.wnc, (prep_waves + p.ksc - 1) / p.ksc);
  if (p.wnc > max_wnc) return false;
  p.grid = (wave_quads + p.wnc - 1) / p.wnc;
  p.tasks = bpc_pad * 4 <= 64 * p.ksc * p.wnc ? 1 : 2;
  p.exact = bpc % 16 == 0 && p.ksc * p.steps == steps_total;
  // A short K with a few blocks beyond its full steps (576 = 16 + 2 blocks), four quads per wave:
  // the quads share one more step for their leftovers instead of a nearly empty step each.
  p.tail = 0;
  if (fmt == MGN_FMT_Q4 && p.ksc == 1 && p.qpw == 4 && p.steps == 2 && p.tasks == 1) {
    const uint32_t left = bpc - 16;
    if (left == 1 || left == 2 || left == 4) {
      p.tail = left;
      p.steps = 1;
      p.exact = true;
    }
  }
  const uint32_t nj = 2 * mrows;
  const size_t plane = (size_t)bpc_pad * nj + (fmt == MGN_FMT_Q8 ? plane_pad<MGN_FMT_Q8>(nj) : 0u);
  const size_t cpb = fmt == MGN_FMT_Q8 ? cinit_per_block<MGN_FMT_Q8>() : 1u;
  p.lds = 4 * plane * 16 + (size_t)bpc_pad * cpb * mrows * 8 + (size_t)p.wnc * p.ksc * mrows * 16 + 16 * mrows * 4 + 64;
  if (p.lds > 150 * 1024) return false;
  *out = p;
  return true;
}

uint32_t total_quads(const LaunchArgs& x) {
  uint32_t q = (x.w.n + 3) / 4;
  for (int j = 0; j < x.n_more; j++) q += (x.more[j].w.n + 3) / 4;
  return q;
}

// The plan for a launch.  When the activations of all of K do not fit in LDS, K is cut into
// even parts that different workgroups take (plain launches only: one weight, no prologue).
bool plan_mfma_gemv(const LaunchArgs& x, uint32_t mrows, MfmaGemvPlan* out) {
  const bool plain = x.pro_kind == kProNone && x.n_more == 0;
  const uint32_t nquads = total_quads(x);
  if (plan_one_part(x.w.fmt, x.w.k, nquads, mrows, x.num_cus, !plain, out)) return true;
  if (!plain || !x.handover) return false;
  const uint32_t steps_total = (x.w.k / 32 + 15) / 16;
  // Four parts first: a workgroup then prepares a quarter of the activations and mostly needs no
  // K split of its own, which outweighs the two further partial sums per output (measured on
  // twelve shapes with K from 9728 to 32768: 2 to 25 % faster than two parts on ten, 3 % slower
  // on K = 11008).  Three, six and seven parts leave a ragged last round of workgroups.
  static const uint32_t kPartOrder[] = {4, 2, 3, 5, 6, 7, 8};
  for (const uint32_t kp : kPartOrder) {
    // parts of a whole number of 16-block steps; the last one may be short, never empty
    const uint32_t part_steps = (steps_total + kp - 1) / kp;
    if ((kp - 1) * part_steps >= steps_total) continue;
    if ((size_t)(kp - 1) * mrows * x.w.n * sizeof(float) > x.handover_bytes) continue;  // the last part keeps its own sums
    MfmaGemvPlan p;
    if (!plan_one_part(x.w.fmt, part_steps * 512, nquads, mrows, std::max(1, x.num_cus / (int)kp), true, &p)) continue;
    if (p.qpw != 1) continue;
    p.kparts = kp;
    p.part_k = part_steps * 512;
    p.exact = false;  // the K-part kernels always mask (the last part may reach past the end of K)
    *out = p;
    return true;
  }
  return false;
}

template <int FMT, int MROWS, int STEPS, int QPW, int PRO, int TASKS, bool EXACT, bool KSPLIT, bool TAIL = false>
int launch_tasks(ihipStream_t* s, const LaunchArgs& x, const MfmaGemvPlan& p) {
  auto kern = gemv_mfma_kernel<FMT, MROWS, STEPS, QPW, PRO, TASKS, EXACT, KSPLIT, TAIL>;
  static std::atomic<uint64_t> big_lds_done{0};
  if (p.lds > 64 * 1024)
    if (int e = enable_big_lds(kern, x.device, big_lds_done)) return e;
  GemvBatch bt{};
  uint32_t quads = 0;
  for (int j = 0; j < kMaxBatch; j++) {
    if (j == 0 || j <= x.n_more) {
      bt.w[j] = j == 0 ? x.w : x.more[j - 1].w;
      bt.d[j] = j == 0 ? x.d : x.more[j - 1].d;
      bt.c[j] = j == 0 ? x.c : x.more[j - 1].c;
      bt.first_quad[j] = quads;
      quads += (bt.w[j].n + 3) / 4;
    } else {
      bt.w[j] = x.w;
      bt.first_quad[j] = 0xFFFFFFFFu;
    }
  }
  const GemvSplit sp{x.w.k, p.kparts, (float*)x.handover, x.spin_limit, x.fault_flag, x.epilogue};
  // (with K parts: a multiple of 8 quad groups, so that the parts of a group run on one XCD)
  hipLaunchKernelGGL(kern, dim3(p.kparts > 1 ? (p.grid + 7) / 8 * 8 : p.grid, p.kparts), dim3(64 * p.ksc * p.wnc), p.lds, s, (const float*)x.a, x.w.meta, x.w.quants,
                     x.m | (x.a_is_f16 ? 0x80000000u : 0u), p.ksc, p.wnc, p.kparts > 1 ? p.part_k : x.w.k, x.w.n,
                     bt.first_quad[1], bt.first_quad[2],
                     (4096u + p.ksc - 1) / p.ksc, x.pro_weight, x.pro_eps, bt, sp);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

template <int FMT, int MROWS, int STEPS, int QPW, int PRO>
int launch_pro(ihipStream_t* s, const LaunchArgs& x, const MfmaGemvPlan& p) {
  if (p.kparts > 1) {
    if constexpr (PRO == kProNone && QPW == 1)
      return p.tasks == 1 ? launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 1, false, true>(s, x, p)
                          : launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 2, false, true>(s, x, p);
    return (int)hipErrorInvalidValue;
  }
  if (p.tail != 0) {
    if constexpr (FMT == MGN_FMT_Q4 && STEPS == 1 && QPW == 4 && PRO == kProNone)
      return launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 1, true, false, true>(s, x, p);
    return (int)hipErrorInvalidValue;
  }
  if (p.exact)
    return p.tasks == 1 ? launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 1, true, false>(s, x, p)
                        : launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 2, true, false>(s, x, p);
  return p.tasks == 1 ? launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 1, false, false>(s, x, p)
                      : launch_tasks<FMT, MROWS, STEPS, QPW, PRO, 2, false, false>(s, x, p);
}

template <int FMT, int MROWS, int STEPS, int QPW>
int launch_steps(ihipStream_t* s, const LaunchArgs& x, const MfmaGemvPlan& p) {
  if constexpr (QPW == 1) {  // fused prologues come with one quad per wave only
    if (x.pro_kind == kProRmsNorm) return launch_pro<FMT, MROWS, STEPS, QPW, kProRmsNorm>(s, x, p);
    if (x.pro_kind == kProSwiglu) return launch_pro<FMT, MROWS, STEPS, QPW, kProSwiglu>(s, x, p);
  }
  if (x.pro_kind != kProNone) return (int)hipErrorInvalidValue;
  return launch_pro<FMT, MROWS, STEPS, QPW, kProNone>(s, x, p);
}

template <int FMT, int MROWS>
int launch_t(ihipStream_t* s, const LaunchArgs& x) {
  MfmaGemvPlan p;
  if (!plan_mfma_gemv(x, MROWS, &p)) return (int)hipErrorInvalidValue;
  switch (p.steps * 8 + p.qpw) {
    case 1 * 8 + 1: return launch_steps<FMT, MROWS, 1, 1>(s, x, p);
    case 1 * 8 + 2: return launch_steps<FMT, MROWS, 1, 2>(s, x, p);
    case 1 * 8 + 4: return launch_steps<FMT, MROWS, 1, 4>(s, x, p);
    case 2 * 8 + 1: return launch_steps<FMT, MROWS, 2, 1>(s, x, p);
    case 2 * 8 + 2: return launch_steps<FMT, MROWS, 2, 2>(s, x, p);
    case 2 * 8 + 4: return launch_steps<FMT, MROWS, 2, 4>(s, x, p);
    case 3 * 8 + 1: return launch_steps<FMT, MROWS, 3, 1>(s, x, p);
    case 3 * 8 + 2: return launch_steps<FMT, MROWS, 3, 2>(s, x, p);
    case 4 * 8 + 1: return launch_steps<FMT, MROWS, 4, 1>(s, x, p);
    case 4 * 8 + 2: return launch_steps<FMT, MROWS, 4, 2>(s, x, p);
    case 5 * 8 + 1: return launch_steps<FMT, MROWS, 5, 1>(s, x, p);
    case 6 * 8 + 1: return launch_steps<FMT, MROWS, 6, 1>(s, x, p);
    case 7 * 8 + 1: return launch_steps<FMT, MROWS, 7, 1>(s, x, p);
    case 8 * 8 + 1: return launch_steps<FMT, MROWS, 8, 1>(s, x, p);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace
}  // namespace mgn
