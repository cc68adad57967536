// Tiled dequant-GEMM on the matrix cores for M >= 5: C[M,N] = A[M,K] x W (+ D), f32 or fp16
// activations (skinny decode batches, and prefill).
//
// The reference runs every quantized matmul with M > 1 through its 64x64x32 tiled shader,
// dequantizing each weight element on load and multiplying on the scalar ALUs
// (src/shaders/matmul.wgsl:43-90, src/codegen.rs:748-805), and keeps quantized weights off its
// tensor-core path (src/runtime.rs:1634).  Here the raw quants are the MFMA's B operand and the
// block scale is applied to the accumulators.
//
//   v_mfma_f32_16x16x32_f16: one instruction contracts one 32-element quant block of 16
//   columns against 16 activation rows.  Lane (c, g), c = lane % 16, g = lane / 16, supplies
//   k = 8g..8g+7 of column c (B) or of row c (A) and receives rows 4g..4g+3 of column c (D).
//   B operand: dword g of the block's nibbles, masked to fp16 bits 4-7 (n * 2^-20, exact;
//     Q8: the block's bytes 8g..8g+7 as (q + 128) * 2^-24 in bits 0-7).  The quants travel from
//     memory as whole 128/256-byte runs of a column's blocks, are parked in a wave-private LDS
//     slice and read back one dword (Q8: two) per lane and block.
//   A operand: the activations, converted ONCE per call by a small kernel into an "image" in
//     the instruction's own lane order (image_kernel below), which every workgroup then only
//     copies into LDS, slice by slice, double-buffered.  f32 activations are scaled per (row,
//     256-element K slice) by a power of two and split hi + lo into two fp16 operands that are
//     multiplied into the same accumulator, so products are exact, any finite magnitude is
//     representable and only f32 accumulation rounds; fp16 activations are used as they are.
//   Per block: D = sum n x on the matrix cores, then P += d * D on the vector ALU (4 FMAs per
//     lane).  The format's additive part (m * sum(x) for Q4, -128 * scale * sum(x) for Q8's byte
//     bias) is one more MFMA per slice of 8 blocks: its A operand holds the blocks' mean
//     activations (hi, lo), its B operand the blocks' m (or scale), both exact fp16 values.
//     A slice's P is multiplied by the rows' inverse power-of-two scales and added to the
//     accumulators.
//
// Work split: grid = (K parts, column groups, row groups).  A workgroup owns wnc column tiles of
// 16 columns, R row tiles of 16 rows and a range of K slices; ksc waves share a column tile and
// take the slices of a phase side by side (their sums meet in LDS, in a fixed order); with too
// few tiles to fill the chip K is also cut into parts for different workgroups, whose partial
// tiles the last one to finish adds in part order (deterministic).
#include <algorithm>

#include "kernels_common.hip.h"

namespace mgn {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));

__device__ __forceinline__ half8 as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const u32x4_t v = {a, b, c, d};
  return __builtin_bit_cast(half8, v);
}
__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ float half_lo(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[0]; }
__device__ __forceinline__ float half_hi(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[1]; }

// one dword of nibbles -> B operand (8 fp16): (n0,n4),(n1,n5),(n2,n6),(n3,n7), each n * 2^-20
__device__ __forceinline__ half8 nibbles_to_operand(uint32_t wd) {
  return as_half8((wd << 4) & 0x00F000F0u, wd & 0x00F000F0u, (wd >> 4) & 0x00F000F0u, (wd >> 8) & 0x00F000F0u);
}
// two dwords of int8 -> B operand: (b0,b1),(b2,b3),(b4,b5),(b6,b7), each (q + 128) * 2^-24
__device__ __forceinline__ half8 bytes_to_operand(uint32_t w0, uint32_t w1) {
  const uint32_t u0 = w0 ^ 0x80808080u, u1 = w1 ^ 0x80808080u;
  return as_half8(__builtin_amdgcn_perm(0u, u0, 0x0c010c00u), __builtin_amdgcn_perm(0u, u0, 0x0c030c02u),
                  __builtin_amdgcn_perm(0u, u1, 0x0c010c00u), __builtin_amdgcn_perm(0u, u1, 0x0c030c02u));
}

// max over aligned groups of 32 consecutive lanes (every lane ends with the group's maximum)
__device__ __forceinline__ float group_max32(float v) {
  v = fmaxf(v, dpp_move<kDppQuadXor1>(v));
  v = fmaxf(v, dpp_move<kDppQuadXor2>(v));
  v = fmaxf(v, dpp_move<kDppRowHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppRowMirror>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return v;
}

// Power of two that brings a row slice's largest magnitude into [2^11, 2^12) (1 if the slice
// is all zero, tiny, huge or not finite).  *inv gets the reciprocal.
__device__ __forceinline__ float slice_scale(float amax, float* inv) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, amax);
  const int e = (int)(bits >> 23) - 127;  // floor(log2(amax)) for normal values
  if (bits == 0 || e >= 100 || e <= -100) {
    *inv = 1.0f;
    return 1.0f;
  }
  const int sh = 11 - e;
  *inv = __builtin_bit_cast(float, (uint32_t)(127 - sh) << 23);
  return __builtin_bit_cast(float, (uint32_t)(127 + sh) << 23);
}

// ---- the activation image ----
// One image per (row tile of 16 rows, K slice of 8 blocks = 256 elements), in uint4 units:
//   [(kb * HL + h) * 64 + lane]  A operand of block kb, h = 0 high halves, h = 1 low halves (f32
//                                activations only: HL = 2), for A lane = row + 16 * g
//   [8 * HL * 64 + lane]         A operand of the slice's additive MFMA: lanes (row, g' < 2) hold
//                                (mean_hi | mean_lo << 16) of blocks 4g'..4g'+3, the rest is zero
//   [8 * HL * 64 + 64 + 0..15]   (as float) the rows' inverse scales times the quants' operand scale
//                                (2^20 for Q4, 2^24 for Q8; f32 activations only)
// The element order inside an operand follows the B side: Q4 pairs k with k + 4, Q8 is natural.
constexpr uint32_t kSliceBlocks = 8;
constexpr uint32_t image_units(bool f32a) { return kSliceBlocks * (f32a ? 2u : 1u) * 64u + 64u + 16u; }

// grid.x = row tiles * slices; 512 threads: half-wave r (0..15) converts row r of the tile,
// lane l = kb * 4 + g of it the 8 elements k = 32 kb + 8 g .. + 7 of the slice.
template <int FMT, bool F32A>
__global__ __launch_bounds__(512) void image_kernel(const void* __restrict__ a, uint4* __restrict__ image, uint32_t m,
                                                    uint32_t k, uint32_t nslices, uint32_t a_stride) {
  constexpr uint32_t HL = F32A ? 2 : 1;
  constexpr uint32_t UNITS = image_units(F32A);
  const uint32_t rt = blockIdx.x / nslices, sl = blockIdx.x - rt * nslices;
  const uint32_t r = threadIdx.x >> 5, l = threadIdx.x & 31, kb = l >> 2, g = l & 3;
  const uint32_t row = rt * 16 + r, k0 = sl * 256 + kb * 32 + g * 8;
  const bool ok = row < m && k0 < k;  // K is a multiple of 32: a task lies inside or outside as a whole
  float x[8];
  if constexpr (F32A) {
    const float4* src = (const float4*)((const float*)a + (ok ? (size_t)row * a_stride + k0 : (size_t)0));
    const float4 v0 = src[0], v1 = src[1];
    x[0] = v0.x, x[1] = v0.y, x[2] = v0.z, x[3] = v0.w, x[4] = v1.x, x[5] = v1.y, x[6] = v1.z, x[7] = v1.w;
  } else {
    const uint4 v = *(const uint4*)((const _Float16*)a + (ok ? (size_t)row * a_stride + k0 : (size_t)0));
    x[0] = half_lo(v.x), x[1] = half_hi(v.x), x[2] = half_lo(v.y), x[3] = half_hi(v.y);
    x[4] = half_lo(v.z), x[5] = half_hi(v.z), x[6] = half_lo(v.w), x[7] = half_hi(v.w);
  }
#pragma unroll
  for (int e = 0; e < 8; e++) x[e] = ok ? x[e] : 0.0f;
  float inv = 1.0f;
  if constexpr (F32A) {
    // NaN never wins fmaxf; an infinity does and switches scaling off
    float am = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                     fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
    am = group_max32(am);
    const float scale = slice_scale(am, &inv);
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] *= scale;
  }
  float p[8];
  if constexpr (FMT == MGN_FMT_Q4) {
    p[0] = x[0], p[1] = x[4], p[2] = x[1], p[3] = x[5], p[4] = x[2], p[5] = x[6], p[6] = x[3], p[7] = x[7];
  } else {
#pragma unroll
    for (int e = 0; e < 8; e++) p[e] = x[e];
  }
  uint4* const img = image + ((size_t)rt * nslices + sl) * UNITS;
  const uint32_t alane = r + 16 * g;
  const uint32_t hp[4] = {pack_rtz(p[0], p[1]), pack_rtz(p[2], p[3]), pack_rtz(p[4], p[5]), pack_rtz(p[6], p[7])};
  img[(kb * HL) * 64 + alane] = make_uint4(hp[0], hp[1], hp[2], hp[3]);  // fp16 inputs convert back exactly
  float s = 0.0f;
  if constexpr (F32A) {
    float res[8];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      res[2 * e] = p[2 * e] - half_lo(hp[e]);
      res[2 * e + 1] = p[2 * e + 1] - half_hi(hp[e]);
    }
    img[(kb * HL + 1) * 64 + alane] =
        make_uint4(pack_rtz(res[0], res[1]), pack_rtz(res[2], res[3]), pack_rtz(res[4], res[5]), pack_rtz(res[6], res[7]));
  }
  s = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
  s += dpp_move<kDppQuadXor1>(s);
  s += dpp_move<kDppQuadXor2>(s);
  uint32_t* const extra = (uint32_t*)(img + kSliceBlocks * HL * 64);
  if (g == 0) {
    const float mean = s * 0.03125f;
    const uint32_t mh = pack_rtz(mean, 0.0f);
    extra[(r + 16 * (kb >> 2)) * 4 + (kb & 3)] = (mh & 0xFFFFu) | (pack_rtz(mean - half_lo(mh), 0.0f) << 16);
  }
  // lanes (row, g' >= 2) of the additive operand stay zero; the rows' inverse scales follow
  if (threadIdx.x < 32 * 4) extra[32 * 4 + threadIdx.x] = 0u;
  if (l == 0) ((float*)extra)[64 * 4 + r] = inv * (FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f);
}

struct TileTail {  // arguments first needed in the epilogue
  const float* dres;
  float* c;
  float* scratch;      // [parts][row groups * R * 16][n] partial results when parts > 1
  uint32_t* counters;  // one arrival counter per (row group, column group), zero between launches
  uint32_t epilogue;   // unary operations on the output (apply_epilogue)
};

constexpr int park_stride(int fmt) { return fmt == MGN_FMT_Q4 ? 8 * 16 + 16 : 8 * 32 + 16; }  // bytes per parked column
// Weight slices in flight per wave ahead of the one in use.  Loads return in issue order and the
// image of phase p + 2 is requested in phase p just before weight slice p + kDepth: waiting for
// that image at the end of phase p + 1 also waits for slice p + kDepth - 1 and everything older.
// With kDepth = 3 that is the slice needed next anyway, so the image never holds the stream back.
constexpr int kDepth = 3;
constexpr int kUnroll = 6;  // phases per loop body: a multiple of kDepth and of the two image register sets

// blockDim.x = 64 * ksc * wnc (at most 8 waves).  Wave w: K split ks = w % ksc, column tile
// slot wn = w / ksc.  In phase p the workgroup holds the images of slices
// (part * nph + p) * ksc + 0..ksc-1 in LDS and wave (ks, wn) multiplies slice ... + ks.
// The image holds gridDim.z * R row tiles of nsp = parts * nph * ksc slices each (rows past m and
// slices past the end of K are zero), so a phase's images are one linear run per row tile.
// CPT: uint4 units of a later phase's images a thread copies while the current one is multiplied.
template <int FMT, bool F32A, int R, int CPT>
__global__ __launch_bounds__(512) void tile_mfma_kernel(const uint4* __restrict__ image, const void* __restrict__ meta_arg,
                                                         const void* __restrict__ quants_arg, uint32_t m, uint32_t kdim,
                                                         uint32_t n, uint32_t wnc, uint32_t ksc, uint32_t nph, uint32_t parts,
                                                         uint32_t nslices, TileTail tail) {
  constexpr uint32_t HL = F32A ? 2 : 1;
  constexpr uint32_t UNITS = image_units(F32A);
  constexpr float kOpScale = FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f;  // 2^20, 2^24
  constexpr int QB = FMT == MGN_FMT_Q4 ? 16 : 32;  // quant bytes per block
  constexpr int MB = FMT == MGN_FMT_Q4 ? 4 : 2;    // scale bytes per block
  constexpr int NLQ = QB / 8;                      // 16-byte quant loads per lane per slice (16 columns x 8 blocks)
  constexpr int NLM = FMT == MGN_FMT_Q4 ? 2 : 1;   // 16-byte scale loads per lane per slice
  constexpr int kStride = park_stride(FMT);
  constexpr uint32_t LPC = QB / 2;   // lanes per column in one quant load
  constexpr uint32_t CPL = 64 / LPC;  // columns per quant load
  extern __shared__ uint4 lds4[];
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wn = wave / ksc, ks = wave - wn * ksc;
  const uint32_t nthreads = 64 * ksc * wnc;
  const uint32_t c = lane & 15, g = lane >> 4;
  const uint32_t part = blockIdx.x, cg = blockIdx.y, rg = blockIdx.z;
  const uint32_t bpc = kdim / 32;
  const uint32_t col_tile = cg * wnc + wn;
  const uint32_t col = col_tile * 16 + c;
  const bool col_ok = col < n;
  const uint32_t nsp = parts * nph * ksc;

  const uint32_t buf_units = ksc * R * UNITS;  // one phase's images
  uint4* const imgbuf = lds4;                  // [2][R][ksc][UNITS]
  uint8_t* const park = (uint8_t*)(lds4 + 2 * buf_units) + wave * (16 * kStride);

  // ---- image copy ----
  // Unit u of a phase: row tile rr = u / (ksc * UNITS), then ksc * UNITS consecutive units of the
  // image (the phase's ksc slices lie side by side).  A thread's units keep their place from phase
  // to phase: only the uniform base moves on.
  // The image of phase q is loaded during phase q - 2 and written to LDS at the end of phase
  // q - 1, from register set q & 1.  (Loads return in issue order: waiting for an image that was
  // requested right behind a weight slice would wait for that slice, long before it is needed.)
  u32x4_t cp[2][CPT];  // (native vectors: arrays of the HIP struct type are not always promoted to registers)
  uint32_t cp_off[CPT];
#pragma unroll
  for (int j = 0; j < CPT; j++) {
    const uint32_t u = min(tid + j * nthreads, buf_units - 1);
    const uint32_t rr = u / (ksc * UNITS), off = u - rr * (ksc * UNITS);
    cp_off[j] = (rr * nsp * UNITS + off) * 16;
  }
  const uint8_t* const img0 = (const uint8_t*)(image + ((size_t)rg * R * nsp + (size_t)part * nph * ksc) * UNITS);
  auto copy_load = [&](int set, uint32_t p) {
    const uint8_t* const base = img0 + (size_t)p * ksc * UNITS * 16;  // uniform
#pragma unroll
    for (int j = 0; j < CPT; j++) cp[set][j] = *(const u32x4_t*)(base + cp_off[j]);
  };
  auto copy_store = [&](int set, uint32_t buf) {
#pragma unroll
    for (int j = 0; j < CPT; j++) {
      const uint32_t u = tid + j * nthreads;
      if (u < buf_units) *(u32x4_t*)(imgbuf + buf * buf_units + u) = cp[set][j];
    }
  };

  // ---- weight slices: 16 columns x 8 blocks per wave and phase ----
  // Quants: whole 128-byte (Q8: 256-byte) runs of a column's blocks, 8 (4) columns per load
  // instruction.  Scale words: the lane's own column, all 8 blocks (the four lanes of a column
  // load the same words).  A lane's offsets are fixed (a column past the end re-reads the last
  // one); the slice only moves the uniform base.  Slices past the end of K re-read the last one.
  u32x4_t wq[kDepth][NLQ];
  u32x4_t wm[kDepth][NLM];
  uint32_t q_off[NLQ];
#pragma unroll
  for (int j = 0; j < NLQ; j++) q_off[j] = min(col_tile * 16 + CPL * j + lane / LPC, n - 1) * bpc * QB + (lane % LPC) * 16;
  const uint32_t m_off = min(col, n - 1) * bpc * MB;
  auto fetch = [&](int slot, uint32_t p) {
    const uint32_t kb0 = min((part * nph + p) * ksc + ks, nslices - 1) * kSliceBlocks;  // uniform
    const uint8_t* const qb = (const uint8_t*)quants_arg + (size_t)kb0 * QB;
    const uint8_t* const mb = (const uint8_t*)meta_arg + (size_t)kb0 * MB;
#pragma unroll
    for (int j = 0; j < NLQ; j++) wq[slot][j] = __builtin_nontemporal_load((const u32x4_t*)(qb + q_off[j]));
    typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
#pragma unroll
    for (int j = 0; j < NLM; j++) {
      const u32x4_a2 v = __builtin_nontemporal_load((const u32x4_a2*)(mb + m_off) + j);
      wm[slot][j] = u32x4_t{v.x, v.y, v.z, v.w};
    }
  };

  floatx4 acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

  // prologue: first images into LDS, first weight slices on their way
  copy_load(0, 0);
#pragma unroll
  for (int d = 0; d < kDepth; d++) fetch(d, min((uint32_t)d, nph - 1));
  copy_load(1, min(1u, nph - 1));
  copy_store(0, 0);
  lds_barrier();

  const uint8_t* const park_rd = park + c * kStride + g * (QB / 4);  // this lane's piece of block 0 of its column
  // The phase loop runs in groups of kUnroll with every load, LDS store and barrier unconditional
  // (loads past the last phase re-read the last one's data): with no branch that rejoins in front
  // of a memory operation the compiler's wait counts are exact, and a wave only ever waits for the
  // slice it is about to use.
  for (uint32_t p0 = 0; p0 < nph; p0 += kUnroll) {
#pragma unroll
    for (int ph = 0; ph < kUnroll; ph++) {
      const uint32_t p = p0 + ph;
      constexpr int kSlots = kDepth;
      const int slot = ph % kSlots;
      if (p >= nph) break;  // uniform: leaves the loop, so no path joins back in front of a memory operation
      {
        copy_load(ph & 1, min(p + 2, nph - 1));
        const uint32_t sl_raw = (part * nph + p) * ksc + ks;
        const bool live = p < nph && sl_raw < nslices && col_tile * 16 < n;  // uniform over the wave
        // park this slice's quants, then refill the slot
#pragma unroll
        for (int j = 0; j < NLQ; j++) *(u32x4_t*)(park + (CPL * j + lane / LPC) * kStride + (lane % LPC) * 16) = wq[slot][j];
        uint32_t mw[8];
        if constexpr (FMT == MGN_FMT_Q4) {
          mw[0] = wm[slot][0].x, mw[1] = wm[slot][0].y, mw[2] = wm[slot][0].z, mw[3] = wm[slot][0].w;
          mw[4] = wm[slot][1].x, mw[5] = wm[slot][1].y, mw[6] = wm[slot][1].z, mw[7] = wm[slot][1].w;
        } else {
          const uint32_t v[4] = {wm[slot][0].x, wm[slot][0].y, wm[slot][0].z, wm[slot][0].w};
#pragma unroll
          for (int e = 0; e < 4; e++) mw[2 * e] = v[e] & 0xFFFFu, mw[2 * e + 1] = v[e] >> 16;
        }
        __builtin_amdgcn_sched_barrier(0);
        fetch(slot, min(p + kDepth, nph - 1));
        __builtin_amdgcn_sched_barrier(0);
        if (live) {
          // blocks past the end of K (last slice of a K that is no multiple of 256) count for nothing
          const uint32_t kb0 = sl_raw * kSliceBlocks;
          if (kb0 + kSliceBlocks > bpc) {
#pragma unroll
            for (int s = 0; s < 8; s++) mw[s] = kb0 + s < bpc ? mw[s] : 0u;
          }
          const uint8_t* const ib = (const uint8_t*)(imgbuf + (p & 1) * buf_units + ks * UNITS + lane);
          constexpr uint32_t kRowTile = 16;  // bytes per uint4 unit
          const uint32_t rstride = ksc * UNITS * kRowTile;  // bytes between the row tiles of a buffer
          // Software pipeline over the 8 blocks: LDS reads two blocks ahead, unpack and MFMAs one
          // block ahead of the scaling FMAs that consume the previous block's products.
          uint32_t bq[8][FMT == MGN_FMT_Q4 ? 1 : 2];
          u32x4_t aop[8][R][HL];
          floatx4 dsum[2][R];
          floatx4 P[R];
#pragma unroll
          for (int r = 0; r < R; r++) P[r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
          auto lds_reads = [&](int s) {
            if constexpr (FMT == MGN_FMT_Q4) {
              bq[s][0] = *(const uint32_t*)(park_rd + s * 16);
            } else {
              const uint2 q = *(const uint2*)(park_rd + s * 32);
              bq[s][0] = q.x, bq[s][1] = q.y;
            }
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
              for (uint32_t h = 0; h < HL; h++) aop[s][r][h] = *(const u32x4_t*)(ib + r * rstride + (s * HL + h) * 64 * 16);
          };
          auto mfmas = [&](int s) {
            half8 bop;
            if constexpr (FMT == MGN_FMT_Q4) bop = nibbles_to_operand(bq[s][0]);
            else bop = bytes_to_operand(bq[s][0], bq[s][1]);
#pragma unroll
            for (int r = 0; r < R; r++) {
              floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, aop[s][r][0]), bop,
                                                                 floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
              if constexpr (F32A) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, aop[s][r][HL - 1]), bop, d, 0, 0, 0);
              dsum[s & 1][r] = d;
            }
          };
          auto scale = [&](int s) {
            const float dq = half_bits_to_float(mw[s] & 0xFFFFu);
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
              for (int i = 0; i < 4; i++) P[r][i] = __fmaf_rn(dq, dsum[s & 1][r][i], P[r][i]);
          };
          lds_reads(0);
          lds_reads(1);
          __builtin_amdgcn_sched_barrier(0);
          mfmas(0);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int s = 0; s < 8; s++) {
            if (s + 2 < 8) lds_reads(s + 2);
            __builtin_amdgcn_sched_barrier(0);
            if (s + 1 < 8) mfmas(s + 1);
            __builtin_amdgcn_sched_barrier(0);
            scale(s);
            __builtin_amdgcn_sched_barrier(0);
          }
          // additive part of the slice's 8 blocks: mean(x) * m (Q4) or mean(x) * scale (Q8), times 32
          // (the means) and, for Q8, times -128 (the byte bias); 2^-20 (2^-24) like the quant sums
          uint32_t bw[4];
          const uint32_t upper = 0u - (g & 1u);  // all ones in the lanes that take blocks 4..7
#pragma unroll
          for (int j = 0; j < 4; j++) {
            // (bit arithmetic, not a select between array elements: that would be turned into an
            // indexed load from a stack copy of the array)
            const uint32_t w = mw[j] ^ ((mw[j] ^ mw[4 + j]) & upper);
            bw[j] = FMT == MGN_FMT_Q4 ? __builtin_amdgcn_perm(w, w, 0x07060706u) : __builtin_amdgcn_perm(w, w, 0x05040504u);
          }
          const half8 bm = as_half8(bw[0], bw[1], bw[2], bw[3]);
          constexpr float kAdd = (FMT == MGN_FMT_Q4 ? 32.0f : -4096.0f) / kOpScale;
#pragma unroll
          for (int r = 0; r < R; r++) {
            const uint8_t* const ir = ib + r * rstride + 8 * HL * 64 * 16;
            const floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, *(const u32x4_t*)ir), bm,
                                                                     floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            if constexpr (F32A) {
              // the rows' inverse slice scales (times 2^20 or 2^24: the operand scale of the quants)
              const float4 inv = *(const float4*)(ir - lane * 16 + 64 * 16 + g * 16);
              acc[r][0] = __fmaf_rn(__fmaf_rn(kAdd, d[0], P[r][0]), inv.x, acc[r][0]);
              acc[r][1] = __fmaf_rn(__fmaf_rn(kAdd, d[1], P[r][1]), inv.y, acc[r][1]);
              acc[r][2] = __fmaf_rn(__fmaf_rn(kAdd, d[2], P[r][2]), inv.z, acc[r][2]);
              acc[r][3] = __fmaf_rn(__fmaf_rn(kAdd, d[3], P[r][3]), inv.w, acc[r][3]);
            } else {
#pragma unroll
              for (int i = 0; i < 4; i++) acc[r][i] += __fmaf_rn(kAdd, d[i], P[r][i]);
            }
          }
        }
        copy_store((ph + 1) & 1, (p + 1) & 1);  // that LDS buffer was last read before the previous barrier
        lds_barrier();
      }
    }
  }
  if constexpr (!F32A) {
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] *= kOpScale;
  }

  // ---- combine the K splits of the workgroup (fixed order) ----
  float* const red = (float*)lds4;  // reused: [wn][ks - 1][R][4][64]
  if (ksc > 1) {
    if (ks > 0) {
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int i = 0; i < 4; i++) red[(((wn * (ksc - 1) + ks - 1) * R + r) * 4 + i) * 64 + lane] = acc[r][i];
    }
    lds_barrier();
    if (ks == 0) {
      for (uint32_t s = 1; s < ksc; s++)
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
          for (int i = 0; i < 4; i++) acc[r][i] += red[(((wn * (ksc - 1) + s - 1) * R + r) * 4 + i) * 64 + lane];
    }
  }
  const bool writer = ks == 0 && col_ok && col_tile * 16 < n;
  const uint32_t row0 = rg * R * 16;

  if (parts > 1) {
    // ---- K parts of other workgroups: the last one to arrive adds them up in part order ----
    // Each XCD has its own L2, so partial tiles travel as device-scope relaxed atomics:
    // write-through stores, complete (in memory) once acknowledged, and L2-coherent loads.
    const size_t plane = (size_t)gridDim.z * R * 16 * n;  // floats per part
    if (writer) {
      float* const mine = tail.scratch + (size_t)part * plane + (size_t)row0 * n + col;
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          __hip_atomic_store(mine + (size_t)(r * 16 + 4 * g + i) * n, acc[r][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // every wave waits until its write-through stores have been acknowledged, i.e. have
    // reached memory; the barrier then orders all of them before the count
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t* const flag = (uint32_t*)lds4 + wnc * (ksc - 1) * R * 4 * 64;  // behind the K-split sums
    if (tid == 0) {
      uint32_t* const ctr = tail.counters + rg * gridDim.y + cg;
      const uint32_t seen = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = seen == parts - 1;
      if (last) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
      *flag = last ? 1u : 0u;
    }
    __syncthreads();
    if (*flag == 0u) return;
    if (writer) {
      const float* const base = tail.scratch + (size_t)row0 * n + col;
#pragma unroll
      for (int r = 0; r < R; r++) acc[r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
      for (uint32_t pp = 0; pp < parts; pp++) {
        float t[R][4];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
          for (int i = 0; i < 4; i++)
            t[r][i] = __hip_atomic_load(base + pp * plane + (size_t)(r * 16 + 4 * g + i) * n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
          for (int i = 0; i < 4; i++) acc[r][i] += t[r][i];
      }
    }
  }
  if (writer) {
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t row = row0 + r * 16 + 4 * g + i;
        if (row < m) {
          const size_t o = (size_t)row * n + col;
          tail.c[o] = apply_epilogue(tail.dres ? acc[r][i] + tail.dres[o] : acc[r][i], tail.epilogue);
        }
      }
  }
}

struct TilePlan {
  uint32_t r, wnc, ksc, nph, parts, colgroups, rowgroups, cpt, nslices;
  uint32_t nsp;  // slices per row tile in the image: parts * nph * ksc >= nslices
  bool f32a;
  size_t lds, partial_bytes, image_bytes;
};

size_t tile_lds_bytes(int fmt, bool f32a, uint32_t r, uint32_t wnc, uint32_t ksc) {
  const size_t img = (size_t)2 * ksc * r * image_units(f32a) * 16;
  const size_t parkb = (size_t)ksc * wnc * 16 * park_stride(fmt);
  const size_t red = (size_t)wnc * (ksc - 1) * r * 4 * 64 * 4;
  return std::max(img + parkb, red + 64);
}

// Picks rows per workgroup, the workgroup shape and the K split.  Model: a workgroup's time is the
// largest of its share of the weight stream (the chip's HBM rate split over the workgroups that
// run together), the images it copies out of L2 and its vector-ALU work; a launch takes `rounds`
// of those; K parts add the hand-over through memory.
bool plan_tile(const LaunchArgs& x, TilePlan* out) {
  const bool f32a = !x.a_is_f16;
  const int fmt = x.w.fmt;
  const uint32_t bpc = x.w.k / 32, n_tiles = (x.w.n + 15) / 16;
  if (x.m == 0 || bpc == 0) return false;
  if ((uint64_t)x.w.n * bpc * 32 >= (1ull << 32)) return false;  // a lane's weight offsets are 32-bit
  const uint32_t nslices = (bpc + kSliceBlocks - 1) / kSliceBlocks;
  const double blockbytes = fmt == MGN_FMT_Q4 ? 20.0 : 34.0;
  const uint32_t units = image_units(f32a);
  double best = 0;
  TilePlan bp{};
  // (f32 activations: two operands per block and row tile; four row tiles would not fit the registers)
  const uint32_t rmax = x.m <= 16 ? 1 : (x.m <= 32 || f32a) ? 2 : 4;
  for (uint32_t r = rmax; r >= 1; r /= 2) {
    const uint32_t rowgroups = (x.m + 16 * r - 1) / (16 * r);
    if (rowgroups > 65535) continue;
    for (uint32_t ksc = 1; ksc <= 4; ksc *= 2) {
      for (uint32_t wnc = 8 / ksc; wnc >= 1; wnc--) {
        if (wnc > n_tiles && wnc > 4) continue;  // waves without a column tile only help to copy the images
        const uint32_t waves = ksc * wnc;
        const size_t lds = tile_lds_bytes(fmt, f32a, r, wnc, ksc);
        if (lds > 160 * 1024) continue;
        const uint32_t cpt = (ksc * r * units + 64 * waves - 1) / (64 * waves);
        if (cpt > 6 || (cpt > 4 && r == 4)) continue;  // two image sets must stay in registers
        if (waves > 8) continue;  // 256 registers per lane: the prefetched weight slices and two image sets need them
        const uint32_t colgroups = (n_tiles + wnc - 1) / wnc;
        if (colgroups > 65535) continue;
        const uint32_t phases = (nslices + ksc - 1) / ksc;
        for (uint32_t parts = 1; parts <= phases && parts <= 16; parts++) {
          const uint32_t nph = (phases + parts - 1) / parts;
          if ((phases + nph - 1) / nph != parts) continue;  // same split, already seen
          const size_t partial = parts > 1 ? (size_t)parts * rowgroups * r * 16 * x.w.n * 4 : 0;
          if (partial > x.scratch_bytes) break;
          if (parts > 1 && (uint64_t)rowgroups * colgroups > x.n_counters) break;
          const uint64_t wgs = (uint64_t)rowgroups * colgroups * parts;
          const uint32_t per_cu = std::max<uint32_t>(1, std::min<uint32_t>((uint32_t)(160 * 1024 / lds), 16 / waves));
          const double slots = (double)x.num_cus * per_cu;
          const double rounds = std::ceil((double)wgs / slots);
          const double together = std::min<double>((double)wgs, slots);
          // seconds, roughly: HBM 5.5 TB/s over the workgroups running together; 100 GB/s of image
          // copies per CU; vector ALU at 2 GHz with waves / 4 waves per SIMD
          const double wbytes = (double)nph * ksc * kSliceBlocks * std::min(wnc, n_tiles) * 16 * blockbytes;
          const double t_hbm = wbytes * together / 5.5e12;
          const double ibytes = (double)nph * ksc * r * units * 16;
          const double t_img = ibytes * per_cu / 100e9;
          const double instr = 70.0 + 8.0 * (9.0 + r * ((f32a ? 2.0 : 1.0) + 4.5));
          const double t_alu = nph * instr * 4.0 * std::ceil(waves * per_cu / 4.0) / 2.0e9;
          double t = rounds * (std::max(t_hbm, std::max(t_img, t_alu)) + 0.6e-6);
          if (parts > 1) t += 2.5e-6 + (double)parts * r * 16 * std::min(wnc, n_tiles) * 16 * 4 / 50e9;
          if (waves < 4) t *= 1.3;  // few waves hide little latency
          // a lone workgroup on a CU runs its phases in lockstep (load, multiply, store, barrier);
          // two or more drift apart and overlap them (measured: 22.5 -> 17.7 us at M = 16, 4096 x 14336)
          if (per_cu < 2 || wgs < 2 * (uint64_t)x.num_cus) t *= 1.3;
          if (best == 0 || t < best) {
            best = t;
            bp.r = r, bp.wnc = wnc, bp.ksc = ksc, bp.nph = nph, bp.parts = parts, bp.colgroups = colgroups;
            bp.rowgroups = rowgroups, bp.cpt = cpt, bp.nslices = nslices, bp.f32a = f32a;
            bp.lds = lds, bp.partial_bytes = partial;
            bp.nsp = parts * nph * ksc;
            bp.image_bytes = (size_t)rowgroups * r * bp.nsp * units * 16;
          }
        }
      }
    }
  }
  if (best == 0) return false;
  *out = bp;
  return true;
}

template <int FMT, bool F32A, int R, int CPT>
int launch_cpt(ihipStream_t* s, const LaunchArgs& x, const TilePlan& p, uint4* image) {
  auto kern = tile_mfma_kernel<FMT, F32A, R, CPT>;
  static std::atomic<uint64_t> big_lds_done{0};
  if (p.lds > 64 * 1024)
    if (int e = enable_big_lds(kern, x.device, big_lds_done)) return e;
  const TileTail tail{x.d, x.c, (float*)x.scratch, x.counters, x.epilogue};
  hipLaunchKernelGGL(kern, dim3(p.parts, p.colgroups, p.rowgroups), dim3(64 * p.ksc * p.wnc), p.lds, s, image, x.w.meta, x.w.quants,
                     x.m, x.w.k, x.w.n, p.wnc, p.ksc, p.nph, p.parts, p.nslices, tail);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

template <int FMT, bool F32A, int R>
int launch_r(ihipStream_t* s, const LaunchArgs& x, const TilePlan& p, uint4* image) {
  switch (p.cpt) {
    case 1: return launch_cpt<FMT, F32A, R, 1>(s, x, p, image);
    case 2: return launch_cpt<FMT, F32A, R, 2>(s, x, p, image);
    case 3: return launch_cpt<FMT, F32A, R, 3>(s, x, p, image);
    case 4: return launch_cpt<FMT, F32A, R, 4>(s, x, p, image);
    case 5:
    case 6: return launch_cpt<FMT, F32A, R, 6>(s, x, p, image);
    default: return (int)hipErrorInvalidValue;
  }
}

template <int FMT, bool F32A>
int launch_fa(ihipStream_t* s, const LaunchArgs& x, const TilePlan& p) {
  // the image lives behind the partial sums in the workspace
  uint4* const image = (uint4*)((char*)x.scratch + ((p.partial_bytes + 255) & ~(size_t)255));
  const uint32_t a_stride = x.w.k;
  hipLaunchKernelGGL((image_kernel<FMT, F32A>), dim3(p.rowgroups * p.r * p.nsp), dim3(512), 0, s, x.a, image, x.m, x.w.k,
                     p.nsp, a_stride);
  MGN_HIP_LAUNCH_CHECK();
  return p.r == 1 ? launch_r<FMT, F32A, 1>(s, x, p, image) : p.r == 2 ? launch_r<FMT, F32A, 2>(s, x, p, image)
                                                                      : launch_r<FMT, F32A, 4>(s, x, p, image);
}

size_t tile_workspace_bytes(const TilePlan& p) { return ((p.partial_bytes + 255) & ~(size_t)255) + p.image_bytes; }

}  // namespace

bool tile_mfma_supported(const LaunchArgs& x) {
  TilePlan p;
  if (!plan_tile(x, &p)) return false;
  return tile_workspace_bytes(p) <= x.scratch_bytes;
}

bool describe_tile_mfma(const LaunchArgs& x, mgn_plan_info* out) {
  TilePlan p;
  if (!plan_tile(x, &p) || tile_workspace_bytes(p) > x.scratch_bytes) return false;
  out->route = MGN_ROUTE_TILE_MFMA;
  out->grid[0] = p.parts, out->grid[1] = p.colgroups, out->grid[2] = p.rowgroups;
  out->threads = 64 * p.ksc * p.wnc;
  out->lds_bytes = (uint32_t)p.lds;
  out->waves_n = p.wnc, out->k_splits = p.ksc, out->k_parts = p.parts, out->steps = p.nph;
  out->quads_per_wave = 0, out->full_steps = 0, out->tail_blocks = 0;
  out->workspace_bytes = tile_workspace_bytes(p);
  return true;
}

int launch_matmul_tile_mfma(ihipStream_t* s, const LaunchArgs& x) {
  TilePlan p;
  if (!plan_tile(x, &p) || tile_workspace_bytes(p) > x.scratch_bytes) return (int)hipErrorInvalidValue;
  if (x.w.fmt == MGN_FMT_Q4) return x.a_is_f16 ? launch_fa<MGN_FMT_Q4, false>(s, x, p) : launch_fa<MGN_FMT_Q4, true>(s, x, p);
  return x.a_is_f16 ? launch_fa<MGN_FMT_Q8, false>(s, x, p) : launch_fa<MGN_FMT_Q8, true>(s, x, p);
}

}  // namespace mgn
