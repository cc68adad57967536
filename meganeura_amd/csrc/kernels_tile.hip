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
//   B operand: dword g of the block's nibbles, masked into the mantissa bits of fp16 subnormals
//     (n * 2^-20, exact; with f32 activations the even nibbles stay at n * 2^-24 and their
//     activations are stored times 16: two shifts fewer per dword; Q8: the block's bytes
//     8g..8g+7 as (q + 128) * 2^-24 in bits 0-7).
//   A operand: the activations, converted into an "image" in the instruction's own lane order.
//     f32 activations are scaled per (row, 256-element K slice) by a power of two and split
//     hi + lo into two fp16 operands that are multiplied into the same accumulator: 22
//     significant bits relative to the slice's largest magnitude (each half is cut, not rounded,
//     to 11), products with the quants exact on those, f32 accumulation rounds; any magnitude
//     below 2^100 is representable (beyond, the slice's inverse scale is a NaN and the row comes
//     out non-finite).  fp16 activations are used as they are.
//   Per block: D = sum n x on the matrix cores, then P += d * D on the vector ALU (4 FMAs per
//     lane).  The format's additive part (m * sum(x) for Q4, -128 * scale * sum(x) for Q8's byte
//     bias) is one more MFMA per slice of 8 blocks: its A operand holds the blocks' mean
//     activations (hi, lo), its B operand the blocks' m (or scale), exact fp16 values times a
//     power of two chosen per weight (AddLift).  (fp16 activations: two MFMAs, hi and lo apart,
//     because lo is kept times 2^11; see convert_task.)
//     With f32 activations a slice's P is multiplied by the rows' inverse power-of-two scales
//     before it is added to the accumulators.
//
// Two kernels share this arithmetic.
//   tile_mfma_kernel (any M): image_kernel converts the activations ONCE per call into images
//     in the workspace, which every workgroup copies into LDS slice by slice, double-buffered.
//     The quants travel from memory as whole 128/256-byte runs of a column's blocks, are parked
//     in a wave-private LDS slice and read back one dword (Q8: two) per lane and block.
//     grid = (K parts, column groups, row groups): a workgroup owns wnc column tiles of 16
//     columns, R row tiles of 16 rows and a range of K slices; ksc waves share a column tile and
//     take the slices of a phase side by side (their sums meet in LDS, in a fixed order).
//   tile_resident_kernel (row groups of 16 or 32 rows): every workgroup converts its own rows
//     of its K part and keeps the images in LDS; no second launch, no image traffic (see there).
// With too few tiles to fill the chip K is also cut into parts for different workgroups, whose
// partial tiles the last one to finish adds in part order (deterministic).
#include <algorithm>
#include <cmath>
#include <type_traits>

#include "kernels_operand.hip.h"

namespace mgn {
namespace {

// What the additive MFMA's result (block means times m, or times the Q8 scale) is multiplied by:
// 32 for the means and, for Q8, -128 for the byte bias, over the quants' operand scale.
template <int FMT>
constexpr float additive_constant() { return FMT == MGN_FMT_Q4 ? 32.0f / 1048576.0f : -4096.0f / 16777216.0f; }

// The additive MFMA's B operand holds the blocks' own constants (m, or the Q8 scale) as fp16, and
// the matrix cores lose low bits of products whose operand is an fp16 subnormal (Q8 scales below
// 2^-14: 2 * 10^-4 of a typical output, measured).  The constants are therefore multiplied by a
// power of two first, the largest that keeps the weight's largest constant finite (exact, one
// packed multiplication per dword), and the instruction's result by its inverse.
struct AddLift {
  uint32_t up2;  // 2^s twice, as fp16
  float down;    // 2^-s
  __device__ __forceinline__ uint32_t up(uint32_t pair) const {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, pair) * __builtin_bit_cast(half2_t, up2));
  }
};

// max over aligned groups of 32 consecutive lanes (every lane ends with the group's maximum)
__device__ __forceinline__ float group_max32(float v) {
  v = fmaxf(v, dpp_move<kDppQuadXor1>(v));
  v = fmaxf(v, dpp_move<kDppQuadXor2>(v));
  v = fmaxf(v, dpp_move<kDppRowHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppRowMirror>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return v;
}

// ---- the activation image ----
// One image per (row tile of 16 rows, K slice of 8 blocks = 256 elements), in uint4 units:
//   [(kb * HL + h) * 64 + image_slot(row, g, kb)]
//                                A operand of block kb, h = 0 high halves, h = 1 low halves (f32
//                                activations only: HL = 2), for A lane = row + 16 * g.  The slot is
//                                the lane with its row rotated by 2 g + 8 (kb % 2): the eight lanes
//                                that write together during the conversion (one row, two blocks, four
//                                g) then fall into different LDS banks, and so do the readers'.
//   [8 * HL * 64 + lane]         A operand of the slice's additive MFMA: lanes (row, g' < 2) hold
//                                (mean_hi | mean_lo << 16) of blocks 4g'..4g'+3; f32 activations: the
//                                rest is zero; fp16 activations: the rest is not written, mean_lo is
//                                the part of the mean below mean_hi TIMES 2^11, and the readers take
//                                the two halves apart (mean_operands)
//   [8 * HL * 64 + 64 + 0..15]   (as float) f32 activations only: the rows' inverse scales times the
//                                quants' operand scale (2^20 for Q4, 2^24 for Q8)
// The element order inside an operand follows the B side: Q4 pairs k with k + 4, Q8 is natural.
// Q4 with f32 activations: the even elements are stored times 16 (see nibbles_to_operand) and the
// slice scale aims at 2^7 instead of 2^11 to leave room for that.
constexpr uint32_t kSliceBlocks = 8;
__device__ __forceinline__ uint32_t image_slot(uint32_t row, uint32_t g, uint32_t kb_parity) {
  return ((row + 2 * g + 8 * kb_parity) & 15u) + 16 * g;
}
constexpr uint32_t image_units(bool f32a) { return kSliceBlocks * (f32a ? 2u : 1u) * 64u + 64u + 16u; }

// Eight consecutive activations of a row as they come from memory: 8 f32 words or 4 words of fp16 pairs.
template <bool F32A>
struct TaskWords {
  uint32_t w[F32A ? 8 : 4];
};

template <bool F32A>
__device__ __forceinline__ void load_task(const void* __restrict__ a, size_t elem, TaskWords<F32A>& x) {
  if constexpr (F32A) {
    const uint4* src = (const uint4*)((const float*)a + elem);
    const uint4 v0 = src[0], v1 = src[1];
    x.w[0] = v0.x, x.w[1] = v0.y, x.w[2] = v0.z, x.w[3] = v0.w, x.w[4] = v1.x, x.w[5] = v1.y, x.w[6] = v1.z, x.w[7] = v1.w;
  } else {
    const uint4 v = *(const uint4*)((const _Float16*)a + elem);
    x.w[0] = v.x, x.w[1] = v.y, x.w[2] = v.z, x.w[3] = v.w;
  }
}

// One task of the conversion: half-wave lane l = kb * 4 + g turns the 8 activations k0 .. k0 + 7
// (k0 = 256 slice + 32 kb + 8 g) of row `row` into its piece of the image `img` of that (row tile,
// slice); r = row % 16.  All 32 lanes of the half-wave (one row of one slice) must call it together.
template <int FMT, bool F32A>
__device__ __forceinline__ void convert_task(const TaskWords<F32A>& xin, bool ok, uint4* __restrict__ img, uint32_t r, uint32_t l) {
  constexpr uint32_t HL = F32A ? 2 : 1;
  const uint32_t kb = l >> 2, g = l & 3;
  const uint32_t alane = image_slot(r, g, kb & 1);
  float s, inv = 1.0f;
  if constexpr (F32A) {
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] = ok ? __builtin_bit_cast(float, xin.w[e]) : 0.0f;
    // NaN never wins fmaxf; an infinity does and switches scaling off
    float am = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                     fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
    am = group_max32(am);
    constexpr bool kSplit = FMT == MGN_FMT_Q4;
    const float scale = slice_scale<kSplit ? 7 : 11>(am, &inv);
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] *= (kSplit && e % 2 == 0) ? scale * 16.0f : scale;
    float p[8];
    if constexpr (FMT == MGN_FMT_Q4) {
      p[0] = x[0], p[1] = x[4], p[2] = x[1], p[3] = x[5], p[4] = x[2], p[5] = x[6], p[6] = x[3], p[7] = x[7];
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) p[e] = x[e];
    }
    const uint32_t hp[4] = {pack_rtz(p[0], p[1]), pack_rtz(p[2], p[3]), pack_rtz(p[4], p[5]), pack_rtz(p[6], p[7])};
    img[(kb * HL) * 64 + alane] = make_uint4(hp[0], hp[1], hp[2], hp[3]);
    float res[8];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      res[2 * e] = p[2 * e] - half_lo(hp[e]);
      res[2 * e + 1] = p[2 * e + 1] - half_hi(hp[e]);
    }
    img[(kb * HL + 1) * 64 + alane] =
        make_uint4(pack_rtz(res[0], res[1]), pack_rtz(res[2], res[3]), pack_rtz(res[4], res[5]), pack_rtz(res[6], res[7]));
    if constexpr (FMT == MGN_FMT_Q4) s = ((x[0] + x[2]) + (x[4] + x[6])) * 0.0625f + ((x[1] + x[3]) + (x[5] + x[7]));
    else s = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
  } else {
    // fp16 activations are operands as they are: only their order changes (Q4 pairs k with k + 4)
    const uint32_t v[4] = {ok ? xin.w[0] : 0u, ok ? xin.w[1] : 0u, ok ? xin.w[2] : 0u, ok ? xin.w[3] : 0u};
    if constexpr (FMT == MGN_FMT_Q4) {
      img[kb * 64 + alane] = make_uint4(__builtin_amdgcn_perm(v[2], v[0], 0x05040100u), __builtin_amdgcn_perm(v[2], v[0], 0x07060302u),
                                        __builtin_amdgcn_perm(v[3], v[1], 0x05040100u), __builtin_amdgcn_perm(v[3], v[1], 0x07060302u));
    } else {
      img[kb * 64 + alane] = make_uint4(v[0], v[1], v[2], v[3]);
    }
    const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v[0]), ones, 0.0f, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v[1]), ones, s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v[2]), ones, s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v[3]), ones, s, false);
  }
  s += dpp_move<kDppQuadXor1>(s);
  s += dpp_move<kDppQuadXor2>(s);
  uint32_t* const extra = (uint32_t*)(img + kSliceBlocks * HL * 64);
  const float mean = s * 0.03125f;
  const uint32_t mh = pack_rtz(mean, 0.0f);
  if constexpr (!F32A) {
    // A block of fp16 activations sums to at most 2^21, its mean to at most 65504: no scale is
    // needed to keep it in range.  hi is the mean cut to fp16 and lo the rest times 2^11, which fp16
    // holds exactly down to the smallest sums (the rest is a multiple of 2^-29 below 2^-24) and
    // without overflow at the largest; the readers multiply lo's products by 2^-11.  So the
    // conversion needs no maximum over the slice, no scale and no inverse: a permutation and a sum.
    if (g == 0) extra[(r + 16 * (kb >> 2)) * 4 + (kb & 3)] = (mh & 0xFFFFu) | (pack_rtz((mean - half_lo(mh)) * 2048.0f, 0.0f) << 16);
    return;
  }
  if (g == 0) extra[(r + 16 * (kb >> 2)) * 4 + (kb & 3)] = (mh & 0xFFFFu) | (pack_rtz(mean - half_lo(mh), 0.0f) << 16);
  // lanes (row, g' >= 2) of the additive operand stay zero (8 dwords per half-wave lane... 16 rows x 32
  // lanes cover the 128 dwords); the rows' inverse scales, times the quants' operand scale, follow
  if (l < 8) extra[32 * 4 + r * 8 + l] = 0u;
  if (l == 0) ((float*)extra)[64 * 4 + r] = inv * (FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f);
}

// fp16 activations: the two A operands of a row tile's additive MFMAs, mean_hi and mean_lo apart
// (`extra`: the row tile's additive words in the image).  Lanes (row, g' >= 2) have no blocks.
__device__ __forceinline__ void mean_operands(const uint8_t* extra, uint32_t lane, uint32_t g, half8* hi, half8* lo) {
  const u32x4_t w = *(const u32x4_t*)(extra + (lane & 31) * 16);
  const bool has = g < 2;
  *hi = as_half8(has ? w.x & 0xFFFFu : 0u, has ? w.y & 0xFFFFu : 0u, has ? w.z & 0xFFFFu : 0u, has ? w.w & 0xFFFFu : 0u);
  *lo = as_half8(has ? w.x >> 16 : 0u, has ? w.y >> 16 : 0u, has ? w.z >> 16 : 0u, has ? w.w >> 16 : 0u);
}

// grid.x = row tiles * slices; 512 threads: half-wave r (0..15) converts row r of the tile,
// lane l = kb * 4 + g of it the 8 elements k = 32 kb + 8 g .. + 7 of the slice.
template <int FMT, bool F32A>
__global__ __launch_bounds__(512) void image_kernel(const void* __restrict__ a, uint4* __restrict__ image, uint32_t m,
                                                    uint32_t k, uint32_t nslices, uint32_t a_stride) {
  constexpr uint32_t UNITS = image_units(F32A);
  const uint32_t rt = blockIdx.x / nslices, sl = blockIdx.x - rt * nslices;
  const uint32_t r = threadIdx.x >> 5, l = threadIdx.x & 31;
  const uint32_t row = rt * 16 + r, k0 = sl * 256 + l * 8;
  const bool ok = row < m && k0 < k;  // K is a multiple of 32: a task lies inside or outside as a whole
  TaskWords<F32A> x;
  load_task<F32A>(a, ok ? (size_t)row * a_stride + k0 : (size_t)0, x);
  convert_task<FMT, F32A>(x, ok, image + ((size_t)rt * nslices + sl) * UNITS, r, l);
}

// One slice (8 K blocks) of one 16-column tile against R row tiles: the wave's parked quants at
// park_rd (this lane's piece of block 0 of its column), the slice's image at ib (row tile 0, row
// tiles rstride bytes apart), the column's 8 scale words in mw.
template <int FMT, bool F32A, int R>
__device__ __forceinline__ void slice_mac(const uint8_t* park_rd, const uint8_t* ib, uint32_t rstride, const uint32_t (&mw)[8],
                                          uint32_t g, uint32_t lane, AddLift lift, floatx4 (&acc)[R]) {
  constexpr uint32_t HL = F32A ? 2 : 1;
    // Software pipeline over the 8 blocks: LDS reads two blocks ahead, unpack and MFMAs one
    // block ahead of the scaling FMAs that consume the previous block's products.
    const uint32_t slot_off[2] = {image_slot(lane & 15, g, 0) * 16, image_slot(lane & 15, g, 1) * 16};
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
        for (uint32_t h = 0; h < HL; h++) aop[s][r][h] = *(const u32x4_t*)(ib + slot_off[s & 1] + r * rstride + (s * HL + h) * 64 * 16);
    };
    auto mfmas = [&](int s) {
      half8 bop;
      if constexpr (FMT == MGN_FMT_Q4) bop = nibbles_to_operand<F32A>(bq[s][0]);
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
      bw[j] = lift.up(FMT == MGN_FMT_Q4 ? __builtin_amdgcn_perm(w, w, 0x07060706u) : __builtin_amdgcn_perm(w, w, 0x05040504u));
    }
    const half8 bm = as_half8(bw[0], bw[1], bw[2], bw[3]);
    const float kAdd = additive_constant<FMT>() * lift.down;
#pragma unroll
    for (int r = 0; r < R; r++) {
      const uint8_t* const ir = ib + lane * 16 + r * rstride + 8 * HL * 64 * 16;
      if constexpr (F32A) {
        const floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, *(const u32x4_t*)ir), bm,
                                                                 floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        // the rows' inverse slice scales (times 2^20 or 2^24: the operand scale of the quants)
        const float4 inv = *(const float4*)(ir - lane * 16 + 64 * 16 + g * 16);
        acc[r][0] = __fmaf_rn(__fmaf_rn(kAdd, d[0], P[r][0]), inv.x, acc[r][0]);
        acc[r][1] = __fmaf_rn(__fmaf_rn(kAdd, d[1], P[r][1]), inv.y, acc[r][1]);
        acc[r][2] = __fmaf_rn(__fmaf_rn(kAdd, d[2], P[r][2]), inv.z, acc[r][2]);
        acc[r][3] = __fmaf_rn(__fmaf_rn(kAdd, d[3], P[r][3]), inv.w, acc[r][3]);
      } else {
        // the means' hi and lo apart, lo's products times 2^-11 (see convert_task)
        half8 ah, al;
        mean_operands(ir - lane * 16, lane, g, &ah, &al);
        const floatx4 dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bm, floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        const floatx4 dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bm, floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[r][i] += __fmaf_rn(kAdd * (1.0f / 2048.0f), dl[i], __fmaf_rn(kAdd, dh[i], P[r][i]));
      }
    }
  }

struct TileTail {  // arguments first needed in the epilogue
  const float* dres;
  float* c;
  float* scratch;      // partial results when parts > 1 (general kernel: [parts][row groups * R * 16][n])
  uint32_t* counters;  // one arrival counter per (row group, column group), zero between launches
  uint32_t epilogue;   // unary operations on the output (apply_epilogue)
  // the resident kernel's K parts: the counter-free hand-over workspace (kHandoverEmpty between
  // launches), the polls a reading wave makes at most, the word it sets when it gives up
  float* handover;
  uint32_t spin_limit;
  uint32_t* fault_flag;
  uint32_t spread;  // resident kernel: every part adds up a share of the tiles (all workgroups of the launch resident)
  AddLift lift;     // (needed in the walk; rides along here)
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
          const uint8_t* const ib = (const uint8_t*)(imgbuf + (p & 1) * buf_units + ks * UNITS);
          constexpr uint32_t kRowTile = 16;  // bytes per uint4 unit
          const uint32_t rstride = ksc * UNITS * kRowTile;  // bytes between the row tiles of a buffer
          slice_mac<FMT, F32A, R>(park_rd, ib, rstride, mw, g, lane, tail.lift, acc);
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
    if (row0 + R * 16 <= m && !tail.dres && tail.epilogue == 0) {  // (uniform) whole rows, nothing to add or apply
      float* dst = tail.c + (size_t)(row0 + 4 * g) * n + col;
#pragma unroll
      for (int r = 0; r < R; r++) {
#pragma unroll
        for (int i = 0; i < 4; i++) dst[(size_t)i * n] = acc[r][i];
        dst += (size_t)16 * n;
      }
      return;
    }
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

// ---- the images stay in LDS ----
// grid = (K parts, column groups, row groups); 512 threads.  A workgroup converts the activations
// of its K part (its 16 or 32 rows, NSL slices of 256 elements) into images in LDS itself, once; after one barrier
// every wave walks its own Q pairs of column tiles down the part's slices, pair after pair, with
// whole slices of both tiles in flight in registers and no further synchronisation.  The two
// tiles of a pair are multiplied side by side, so every A operand read from LDS serves both (LDS
// bandwidth is what limits a wave that reads each operand for one tile only).
//
// The quants reach the B operand's lane order in one of two ways.
// Through LDS (PARK, whenever a strip per wave fits beside the images): the wave loads whole
// cache lines, 8 (Q8: 16) lanes per column, parks them in its own strip with a padded column
// stride and every lane reads its operands back block by block.
// Without LDS: lane (c, g) loads 16 bytes of column c, and the four lanes of a column exchange
// dwords with the row swap instructions (v_permlane32_swap, v_permlane16_swap: rows of 16 lanes).
//   Q4: lane (c, g) loads block g (then 4 + g) of the slice; a 4x4 transpose over (row, dword)
//       leaves dword g of blocks 0..3 (4..7): the block's elements 8g..8g+7.
//   Q8: load j, lane (c, g): half g / 2 of block 2j + g % 2; swapping (x, z) and (y, w) between
//       the odd and even rows leaves dwords 2g, 2g+1 of block 2j in (x, y), of 2j+1 in (z, w).
// That form touches half a cache line per column and instruction, twice as many lines per byte,
// and the CU's memory pipeline charges per line: M = 16 on 4096 x 14336 takes 14.0 us with it and
// 13.3 us parked (Q8: 18.9 and 16.6 us).  It remains for the plans whose LDS is full (two pairs
// of tiles per wave with f32 activations).
// The scale words are wanted by all four lanes of a column; loading them per lane would ask the
// memory pipeline for every word four times.  Each wave instead loads the words of all its
// columns and slices once, in whole cache lines, parks them in its own LDS strip and reads a
// step's eight words per tile from there.
//
// What a call costs outside the multiplication is what these choices are about: a CU's vector
// memory pipeline takes about three cycles per cache line a load instruction touches, so the
// loads of the prologue (activations, scale words, the first slices) hold the waves for
// thousands of cycles before the first multiplication; quants are requested one slice ahead and
// not before the conversion is under way.  The walk is written out step by step (NSL and Q are compile-time) with
// scheduling fences between its stages: left to itself the compiler moves the loads of later
// steps behind the multiplications and the call takes a third longer.
// K is cut into parts of NSL slices; the parts' partial tiles meet as in the kernel above.
constexpr int kSide = 2;            // column tiles a wave multiplies side by side

// One slice (8 K blocks) of kSide column tiles against R row tiles: the tiles' quants in B operand
// order (q, see above), their 8 scale words (mw), the slice's image at ib (row tile 0, row tiles
// rstride bytes apart).
// PARK: the quants are not in q but parked in LDS, column by column (park_stride apart, tile u
// 16 columns on): park_rd is this lane's piece of block 0 of its column of tile 0.
template <int FMT, bool F32A, int R, bool PARK>
__device__ __forceinline__ void slice_mac_side(const u32x4_t (&q)[kSide][FMT == MGN_FMT_Q4 ? 2 : 4], const uint8_t* park_rd,
                                               const uint32_t (&mw)[kSide][8], const uint8_t* ib, uint32_t rstride, uint32_t g,
                                               uint32_t lane, AddLift lift, floatx4 (&acc)[kSide][R]) {
  constexpr uint32_t HL = F32A ? 2 : 1;
  const uint32_t slot_off[2] = {image_slot(lane & 15, g, 0) * 16, image_slot(lane & 15, g, 1) * 16};
  u32x4_t aop[3][R][HL];
  uint32_t bq[3][kSide][FMT == MGN_FMT_Q4 ? 1 : 2];  // PARK: the lane's quants of a block
  floatx4 dsum[2][kSide][R];
  floatx4 P[kSide][R];
#pragma unroll
  for (int u = 0; u < kSide; u++)
#pragma unroll
    for (int r = 0; r < R; r++) P[u][r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
  auto lds_reads = [&](int s) {
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (uint32_t h = 0; h < HL; h++) aop[s % 3][r][h] = *(const u32x4_t*)(ib + slot_off[s & 1] + r * rstride + (s * HL + h) * 64 * 16);
    if constexpr (PARK) {
#pragma unroll
      for (int u = 0; u < kSide; u++) {
        const uint8_t* src = park_rd + u * 16 * park_stride(FMT) + s * (FMT == MGN_FMT_Q4 ? 16 : 32);
        if constexpr (FMT == MGN_FMT_Q4) {
          bq[s % 3][u][0] = *(const uint32_t*)src;
        } else {
          const uint2 v = *(const uint2*)src;
          bq[s % 3][u][0] = v.x, bq[s % 3][u][1] = v.y;
        }
      }
    }
  };
  auto mfmas = [&](int s) {
#pragma unroll
    for (int u = 0; u < kSide; u++) {
      half8 bop;
      if constexpr (PARK) {
        if constexpr (FMT == MGN_FMT_Q4) bop = nibbles_to_operand<F32A>(bq[s % 3][u][0]);
        else bop = bytes_to_operand(bq[s % 3][u][0], bq[s % 3][u][1]);
      } else if constexpr (FMT == MGN_FMT_Q4) {
        bop = nibbles_to_operand<F32A>(q[u][s >> 2][s & 3]);
      } else {
        bop = (s & 1) ? bytes_to_operand(q[u][s >> 1].z, q[u][s >> 1].w) : bytes_to_operand(q[u][s >> 1].x, q[u][s >> 1].y);
      }
#pragma unroll
      for (int r = 0; r < R; r++) {
        floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, aop[s % 3][r][0]), bop,
                                                           floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        if constexpr (F32A) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, aop[s % 3][r][HL - 1]), bop, d, 0, 0, 0);
        dsum[s & 1][u][r] = d;
      }
    }
  };
  auto scale = [&](int s) {
#pragma unroll
    for (int u = 0; u < kSide; u++) {
      const float dq = half_bits_to_float(mw[u][s] & 0xFFFFu);
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int i = 0; i < 4; i++) P[u][r][i] = __fmaf_rn(dq, dsum[s & 1][u][r][i], P[u][r][i]);
    }
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
  // additive part of the slice's 8 blocks (see slice_mac)
  const uint32_t upper = 0u - (g & 1u);  // all ones in the lanes that take blocks 4..7
  const float kAdd = additive_constant<FMT>() * lift.down;
  half8 bm[kSide];
#pragma unroll
  for (int u = 0; u < kSide; u++) {
    uint32_t bw[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t w = mw[u][j] ^ ((mw[u][j] ^ mw[u][4 + j]) & upper);
      bw[j] = lift.up(FMT == MGN_FMT_Q4 ? __builtin_amdgcn_perm(w, w, 0x07060706u) : __builtin_amdgcn_perm(w, w, 0x05040504u));
    }
    bm[u] = as_half8(bw[0], bw[1], bw[2], bw[3]);
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
    const uint8_t* const ir = ib + lane * 16 + r * rstride + 8 * HL * 64 * 16;
    if constexpr (F32A) {
      const half8 am = __builtin_bit_cast(half8, *(const u32x4_t*)ir);
      // the rows' inverse slice scales (times 2^20 or 2^24)
      const float4 inv = *(const float4*)(ir - lane * 16 + 64 * 16 + g * 16);
#pragma unroll
      for (int u = 0; u < kSide; u++) {
        const floatx4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(am, bm[u], floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        acc[u][r][0] = __fmaf_rn(__fmaf_rn(kAdd, d[0], P[u][r][0]), inv.x, acc[u][r][0]);
        acc[u][r][1] = __fmaf_rn(__fmaf_rn(kAdd, d[1], P[u][r][1]), inv.y, acc[u][r][1]);
        acc[u][r][2] = __fmaf_rn(__fmaf_rn(kAdd, d[2], P[u][r][2]), inv.z, acc[u][r][2]);
        acc[u][r][3] = __fmaf_rn(__fmaf_rn(kAdd, d[3], P[u][r][3]), inv.w, acc[u][r][3]);
      }
    } else {
      // the means' hi and lo apart, lo's products times 2^-11 (see convert_task)
      half8 ah, al;
      mean_operands(ir - lane * 16, lane, g, &ah, &al);
#pragma unroll
      for (int u = 0; u < kSide; u++) {
        const floatx4 dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bm[u], floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        const floatx4 dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bm[u], floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[u][r][i] += __fmaf_rn(kAdd * (1.0f / 2048.0f), dl[i], __fmaf_rn(kAdd, dh[i], P[u][r][i]));
      }
    }
  }
}

// Slices of a part: what fits in LDS beside the waves' scale words (f32 activations in row groups
// of 16, fp16 activations in row groups of 16 or 32).
constexpr int resident_slices(bool f32a, int r) { return f32a && r == 2 ? 2 : 4; }

// Bytes of one column's scale words for the nsl slices of a part, padded so that the 16 columns of
// a tile fall into different LDS banks.
__host__ __device__ constexpr uint32_t meta_stride(int fmt, uint32_t nsl) { return nsl * kSliceBlocks * (fmt == MGN_FMT_Q4 ? 4 : 2) + 16; }

template <int FMT, bool F32A, int R, int Q, bool PARK, bool LATE = false>
__global__ __launch_bounds__(512) void tile_resident_kernel(const void* __restrict__ a, const void* __restrict__ meta_arg,
                                                             const void* __restrict__ quants_arg, uint32_t m, uint32_t kdim,
                                                             uint32_t n, uint32_t parts, uint32_t nslices, uint32_t colgroups,
                                                             TileTail tail) {
  constexpr uint32_t UNITS = image_units(F32A);
  constexpr float kOpScale = FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f;
  constexpr int QB = FMT == MGN_FMT_Q4 ? 16 : 32;
  constexpr int MB = FMT == MGN_FMT_Q4 ? 4 : 2;
  constexpr int NLQ = QB / 8;
  constexpr int NSL = resident_slices(F32A, R);
  constexpr int STEPS = NSL * Q;  // step f of the walk = (pair f / NSL, slice f % NSL)
  constexpr int DEPTH = 1;        // steps whose quants are in flight ahead of the one in use
  constexpr int SLOTS = DEPTH + 1;
  constexpr int NT = NSL * R;     // conversion tasks per half-wave
  // 16-byte units of scale words a lane stages: Q pairs x 32 columns x NSL slices x (32 or 16) bytes / 64 lanes
  constexpr int MU = Q * NSL * MB / 4;
  constexpr uint32_t kUnitsPerColumn = NSL * kSliceBlocks * MB / 16;
  constexpr uint32_t mstride = meta_stride(FMT, NSL);
  extern __shared__ uint4 lds4[];
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t c = lane & 15, g = lane >> 4;
  // grid = (column groups x row groups, rounded up to a multiple of 8; K parts): workgroups go to the
  // eight XCDs in turn by their linear index, so the K parts of a (column group, row group) run on
  // one XCD, which their hand-over below measures 0.5 us better than spread over all eight
  const uint32_t part = blockIdx.y;
  const uint32_t rg = blockIdx.x / colgroups, cg = blockIdx.x - rg * colgroups;
  const uint32_t rowgroups = (m + R * 16 - 1) / (R * 16);
  if (rg >= rowgroups) return;            // padding of the grid
  const uint32_t row0 = rg * (R * 16);    // first row of this workgroup's row group
  const uint32_t bpc = kdim / 32;
  const uint32_t pair0 = (cg * 8 + wave) * Q;  // this wave's first pair of column tiles
  const uint32_t sl0 = part * NSL;             // first slice of this part
  uint4* const img = lds4;                     // [NSL][R][UNITS]
  // this wave's scale words: [Q pairs x 32 columns][mstride bytes]
  uint8_t* const wmeta = (uint8_t*)(lds4 + NSL * R * UNITS) + wave * (Q * 32 * mstride);
  // PARK: this wave's strip for the quants of the step at hand, kSide x 16 columns
  constexpr int kStride = park_stride(FMT);
  uint8_t* const wpark = (uint8_t*)(lds4 + NSL * R * UNITS) + 8 * (Q * 32 * mstride) + wave * (kSide * 16 * kStride);

  // ---- the part's activations: loads first, so that nothing queues in front of them ----
  // Task (s, rr): half-wave r converts row 16 rr + r of slice sl0 + s.
  const uint32_t cr = tid >> 5, cl = tid & 31;
  TaskWords<F32A> xin[NT];
  bool xok[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const uint32_t s = t / R, rr = t % R;
    const uint32_t row = row0 + rr * 16 + cr, k0 = (sl0 + s) * 256 + cl * 8;
    xok[t] = row < m && k0 < kdim;
    load_task<F32A>(a, xok[t] ? (size_t)row * kdim + k0 : (size_t)0, xin[t]);
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- the scale words of all the wave's columns and slices: one pass, through LDS ----
  // A column's words for the part's slices are contiguous (kUnitsPerColumn 16-byte units).  Unit
  // id = 64 j + lane: column id / kUnitsPerColumn (of the wave's Q x 32), unit id % kUnitsPerColumn.
  // Every lane of a column's tile reads them back slice by slice during the walk.
  u32x4_t mu[MU];
  auto load_scale_words = [&]() {
#pragma unroll
    for (int j = 0; j < MU; j++) {
      const uint32_t id = 64 * j + lane;
      const uint32_t wcol = id / kUnitsPerColumn, unit = id % kUnitsPerColumn;
      const uint32_t col = min(pair0 * (kSide * 16) + wcol, n - 1);
      const uint8_t* src = (const uint8_t*)meta_arg + ((size_t)col * bpc + (size_t)sl0 * kSliceBlocks) * MB + unit * 16;
      typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
      const u32x4_a2 v = *(const u32x4_a2*)src;
      mu[j] = u32x4_t{v.x, v.y, v.z, v.w};
    }
  };
  load_scale_words();

  // ---- weight slices ----
  // Slices past the end of K (last part) and columns past N read the pad behind the weights or
  // a neighbour's data; their products are dropped.
  u32x4_t wq[SLOTS][kSide][NLQ];
  constexpr uint32_t LPC = QB / 2, CPL = 64 / LPC;  // PARK: lanes per column, columns per load
  const uint32_t lane_part = FMT == MGN_FMT_Q4 ? g * 16 : (g & 1) * 32 + (g >> 1) * 16;
  uint32_t q_off[Q][kSide][PARK ? NLQ : 1];
#pragma unroll
  for (int p = 0; p < Q; p++)
#pragma unroll
    for (int u = 0; u < kSide; u++) {
      if constexpr (PARK) {
#pragma unroll
        for (int j = 0; j < NLQ; j++)
          q_off[p][u][j] = min(((pair0 + p) * kSide + u) * 16 + CPL * j + lane / LPC, n - 1) * bpc * QB + (lane % LPC) * 16;
      } else {
        q_off[p][u][0] = min(((pair0 + p) * kSide + u) * 16 + c, n - 1) * bpc * QB + lane_part;
      }
    }
  auto fetch = [&](int f) {  // step f into slot f % SLOTS
    const uint8_t* const qb = (const uint8_t*)quants_arg + (size_t)((sl0 + f % NSL) * kSliceBlocks) * QB;
#pragma unroll
    for (int u = 0; u < kSide; u++)
#pragma unroll
      for (int j = 0; j < NLQ; j++)
        wq[f % SLOTS][u][j] = __builtin_nontemporal_load(
            (const u32x4_t*)(qb + (PARK ? q_off[f / NSL][u][PARK ? j : 0] : q_off[f / NSL][u][0] + 64 * j)));
  };
  // ---- activations -> images in LDS; scale words -> LDS ----
  // The first slices of quants are requested between the conversion tasks, not before them: a
  // CU's memory pipeline is busy with the activations until then, and every load queued in
  // front of them delays the conversion that all waves wait for (first request after the second
  // task, one slice ahead from there on: 15.0 -> 14.0 us at M = 16 on 4096 x 14336; two slices
  // ahead or any request before the conversion measured 0.3-2.3 us slower).
  // LATE (row groups of 32 fp16 rows on a chip that the launch fills): not before the last task.
  // The eight tasks of such a workgroup read 64 KB of activations, and with every CU doing the
  // same the weights requested in between only stand in their way: fp16 512 x 1024 x 3072 11.23 ->
  // 10.93 us, 512 x 3072 x 1024 14.22 -> 14.0.  (On half a chip the early request wins: M = 64 on
  // 4096 x 4096, 128 workgroups, 10.2 against 10.45 us; and with f32 activations a later one loses.)
  constexpr int kFirstFetchAfterTask = NT > 1 ? (LATE ? NT - 1 : 1) : 0;
#pragma unroll
  for (int t = 0; t < NT; t++) {
    convert_task<FMT, F32A>(xin[t], xok[t], img + t * UNITS, cr, cl);
    __builtin_amdgcn_sched_barrier(0);
    if (t >= kFirstFetchAfterTask && t - kFirstFetchAfterTask < DEPTH && t - kFirstFetchAfterTask < STEPS) fetch(t - kFirstFetchAfterTask);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int f = NT - kFirstFetchAfterTask; f < DEPTH && f < STEPS; f++) fetch(f);
#pragma unroll
  for (int j = 0; j < MU; j++) {
    const uint32_t id = 64 * j + lane;
    *(u32x4_t*)(wmeta + (id / kUnitsPerColumn) * mstride + (id % kUnitsPerColumn) * 16) = mu[j];
  }
  __builtin_amdgcn_sched_barrier(0);
  lds_barrier();
  __builtin_amdgcn_sched_barrier(0);

  floatx4 res[Q][kSide][R];
#pragma unroll
  for (int p = 0; p < Q; p++)
#pragma unroll
    for (int u = 0; u < kSide; u++)
#pragma unroll
      for (int r = 0; r < R; r++) res[p][u][r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
  const bool pair_live[2] = {pair0 * (kSide * 16) < n, (pair0 + Q - 1) * (kSide * 16) < n};  // uniform over the wave
#pragma unroll
  for (int f = 0; f < STEPS; f++) {
    const int slot = f % SLOTS, wp = f / NSL, ws = f % NSL;
    __builtin_amdgcn_sched_barrier(0);
    if (f + DEPTH < STEPS) fetch(f + DEPTH);
    __builtin_amdgcn_sched_barrier(0);
    // the slot's quants into B operand order, the step's scale words from LDS
    uint32_t mw[kSide][8];
#pragma unroll
    for (int u = 0; u < kSide; u++) {
      const uint8_t* const ms = wmeta + ((wp * kSide + u) * 16 + c) * mstride + ws * (kSliceBlocks * MB);
      if constexpr (FMT == MGN_FMT_Q4) {
        const u32x4_t m0 = *(const u32x4_t*)ms, m1 = *(const u32x4_t*)(ms + 16);
        mw[u][0] = m0.x, mw[u][1] = m0.y, mw[u][2] = m0.z, mw[u][3] = m0.w;
        mw[u][4] = m1.x, mw[u][5] = m1.y, mw[u][6] = m1.z, mw[u][7] = m1.w;
      } else {
        const u32x4_t m0 = *(const u32x4_t*)ms;
        const uint32_t v[4] = {m0.x, m0.y, m0.z, m0.w};
#pragma unroll
        for (int e = 0; e < 4; e++) mw[u][2 * e] = v[e] & 0xFFFFu, mw[u][2 * e + 1] = v[e] >> 16;
      }
      if constexpr (PARK) {
#pragma unroll
        for (int j = 0; j < NLQ; j++)
          *(u32x4_t*)(wpark + (u * 16 + CPL * j + lane / LPC) * kStride + (lane % LPC) * 16) = wq[slot][u][j];
      } else if constexpr (FMT == MGN_FMT_Q4) {
        transpose_rows(wq[slot][u][0]);
        transpose_rows(wq[slot][u][1]);
      } else {
#pragma unroll
        for (int j = 0; j < NLQ; j++) swap_row_pairs(wq[slot][u][j]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t sl_raw = sl0 + ws;
    if (pair_live[wp == 0 ? 0 : 1] && sl_raw < nslices) {  // (with Q = 2, wp is 0 or 1)
      const uint32_t kb0 = sl_raw * kSliceBlocks;
      if (kb0 + kSliceBlocks > bpc) {  // last slice of a K that is no multiple of 256
#pragma unroll
        for (int u = 0; u < kSide; u++)
#pragma unroll
          for (int e = 0; e < 8; e++) mw[u][e] = kb0 + e < bpc ? mw[u][e] : 0u;
      }
      slice_mac_side<FMT, F32A, R, PARK>(wq[slot], wpark + c * kStride + g * (QB / 4), mw, (const uint8_t*)(img + ws * R * UNITS),
                                         UNITS * 16, g, lane, tail.lift, res[wp]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (!F32A) {
#pragma unroll
    for (int p = 0; p < Q; p++)
#pragma unroll
      for (int u = 0; u < kSide; u++)
#pragma unroll
        for (int r = 0; r < R; r++) res[p][u][r] *= kOpScale;
  }
  __builtin_amdgcn_sched_barrier(0);

  if (parts > 1) {
    // K parts of other workgroups.  The parts of a (column group, row group) run on one XCD (see the
    // grid above) and the part with the highest index is dispatched last, when the others are
    // already running or done; it is the one that adds them up, in part order, its own sums last.
    // There is no counter and no barrier: the hand-over workspace holds kHandoverEmpty in every word
    // between launches, a part stores its tiles over it and is done (write-through stores, device
    // scope), and every wave of the adding workgroup polls the slots of its own tiles until none of
    // their words is empty any more, then puts the pattern back for the next launch.  A wait costs
    // one trip to the XCD's L2 per poll, not the three dependent trips through memory of a counted
    // hand-over (stores acknowledged, count returned, tiles read): M = 16 on 4096 x 14336, 4 parts,
    // 12.8 -> 10.6 us.  The wait is bounded: after spin_limit polls the wave sets the context's
    // fault word, which the next synchronising call reports, and goes on with what it has.
    // The partial tiles travel in register order: the float4 a lane holds for (pair, side, row tile)
    // goes out and comes back as one 128-bit access, 1 KiB per wave and instruction, at
    //   (((part * row groups + row group) * column groups + column group) * 8 + wave) * Q * kSide * R + slot
    constexpr uint32_t kSlots = Q * kSide * R;
    constexpr int kDeviceScope = 16;  // the sc1 bit of a buffer instruction's cache policy
    const uint32_t wgs_per_part = rowgroups * colgroups;
    const uint32_t part_stride = wgs_per_part * (8u * kSlots * 1024u);
    const __amdgpu_buffer_rsrc_t partials =
        __builtin_amdgcn_make_buffer_rsrc(tail.handover, 0, (parts - 1) * part_stride, 0x00020000);
    const uint32_t my_off = ((rg * colgroups + cg) * 8u + wave) * (kSlots * 1024u) + lane * 16u;
    if (tail.spread) {
      // Every part adds up a share.  With many parts the one workgroup that reads all the others'
      // tiles takes them in at the rate of a single CU (14 parts: 208 KB, 1.5 us); here every part
      // stores ALL its tiles (its own share included), and tile T = wave * kSlots + slot of the
      // group belongs to part T % parts, whose wave T / parts polls the `parts` copies of that one
      // tile, adds them in part order, stores the outputs and puts the pattern back.  Every part
      // waits for every other, so the planner asks for this only when the whole grid is resident
      // at once (at most one workgroup per CU).  The workspace holds `parts` sets of tiles.
      const __amdgpu_buffer_rsrc_t all_parts = __builtin_amdgcn_make_buffer_rsrc(tail.handover, 0, parts * part_stride, 0x00020000);
#pragma unroll
      for (int p = 0; p < Q; p++)
#pragma unroll
        for (int u = 0; u < kSide; u++)
#pragma unroll
          for (int r = 0; r < R; r++) {
            u32x4_t v = __builtin_bit_cast(u32x4_t, res[p][u][r]);
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = v[i] == kHandoverEmpty ? 0x7FC00000u : v[i];
            __builtin_amdgcn_raw_buffer_store_b128(v, all_parts, part * part_stride + my_off + ((p * kSide + u) * R + r) * 1024u, 0,
                                                   kDeviceScope);
          }
      bool gave_up = false;
      // the tiles this wave adds up: part + parts * (wave, wave + 8, ..) while the group has that many
      for (uint32_t tile = part + wave * parts; tile < 8u * kSlots; tile += 8u * parts) {
        const uint32_t src_wave = tile / kSlots, slot = tile - src_wave * kSlots;
        const uint32_t t_off = ((rg * colgroups + cg) * 8u + src_wave) * (kSlots * 1024u) + slot * 1024u + lane * 16u;
        floatx4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
        constexpr uint32_t PG = 8;
        const u32x4_t empty4 = {kHandoverEmpty, kHandoverEmpty, kHandoverEmpty, kHandoverEmpty};
        for (uint32_t pp0 = 0; pp0 < parts; pp0 += PG) {
          uint32_t v[PG][4];  // (scalars: vectors assigned inside a divergent polling loop have come out wrong)
#pragma unroll
          for (uint32_t j = 0; j < PG; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) v[j][i] = kHandoverEmpty;
          for (uint32_t polls = 0;; polls++) {
            if (polls >= tail.spin_limit) {  // (a limit of 0 looks at nothing: the give-up path, for tests)
              gave_up = true;
              break;
            }
            bool missing = false;
#pragma unroll
            for (uint32_t j = 0; j < PG; j++) {
              const u32x4_t x4 = __builtin_amdgcn_raw_buffer_load_b128(all_parts, min(pp0 + j, parts - 1) * part_stride + t_off, 0, kDeviceScope);
              v[j][0] = x4.x, v[j][1] = x4.y, v[j][2] = x4.z, v[j][3] = x4.w;
              missing |= x4.x == kHandoverEmpty || x4.y == kHandoverEmpty || x4.z == kHandoverEmpty || x4.w == kHandoverEmpty;
            }
            if (!__builtin_amdgcn_ballot_w64(missing)) break;
            __builtin_amdgcn_s_sleep(1);
            asm volatile("" ::: "memory");  // the loads are issued anew on every round
          }
#pragma unroll
          for (uint32_t j = 0; j < PG; j++) {
            if (pp0 + j < parts) {  // uniform
#pragma unroll
              for (int i = 0; i < 4; i++) sum[i] += __builtin_bit_cast(float, v[j][i]);
              __builtin_amdgcn_raw_buffer_store_b128(empty4, all_parts, (pp0 + j) * part_stride + t_off, 0, kDeviceScope);
            }
          }
        }
        // the tile's place in the output: slot = (pair * kSide + side) * R + row tile of wave src_wave
        const uint32_t tp = slot / (kSide * R), tu = (slot / R) % kSide, tr = slot % R;
        const uint32_t col = (((cg * 8 + src_wave) * Q + tp) * kSide + tu) * 16 + c;
        if (col < n) {
          if (row0 + R * 16 <= m && !tail.dres && tail.epilogue == 0) {  // (uniform) whole rows, nothing to add or apply
            float* const dst = tail.c + (size_t)(row0 + tr * 16 + 4 * g) * n + col;
#pragma unroll
            for (int i = 0; i < 4; i++) dst[(size_t)i * n] = sum[i];
          } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
              const uint32_t row = row0 + tr * 16 + 4 * g + i;
              if (row < m) {
                const size_t o = (size_t)row * n + col;
                tail.c[o] = apply_epilogue(tail.dres ? sum[i] + tail.dres[o] : sum[i], tail.epilogue);
              }
            }
          }
        }
      }
      if (gave_up && lane == 0 && tail.fault_flag) *tail.fault_flag = 1u;
      return;
    }
    if (part + 1 < parts) {
#pragma unroll
      for (int p = 0; p < Q; p++)
#pragma unroll
        for (int u = 0; u < kSide; u++)
#pragma unroll
          for (int r = 0; r < R; r++) {
            u32x4_t v = __builtin_bit_cast(u32x4_t, res[p][u][r]);
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = v[i] == kHandoverEmpty ? 0x7FC00000u : v[i];
            __builtin_amdgcn_raw_buffer_store_b128(v, partials, part * part_stride + my_off + ((p * kSide + u) * R + r) * 1024u, 0,
                                                   kDeviceScope);
          }
      return;
    }
    floatx4 sum[kSlots];
#pragma unroll
    for (uint32_t t = 0; t < kSlots; t++) sum[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    bool gave_up = false;
    auto add_parts = [&](auto group) {
      constexpr int PG = decltype(group)::value;
      const u32x4_t empty4 = {kHandoverEmpty, kHandoverEmpty, kHandoverEmpty, kHandoverEmpty};
      for (uint32_t pp0 = 0; pp0 + 1 < parts; pp0 += PG) {
        u32x4_t v[PG][kSlots];
#pragma unroll
        for (int j = 0; j < PG; j++)
#pragma unroll
          for (uint32_t t = 0; t < kSlots; t++) v[j][t] = empty4;
        for (uint32_t polls = 0;; polls++) {
          if (polls >= tail.spin_limit) {  // (a limit of 0 looks at nothing: the give-up path, for tests)
            gave_up = true;
            break;
          }
          bool missing = false;
#pragma unroll
          for (int j = 0; j < PG; j++) {
            const uint32_t po = min(pp0 + j, parts - 2) * part_stride + my_off;  // (the surplus repeats the last part)
#pragma unroll
            for (uint32_t t = 0; t < kSlots; t++) v[j][t] = __builtin_amdgcn_raw_buffer_load_b128(partials, po + t * 1024u, 0, kDeviceScope);
          }
#pragma unroll
          for (int j = 0; j < PG; j++)
#pragma unroll
            for (uint32_t t = 0; t < kSlots; t++)
              missing |= v[j][t].x == kHandoverEmpty || v[j][t].y == kHandoverEmpty || v[j][t].z == kHandoverEmpty || v[j][t].w == kHandoverEmpty;
          if (!__builtin_amdgcn_ballot_w64(missing)) break;
          __builtin_amdgcn_s_sleep(1);
          asm volatile("" ::: "memory");  // the loads are issued anew on every round
        }
#pragma unroll
        for (int j = 0; j < PG; j++) {
          const bool live = pp0 + j + 1 < parts;
          if (live) {  // uniform
#pragma unroll
            for (uint32_t t = 0; t < kSlots; t++) {
              sum[t] += __builtin_bit_cast(floatx4, v[j][t]);
              __builtin_amdgcn_raw_buffer_store_b128(empty4, partials, (pp0 + j) * part_stride + my_off + t * 1024u, 0, kDeviceScope);
            }
          }
        }
      }
    };
    if (parts <= 5) add_parts(std::integral_constant<int, 4>{});
    else add_parts(std::integral_constant<int, 16 / (Q * R)>{});
#pragma unroll
    for (int p = 0; p < Q; p++)
#pragma unroll
      for (int u = 0; u < kSide; u++)
#pragma unroll
        for (int r = 0; r < R; r++) res[p][u][r] = sum[(p * kSide + u) * R + r] + res[p][u][r];
    if (gave_up && lane == 0 && tail.fault_flag) *tail.fault_flag = 1u;
  }
  // The stores end every wave's life, with nothing left to hide them behind: a row group that lies
  // inside M whole, with no residual and no unary operation, stores through one pointer per tile and
  // a running row stride, without a test or a 64-bit product per element.
  const bool whole_rows = row0 + R * 16 <= m && tail.epilogue == 0;  // uniform
#pragma unroll
  for (int p = 0; p < Q; p++)
#pragma unroll
    for (int u = 0; u < kSide; u++) {
      const uint32_t col = ((pair0 + p) * kSide + u) * 16 + c;
      if (col < n) {
        if (whole_rows) {
          const size_t first = (size_t)(row0 + 4 * g) * n + col;
          float* dst = tail.c + first;
          if (tail.dres) {  // (uniform) the residual's loads first, all of a tile column's at once
            const float* src = tail.dres + first;
            float dv[R][4];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
              for (int i = 0; i < 4; i++) dv[r][i] = src[(size_t)(16 * r + i) * n];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
              for (int i = 0; i < 4; i++) dst[(size_t)(16 * r + i) * n] = res[p][u][r][i] + dv[r][i];
            continue;
          }
#pragma unroll
          for (int r = 0; r < R; r++) {
#pragma unroll
            for (int i = 0; i < 4; i++) dst[(size_t)i * n] = res[p][u][r][i];
            dst += (size_t)16 * n;
          }
          continue;
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const uint32_t row = row0 + r * 16 + 4 * g + i;
            if (row < m) {
              const size_t o = (size_t)row * n + col;
              tail.c[o] = apply_epilogue(tail.dres ? res[p][u][r][i] + tail.dres[o] : res[p][u][r][i], tail.epilogue);
            }
          }
      }
    }
}

// s = WeightView::additive_lift: 2^s as an fp16 pair and 2^-s
AddLift add_lift(const WeightView& w) {
  const uint32_t s = std::min<uint32_t>(w.additive_lift, 15u);
  const uint32_t h = (15u + s) << 10;  // fp16 bits of 2^s
  return AddLift{h | (h << 16), std::ldexp(1.0f, -(int)s)};
}

struct ResidentPlan {
  uint32_t r, q, nsl, parts, colgroups, rowgroups, nslices;
  bool park;  // quants through a wave-private LDS strip (if there is room) instead of row swaps
  bool spread;  // the K parts' tiles are added up by all parts, a share each (see the kernel)
  size_t lds, partial_bytes;
  double cost;
};

size_t resident_lds_bytes(int fmt, bool f32a, uint32_t r, uint32_t q, bool park) {
  const uint32_t nsl = resident_slices(f32a, r);
  return (size_t)nsl * r * image_units(f32a) * 16 + (size_t)8 * q * 32 * meta_stride(fmt, nsl) +
         (park ? (size_t)8 * kSide * 16 * park_stride(fmt) : 0);
}

// Row groups of 16 or 32 rows (32 only beyond 16 rows, and then with one pair per wave: registers), Q = 1 or 2 pairs
// of tiles per wave: the combination whose grid takes the fewest rounds over the CUs, weighted by
// what a workgroup does (a fixed part for the conversion and the hand-over, its waves' steps; row
// groups of 32 share every unpacked B operand between two row tiles and win a tie: fp16
// 512 x 1024 x 3072 11.9 us against 15.5 us in row groups of 16).
bool plan_resident(const LaunchArgs& x, ResidentPlan* out) {
  if (x.m == 0 || x.w.k < 32) return false;
  const uint32_t bpc = x.w.k / 32;
  if ((uint64_t)x.w.n * bpc * 32 >= (1ull << 32)) return false;  // a lane's weight offsets are 32-bit
  const bool f32a = !x.a_is_f16;
  const uint32_t nslices = (bpc + kSliceBlocks - 1) / kSliceBlocks, n_tiles = (x.w.n + 15) / 16;
  double best = 0;
  ResidentPlan bp{};
  for (uint32_t r = 1; r <= 2; r++) {
    // Row groups of 32 are for fp16 activations: with f32 only two slices of 32 rows fit in LDS, K falls
    // into twice as many parts, and two row groups of 16 are faster throughout (M = 32 on 4096 x 14336:
    // 22.7 against 33.0 us, 576 x 576: 8.1 against 11.6 us)
    if (r == 2 && (x.m <= 16 || f32a)) continue;
    if (r == 1 && !f32a && x.m > 16 && x.m <= 32) continue;  // fp16: one row group of 32 instead of two of 16
    const uint32_t nsl = resident_slices(f32a, r);
    const uint32_t parts = (nslices + nsl - 1) / nsl;
    const uint32_t rowgroups = (x.m + 16 * r - 1) / (16 * r);
    if (rowgroups > 65535) continue;
    for (uint32_t q = 1; q <= (r == 1 ? 2u : 1u); q++) {
      const uint32_t per_wg = 8 * kSide * q;
      const uint32_t colgroups = (n_tiles + per_wg - 1) / per_wg;
      if (parts > 65535 || (uint64_t)colgroups * rowgroups > 0x7FFFFFF0ull) continue;
      // a workgroup's partial tile: 8 waves x (q kSide r) float4 per lane; the last part keeps its own
      // Every part adds up a share of the tiles when all workgroups are resident at once (every part then
      // waits for every other); the workspace then holds the last part's tiles too.  Measured against
      // the one reader at M = 16 (us, reader / shares): 14336 x 4096, 14 parts, 15.1 / 12.8 (Q8 19.0 /
      // 15.8); 11008 x 4096, 11 parts, 16.0 / 12.1; 8192 x 4096, 8 parts, 13.5 / 11.1; 4096 x 4096, 4
      // parts, 11.4 / 10.8; 3072 x 4096 11.3 / 10.7; 2048 x 14336, 2 parts, 11.7 / 11.1; fp16 512 x
      // 3072 x 1024 14.8 / 14.6.  With four parts or fewer on a nearly full chip it is level or loses
      // (4096 x 11008, 172 workgroups: 12.1 / 12.2; 4096 x 14336, 224 workgroups: 12.5 / 13.0).
      // Resident at once means per XCD: workgroups go to the eight XCDs in turn by their linear index, the
      // groups are in grid x (a multiple of 8) and the parts in y, so an XCD gets ceil(groups / 8) groups
      // with all their parts, one workgroup per CU, on an eighth of the CUs.
      const uint64_t wgs = (uint64_t)parts * colgroups * rowgroups;
      const uint64_t per_xcd = ((uint64_t)colgroups * rowgroups + 7) / 8 * parts;
      const bool spread = !x.shared_device && parts >= 2 && per_xcd <= (uint64_t)x.num_cus / 8 &&
                          (parts >= 5 || 3 * wgs <= 2 * (uint64_t)x.num_cus);
      const uint64_t partial = parts > 1 ? (uint64_t)(spread ? parts : parts - 1) * rowgroups * colgroups * (8u * q * kSide * r * 1024u) : 0;
      if (partial > x.handover_bytes || partial >= (1ull << 32)) continue;
      const double cost = std::ceil((double)wgs / x.num_cus) * (1.5 + q * r * nsl / 4.0) * (r == 2 ? 0.9 : 1.0) + (parts > 1 ? 1.0 : 0.0);
      if (best == 0 || cost < best) {
        best = cost;
        bp.r = r, bp.q = q, bp.nsl = nsl, bp.parts = parts, bp.colgroups = colgroups, bp.rowgroups = rowgroups;
        bp.nslices = nslices, bp.partial_bytes = partial, bp.cost = cost, bp.spread = spread;
        bp.park = resident_lds_bytes(x.w.fmt, f32a, r, q, true) <= 160 * 1024;
        bp.lds = resident_lds_bytes(x.w.fmt, f32a, r, q, bp.park);
      }
    }
  }
  if (best == 0) return false;
  *out = bp;
  return true;
}

template <int FMT, bool F32A, int R, int Q, bool PARK, bool LATE = false>
int launch_resident_q(ihipStream_t* s, const LaunchArgs& x, const ResidentPlan& p) {
  auto kern = tile_resident_kernel<FMT, F32A, R, Q, PARK, LATE>;
  static std::atomic<uint64_t> big_lds_done{0};
  if (p.lds > 64 * 1024)
    if (int e = enable_big_lds(kern, x.device, big_lds_done)) return e;
  const TileTail tail{x.d, x.c, (float*)x.scratch, x.counters, x.epilogue, (float*)x.handover, x.spin_limit, x.fault_flag, p.spread ? 1u : 0u, add_lift(x.w)};
  // (column groups x row groups, K parts); with K parts the first is rounded up to a multiple of 8 (see the kernel)
  const uint64_t groups = (uint64_t)p.colgroups * p.rowgroups;
  const dim3 grid((unsigned)(p.parts > 1 ? (groups + 7) / 8 * 8 : groups), p.parts, 1);
  hipLaunchKernelGGL(kern, grid, dim3(512), p.lds, s, x.a, x.w.meta, x.w.quants, x.m, x.w.k, x.w.n, p.parts, p.nslices,
                     p.colgroups, tail);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

template <int FMT, bool F32A>
int launch_resident_fa(ihipStream_t* s, const LaunchArgs& x, const ResidentPlan& p) {
  if constexpr (!F32A) {
    if (p.r == 2) {
      // the first weight request waits for the conversion when the launch fills the chip (see the kernel)
      const bool late = (uint64_t)p.parts * p.colgroups * p.rowgroups * 10 >= (uint64_t)x.num_cus * 7;
      if (p.park) return late ? launch_resident_q<FMT, F32A, 2, 1, true, true>(s, x, p) : launch_resident_q<FMT, F32A, 2, 1, true>(s, x, p);
      return late ? launch_resident_q<FMT, F32A, 2, 1, false, true>(s, x, p) : launch_resident_q<FMT, F32A, 2, 1, false>(s, x, p);
    }
  }
  if (p.r != 1) return (int)hipErrorInvalidValue;
  if (p.q == 1)
    return p.park ? launch_resident_q<FMT, F32A, 1, 1, true>(s, x, p) : launch_resident_q<FMT, F32A, 1, 1, false>(s, x, p);
  return p.park ? launch_resident_q<FMT, F32A, 1, 2, true>(s, x, p) : launch_resident_q<FMT, F32A, 1, 2, false>(s, x, p);
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
          // the images of every row tile and slice sit behind the partial tiles in the workspace
          const size_t images = (size_t)rowgroups * r * parts * nph * ksc * units * 16;
          if (((partial + 255) & ~(size_t)255) + images > x.scratch_bytes) continue;
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
  const TileTail tail{x.d, x.c, (float*)x.scratch, x.counters, x.epilogue, nullptr, 0, nullptr, 0, add_lift(x.w)};
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

// Which of the two kernels takes a call.  Up to 32 rows: the one with LDS-resident images.  Beyond,
// it runs row groups side by side and still wins where K is short enough for at most four K parts
// and their partial tiles stay small (f32 512 x 1024 x 3072: 16.5 us against 29 us with images
// through the workspace; 128 x 4096 x 4096: 21.8 against 28.8), except for Q8 below 128 rows,
// where too few workgroups carry too much each (64 x 1024 x 3072: 13.9 against 11.2 us), and for
// wide outputs whose partial tiles dominate (64 x 4096 x 14336: 43 against 40 us).
bool use_resident(const LaunchArgs& x, ResidentPlan* rp) {
  if (!plan_resident(x, rp)) return false;
  if (x.m <= 32) return true;
  return rp->parts <= 4 && rp->partial_bytes <= ((size_t)8 << 20) && (x.w.fmt == MGN_FMT_Q4 || x.m >= 128);
}

// The general kernel's plan for as many rows per launch as the workspace has room for (partial
// tiles + activation images): all of them, or blocks of a multiple of 16 rows launched one after
// the other.  False if not even 16 rows fit.
bool plan_tile_rows(const LaunchArgs& x, TilePlan* p, uint32_t* rows) {
  LaunchArgs y = x;
  for (uint32_t mc = x.m;;) {
    y.m = mc;
    if (plan_tile(y, p) && tile_workspace_bytes(*p) <= x.scratch_bytes) {
      *rows = mc;
      return true;
    }
    if (mc <= 16) return false;
    mc = mc > 128 ? (mc / 2 + 63) / 64 * 64 : (mc / 2 + 15) / 16 * 16;
  }
}

}  // namespace

bool tile_mfma_supported(const LaunchArgs& x) {
  ResidentPlan rp;
  if (use_resident(x, &rp)) return true;
  TilePlan p;
  uint32_t rows;
  return plan_tile_rows(x, &p, &rows);
}

// Where the resident kernel measured faster than the 32x32 tiled one, whatever is known about
// the activations.  Up to 16 rows: K >= 544 and workgroups that fill at least three quarters of
// their rounds over the CUs (4096 x 14336 at M = 5..16: 12.5 us against 17.0 us; 14336 x 4096, 14 K
// parts: 15.5-15.9 against 17.6-18.0, Q8 18.3-19.2 against 21.3-22.9; 4096 x 49152, 1.5 rounds: 36.3
// against 43.7, Q8 55.2 against 55.9; 8192 x 28672, 1.75 rounds: 39.9 against 47.8, Q8 59.9 against
// 65.1; on smaller shapes the conversion in every workgroup and the parts' hand-over cost more than
// the tiled kernel's whole call, and so does a round that stays half empty: 5120 x 14336, 0.55 of a
// round, 22.9 against 20.3, Q8 34.3 against 25.1; 6144 x 14336, 0.66: 23.0 against 22.2, Q8 33.4
// against 28.7).  17 to 32 rows of f32 activations, where the tiled kernel runs twice the MFMAs: whenever
// the two row groups' workgroups fit one round (576 x 576: 8.0 against 11.4 us, 4096 x 4096: 11.5
// against 15.8, 8192 x 4096, 8 K parts: 15.0 against 21.6, 14336 x 1536, 14 parts: 15.0 against 22.9,
// 14336 x 4096 at two pairs of tiles per wave 24.2 against 26.4; with more workgroups the weights'
// second pass costs more: 1536 x 49152 33.2 against 24.6, 8192 x 14336 39.7 against 36.1), except
// Q4 at two pairs per wave with K in one part (576 x 49152: 16.2 against 14.5), Q8 at two pairs per
// wave, which has no room to park its quants (4096 x 14336 31.8 against 27.4, 14336 x 4096 33.5
// against 29.8), and Q8 with K parts below K = 2048, where the hand-over is a third of the call
// (1536 x 576 11.9 against 10.5).  Beyond 32 rows: Q4 with K short enough for a single part (f32 activations:
// 128 x 1024 x 3072 9.2 against 13.3 us, 256 x 576 x 1536 8.9 against 13.3, 512 x 1024 x 3072 16.8
// against 17.6; fp16 activations, in row groups of 32: 512 x 1024 x 3072 11.9 against 13.1 us,
// 128 x 1024 x 3072 8.5 against 9.8), and with up to four K parts (which is where the resident form
// ends beyond 32 rows) when the workgroups fill three quarters of their rounds or, with the quants
// parked, fit one (fp16 512 x 3072 x 1024: 14.8-15.6 against 15.3-15.9 us, 512 x 4096 x 1024 15.9
// against 18.6, 48 x 3072 x 4096 10.3 against 13.2; f32 128 x 4096 x 4096 20.1 against 23.2, but
// 128 x 3072 x 3072, two pairs of tiles per wave without room to park the quants on 0.56 of the CUs,
// 20.4 against 19.0);
// Q8 is between 0.8 and 1.4 of the tiled kernel's time on this one and stays where it was.
bool tile_mfma_preferred(const LaunchArgs& x) {
  ResidentPlan rp;
  if (!use_resident(x, &rp)) return false;
  const uint64_t wgs = (uint64_t)rp.parts * rp.colgroups * rp.rowgroups;
  const uint64_t rounds = (wgs + x.num_cus - 1) / x.num_cus;
  if (x.m > 32)
    return x.w.fmt == MGN_FMT_Q4 && (rp.parts == 1 || (rp.park && rounds == 1) || 4 * wgs >= 3 * rounds * (uint64_t)x.num_cus);
  if (x.m > 16) {
    if (x.a_is_f16 || wgs > (uint64_t)x.num_cus) return false;
    if (x.w.fmt == MGN_FMT_Q4) return !(rp.q == 2 && rp.parts == 1);
    return rp.q == 1 && (rp.parts == 1 || rp.nslices >= 8);
  }
  if (rp.r != 1 || rp.nslices < 3) return false;
  return 4 * wgs >= 3 * rounds * (uint64_t)x.num_cus;
}

bool describe_tile_mfma(const LaunchArgs& x, mgn_plan_info* out) {
  ResidentPlan rp;
  if (use_resident(x, &rp)) {
    out->route = MGN_ROUTE_TILE_MFMA;
    out->grid[0] = rp.parts, out->grid[1] = rp.colgroups, out->grid[2] = rp.rowgroups;
    out->threads = 512;
    out->lds_bytes = (uint32_t)rp.lds;
    out->waves_n = 8 * kSide * rp.q, out->k_splits = 1, out->k_parts = rp.parts, out->steps = rp.nsl;
    out->quads_per_wave = 0, out->full_steps = rp.r, out->tail_blocks = 0;
    out->workspace_bytes = rp.partial_bytes;
    return true;
  }
  TilePlan p;
  uint32_t rows;
  if (!plan_tile_rows(x, &p, &rows)) return false;
  out->route = MGN_ROUTE_TILE_MFMA;
  out->grid[0] = p.parts, out->grid[1] = p.colgroups, out->grid[2] = p.rowgroups;
  out->threads = 64 * p.ksc * p.wnc;
  out->lds_bytes = (uint32_t)p.lds;
  out->waves_n = p.wnc, out->k_splits = p.ksc, out->k_parts = p.parts, out->steps = p.nph;
  out->quads_per_wave = (x.m + rows - 1) / rows;  // launches
  out->full_steps = p.r, out->tail_blocks = 0;
  out->workspace_bytes = tile_workspace_bytes(p);
  return true;
}

int launch_matmul_tile_mfma(ihipStream_t* s, const LaunchArgs& x) {
  ResidentPlan rp;
  if (use_resident(x, &rp)) {
    if (x.w.fmt == MGN_FMT_Q4)
      return x.a_is_f16 ? launch_resident_fa<MGN_FMT_Q4, false>(s, x, rp) : launch_resident_fa<MGN_FMT_Q4, true>(s, x, rp);
    return x.a_is_f16 ? launch_resident_fa<MGN_FMT_Q8, false>(s, x, rp) : launch_resident_fa<MGN_FMT_Q8, true>(s, x, rp);
  }
  TilePlan p;
  uint32_t rows;
  if (!plan_tile_rows(x, &p, &rows)) return (int)hipErrorInvalidValue;
  // blocks of rows, one launch pair (images, multiplication) each; they share the workspace and
  // follow each other on the stream
  for (uint32_t r0 = 0; r0 < x.m; r0 += rows) {
    LaunchArgs y = x;
    y.m = std::min(rows, x.m - r0);
    y.a = (const char*)x.a + (size_t)r0 * x.w.k * (x.a_is_f16 ? 2 : 4);
    y.c = x.c + (size_t)r0 * x.w.n;
    y.d = x.d ? x.d + (size_t)r0 * x.w.n : nullptr;
    if (y.m != rows && !plan_tile(y, &p)) return (int)hipErrorInvalidValue;  // the last, shorter block
    int e;
    if (x.w.fmt == MGN_FMT_Q4) e = x.a_is_f16 ? launch_fa<MGN_FMT_Q4, false>(s, y, p) : launch_fa<MGN_FMT_Q4, true>(s, y, p);
    else e = x.a_is_f16 ? launch_fa<MGN_FMT_Q8, false>(s, y, p) : launch_fa<MGN_FMT_Q8, true>(s, y, p);
    if (e) return e;
  }
  return 0;
}

}  // namespace mgn
