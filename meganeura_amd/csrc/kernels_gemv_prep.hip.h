// Activation staging helpers of the decode kernels (MFMA 4x4x4 forms): fp16 splitting, integer
// digits for the int8 matrix instruction, block scaling, lane reductions.
#pragma once
#include "kernels_common.hip.h"

namespace mgn {
namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// fp16 bit patterns used as operands stand for value * 2^-kOperandShift
template <int FMT>
constexpr float operand_scale() { return FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f; }  // 2^20, 2^24
constexpr int kMaxTasks = 2;  // activation chunks a thread prepares at most, per row
// weight blocks in flight per lane ahead of the one in use (measured: 3 for Q4's 20-byte
// blocks, 2 for Q8's 34-byte blocks; the one-row Q4 kernel takes one more where a wave has the
// loads for it, see gemv_mfma_kernel)
template <int FMT>
constexpr int prefetch_depth() { return FMT == MGN_FMT_Q8 ? 2 : 3; }

__device__ __forceinline__ half4 as_half4(uint32_t lo, uint32_t hi) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  const u32x2 v = {lo, hi};
  return __builtin_bit_cast(half4, v);
}

// two floats -> packed fp16 pair, truncating: the low halves computed from the
// residual make up for the truncation
__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ float half_lo(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[0]; }
__device__ __forceinline__ float half_hi(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[1]; }

constexpr int kRowRor4 = 0x124, kRowRor8 = 0x128;  // rotate right within a row of 16 lanes

// Sums over the 16 lanes of a wave that share lane % 4 (the 16 K blocks of a step, per column), for
// MROWS accumulators at once, without a trip through LDS: the halves and rows of the
// wave are folded with the row-swap instructions while the activation rows are handed out to them
// (3 swaps and 3 adds for four rows, where four separate sums take 8 cross-row exchanges), then
// two rotations inside a row.  Every lane ends with the total of column lane % 4 for ONE
// activation row, *row: lanes 16 j .. 16 j + 15 hold row {0, 2, 1, 3}[j] of four (rows past MROWS
// are zero sums), row j / 2 of two, row 0 of one.  *writer: one lane per (row, column).
template <int MROWS>
__device__ __forceinline__ float sum_rows_over_blocks(const float (&acc)[MROWS], uint32_t lane, uint32_t* row, bool* writer) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  // (the instructions swap two registers in place: one value given twice needs a register of its own)
  auto twin = [](float a) {
    float b = a;
    asm volatile("" : "+v"(b));
    return b;
  };
  auto fold32 = [](float a, float b) {  // lanes 0..31: a(lane) + a(lane + 32); lanes 32..63: b(lane - 32) + b(lane)
    const u32x2 s = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b), false, false);
    uint32_t x = s.x, y = s.y;
    asm volatile("" : "+v"(x), "+v"(y));  // (without it the sum came out as x + x)
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
  };
  auto fold16 = [](float a, float b) {  // even rows of 16: a(row) + a(row + 1); odd rows: b(row - 1) + b(row)
    const u32x2 s = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b), false, false);
    uint32_t x = s.x, y = s.y;
    asm volatile("" : "+v"(x), "+v"(y));
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
  };
  const uint32_t j = lane >> 4;
  float v;
  if constexpr (MROWS >= 3) {
    const float t01 = fold32(acc[0], acc[1]), t23 = fold32(acc[2], MROWS > 3 ? acc[MROWS > 3 ? 3 : 0] : 0.0f);
    v = fold16(t01, t23);
    *row = ((j & 1u) << 1) | (j >> 1);
    *writer = (lane & 15u) < 4u;
  } else if constexpr (MROWS == 2) {
    const float t = fold32(acc[0], acc[1]);  // lanes 0..31: row 0, lanes 32..63: row 1
    v = fold16(t, twin(t));
    *row = j >> 1;
    *writer = (lane & 31u) < 4u;
  } else {
    const float t = fold32(acc[0], twin(acc[0]));
    v = fold16(t, twin(t));
    *row = 0;
    *writer = lane < 4u;
  }
  v += dpp_move<kRowRor4>(v);
  v += dpp_move<kRowRor8>(v);
  return v;
}

// ---- one activation row: integer digits on the int8 matrix instruction ----
// With a single activation row the four A rows of v_mfma_i32_4x4x4_16B_i8 hold the base-128
// digits of the activations instead of fp16 halves: x, scaled per 32-element block by a power of
// two to |x| < 2^20 and rounded to an integer, is d0 + 128 d1 + 16384 d2 with d0, d1 in
// [0, 127] and d2 in [-64, 64] -- three int8 rows (the fourth is not used).  The B operand is
// then the nibbles as bytes (two mask operations per four weights instead of seven for eight) or,
// for Q8, the weight bytes as they are; the products are exact integers and the three digit sums
// are put together with two shift-adds.  The vector ALU work per block drops by a third, which
// is what bounds the Q4 kernel when the engine clock is low.
// A block's image is 128 bytes: Q4 [plane i][MFMA 0..7] dwords (MFMA 2c holds elements 8c + 0, 2,
// 4, 6 and MFMA 2c + 1 elements 8c + 1, 3, 5, 7, as the two nibble masks deliver them); Q8
// [half][plane i][MFMA 0..3] dwords in natural order.

// eight scaled activations -> their three digit planes, four bytes per dword: lo[i], hi[i] hold
// plane i of elements (e0, e1, e2, e3) and (e4, e5, e6, e7) of the given order
__device__ __forceinline__ void make_digits(const float (&x)[8], const int (&order)[8], uint32_t (&lo)[3], uint32_t (&hi)[3], int* sum) {
  int v[8];
  int s = 0;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    v[e] = (int)__builtin_rintf(x[e]);
    s += v[e];
  }
  *sum = s;
#pragma unroll
  for (int i = 0; i < 3; i++) {
    uint32_t d[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int val = v[order[e]];
      d[e] = i == 0 ? (uint32_t)val & 127u : i == 1 ? ((uint32_t)val >> 7) & 127u : (uint32_t)(val >> 14) & 255u;
    }
    lo[i] = d[0] | (d[1] << 8) | (d[2] << 16) | (d[3] << 24);
    hi[i] = d[4] | (d[5] << 8) | (d[6] << 16) | (d[7] << 24);
  }
}

// Power of two that brings a block's largest magnitude below 2^12 (1 if the block
// is all zero, tiny or not finite).  *inv gets the reciprocal.  A finite magnitude of 2^100 or
// more is not rescaled either, and the truncating fp16 conversion would clamp it to 65504: its
// *inv is a NaN, so that the block's sums come out non-finite instead of finite and wrong.
__device__ __forceinline__ float block_scale(float amax, float* inv) {
  const uint32_t amax_bits = __builtin_bit_cast(uint32_t, amax);
  const int e = (int)(amax_bits >> 23) - 127;  // floor(log2(amax)) for normal values
  if (amax_bits == 0 || e >= 100 || e <= -100) {
    *inv = (e >= 100 && e < 128) ? __builtin_nanf("") : 1.0f;
    return 1.0f;
  }
  const int sh = 11 - e;  // amax * 2^sh in [2^11, 2^12)
  *inv = __builtin_bit_cast(float, (uint32_t)(127 - sh) << 23);
  return __builtin_bit_cast(float, (uint32_t)(127 + sh) << 23);
}

}  // namespace
}  // namespace mgn
