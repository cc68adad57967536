// Operand helpers shared by the kernels built on v_mfma_f32_16x16x32_f16: how raw quants become
// the instruction's B operand, how f32 activations are scaled before they are split into fp16
// pairs, and the row exchanges that bring a lane's 16-byte loads into operand order.
#pragma once
#include "kernels_common.hip.h"

namespace mgn {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half8 as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const u32x4_t v = {a, b, c, d};
  return __builtin_bit_cast(half8, v);
}
__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ float half_lo(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[0]; }
__device__ __forceinline__ float half_hi(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[1]; }

// one dword of nibbles -> B operand (8 fp16): (n0,n4),(n1,n5),(n2,n6),(n3,n7), each n * 2^-20.
// SPLIT: the even nibbles stay in bits 0-3 of their halves, n * 2^-24 (two shifts fewer); the
// activations they meet are stored times 16 in the image.
template <bool SPLIT>
__device__ __forceinline__ half8 nibbles_to_operand(uint32_t wd) {
  if constexpr (SPLIT) {
    const uint32_t hi = wd >> 8;
    return as_half8(wd & 0x000F000Fu, wd & 0x00F000F0u, hi & 0x000F000Fu, hi & 0x00F000F0u);
  }
  return as_half8((wd << 4) & 0x00F000F0u, wd & 0x00F000F0u, (wd >> 4) & 0x00F000F0u, (wd >> 8) & 0x00F000F0u);
}
// two dwords of int8 -> B operand: (b0,b1),(b2,b3),(b4,b5),(b6,b7), each (q + 128) * 2^-24
__device__ __forceinline__ half8 bytes_to_operand(uint32_t w0, uint32_t w1) {
  const uint32_t u0 = w0 ^ 0x80808080u, u1 = w1 ^ 0x80808080u;
  return as_half8(__builtin_amdgcn_perm(0u, u0, 0x0c010c00u), __builtin_amdgcn_perm(0u, u0, 0x0c030c02u),
                  __builtin_amdgcn_perm(0u, u1, 0x0c010c00u), __builtin_amdgcn_perm(0u, u1, 0x0c030c02u));
}

// Power of two that brings a row slice's largest magnitude into [2^TOP, 2^(TOP+1)) (1 if the
// slice is all zero or tiny).  *inv gets the reciprocal.  A slice that holds an infinity or a
// magnitude of 2^100 and more is not rescaled and its reciprocal is a NaN: the truncating fp16
// conversion would clamp such values to 65504 and the row would come out finite and wrong, so
// the row's sums over that slice are made non-finite instead (the f32 arithmetic of the
// reference overflows or loses all precision at that magnitude).
template <int TOP>
__device__ __forceinline__ float slice_scale(float amax, float* inv) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, amax);
  const int e = (int)(bits >> 23) - 127;  // floor(log2(amax)) for normal values
  if (bits == 0 || e <= -100) {
    *inv = 1.0f;
    return 1.0f;
  }
  if (e >= 100) {
    *inv = __builtin_nanf("");
    return 1.0f;
  }
  const int sh = TOP - e;
  *inv = __builtin_bit_cast(float, (uint32_t)(127 - sh) << 23);
  return __builtin_bit_cast(float, (uint32_t)(127 + sh) << 23);
}

// Lanes (c, g), c = lane % 16, g = lane / 16: component j of lane (c, g) <- component g of lane (c, j)
__device__ __forceinline__ void transpose_rows(u32x4_t& v) {
  u32x2_t s = __builtin_amdgcn_permlane32_swap(v.x, v.z, false, false);
  v.x = s.x, v.z = s.y;
  s = __builtin_amdgcn_permlane32_swap(v.y, v.w, false, false);
  v.y = s.x, v.w = s.y;
  s = __builtin_amdgcn_permlane16_swap(v.x, v.y, false, false);
  v.x = s.x, v.y = s.y;
  s = __builtin_amdgcn_permlane16_swap(v.z, v.w, false, false);
  v.z = s.x, v.w = s.y;
}
// odd rows of (x, y) <-> even rows of (z, w)
__device__ __forceinline__ void swap_row_pairs(u32x4_t& v) {
  u32x2_t s = __builtin_amdgcn_permlane16_swap(v.x, v.z, false, false);
  v.x = s.x, v.z = s.y;
  s = __builtin_amdgcn_permlane16_swap(v.y, v.w, false, false);
  v.y = s.x, v.w = s.y;
}

}  // namespace
}  // namespace mgn
