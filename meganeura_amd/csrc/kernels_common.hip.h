// Device helpers shared by the kernel translation units (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

#include "mgn_internal.h"

namespace mgn {

// IEEE half bits -> float.  v_cvt_f32_f16 keeps half subnormals (the f16
// denormal mode of a HIP kernel is "preserve"), matching half::f16::to_f32
// (src/runtime.rs:2122-2123), not the shader's flush-to-zero decoder
// (src/codegen.rs:739-746).
__device__ __forceinline__ float half_bits_to_float(uint32_t bits) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Streaming (read-once) loads: the weight is far larger than what is reused.
__device__ __forceinline__ uint4 stream_load_u128(const void* p) {
  const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint32_t stream_load_u32(const void* p) {
  return __builtin_nontemporal_load((const uint32_t*)p);
}
__device__ __forceinline__ uint16_t stream_load_u16(const void* p) {
  return __builtin_nontemporal_load((const uint16_t*)p);
}

// Unary operations applied to a finished output element, first to last, four bits each
// (mgn_unary; 0 ends the chain): compile.rs:915-1035 fuse_epilogues with the formulas of
// codegen.rs:62-100.  The chain is the same for every element, so the branches are uniform.
__device__ __forceinline__ float apply_epilogue(float v, uint32_t ops) {
  while (ops != 0) {
    switch (ops & 15u) {
      case MGN_UNARY_RELU: v = fmaxf(v, 0.0f); break;
      case MGN_UNARY_SIGMOID: v = 1.0f / (1.0f + expf(-v)); break;
      case MGN_UNARY_NEG: v = -v; break;
      case MGN_UNARY_SILU: v = v / (1.0f + expf(-v)); break;
      default: break;
    }
    ops >>= 4;
  }
  return v;
}

// Byte N of a word as float: the compiler selects v_cvt_f32_ubyteN for these.
__device__ __forceinline__ float ubyte0(uint32_t v) { return (float)(v & 0xFFu); }
__device__ __forceinline__ float ubyte1(uint32_t v) { return (float)((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ubyte2(uint32_t v) { return (float)((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ubyte3(uint32_t v) { return (float)(v >> 24); }

// One DPP move: lane i receives src from the lane the control word selects.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
  return __builtin_bit_cast(float, r);
}

constexpr int kDppQuadXor1 = 0xB1;     // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

// Sum over aligned groups of WIDTH consecutive lanes (WIDTH a power of two up to
// 64); every lane of a group ends with the group's sum.
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
  if constexpr (WIDTH >= 2) v += dpp_move<kDppQuadXor1>(v);
  if constexpr (WIDTH >= 4) v += dpp_move<kDppQuadXor2>(v);
  if constexpr (WIDTH >= 8) v += dpp_move<kDppRowHalfMirror>(v);
  if constexpr (WIDTH >= 16) v += dpp_move<kDppRowMirror>(v);
  if constexpr (WIDTH >= 32) v += __shfl_xor(v, 16, 64);
  if constexpr (WIDTH >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// src/shaders/swiglu_concat.wgsl:20-32: silu(gate) * up with sig = 1 / (1 + exp(-gate)).
// The hardware's exp2 and reciprocal (1 ulp each) instead of the library's expf and an IEEE
// division: six instructions instead of about thirty.  Every workgroup of a fused launch
// evaluates this for all of K, so it is on the path of every column: 14336 x 4096 at one row
// 10.9 -> 9.9 us.  exp(-gate) overflowing to infinity gives sig = 0 as in the plain formula.
__device__ __forceinline__ float swiglu_act(float gate, float up) {
  const float e = __builtin_amdgcn_exp2f(gate * -1.4426950408889634f);
  const float sig = __builtin_amdgcn_rcpf(1.0f + e);
  return gate * sig * up;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for
// every outstanding global load of the wave (its fences cover global memory),
// which would stall a kernel that keeps weight loads in flight across the barrier.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Kernels that use more than 64 KB of dynamic LDS need the limit raised once per kernel and
// per device (the attribute belongs to the device's copy of the function).  `done` is a
// per-kernel bit set over device ordinals.
template <typename Kernel>
inline int enable_big_lds(Kernel kern, int device, std::atomic<uint64_t>& done) {
  const uint64_t bit = 1ull << (device & 63);
  if (done.load(std::memory_order_acquire) & bit) return 0;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e != hipSuccess) return (int)e;
  done.fetch_or(bit, std::memory_order_release);
  return 0;
}

#define MGN_HIP_LAUNCH_CHECK()                      \
  do {                                              \
    hipError_t e__ = hipGetLastError();             \
    if (e__ != hipSuccess) return (int)e__;         \
  } while (0)

}  // namespace mgn
