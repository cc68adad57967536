// Tiled dequant-GEMM on the matrix cores: C[M,N] = A[M,K] x W (+ D) for M >= 3
// (skinny decode batches with f32 activations, and fp16-activation prefill).
//
// The reference runs every quantized matmul with M > 1 through its 64x64x32 tiled
// shader, dequantizing each weight element on load and multiplying on the scalar
// ALUs (src/shaders/matmul.wgsl, src/codegen.rs:748-805), and keeps quantized
// weights off its tensor-core path (src/runtime.rs:1634).  Here the raw quants are
// the MFMA operand and the block scale is applied to the accumulators:
//
//   v_mfma_f32_32x32x16_f16, wave tile = 32 activation rows x 32 weight columns.
//   B operand: lane (c, g), c = lane%32, g = lane/32, holds 8 weights of column c:
//     a lane loads one whole quant block (column c, K block kb0+g: one 128-bit load)
//     and v_permlane32_swap hands the partner lane the half it needs, so after two
//     swaps the wave holds, for both K blocks, the k-slices the instruction wants.
//     Nibbles are masked to fp16 bits 4-7 (n * 2^-20, exact; see the GEMV kernel for
//     why not bits 0-3), Q8 bytes (q + 128) to bits 0-7.
//   A operand: the activations, re-laid once per workgroup and K chunk into LDS in
//     exactly the per-lane order the instruction reads (consecutive lanes read
//     consecutive 16 bytes).  f32 activations are split hi + lo into two fp16 rows
//     (rows r and r+16 of the tile; the two partial results sit in the same lane
//     and are added at the end), so a tile carries 16 real rows; fp16 activations
//     fill all 32 rows.
//   Per quant block: two MFMAs (K = 32) into a fresh accumulator D, then
//     acc += d * D on the vector ALU (16 FMAs per lane).  The format's additive part
//     (m * sum(x) for Q4, -128 * scale * sum(x) for Q8's byte bias) is one more MFMA
//     per step that accumulates straight into acc: its A operand is the block's
//     mean activation (hi, lo), its B operand 32*m taken from the scale|min word.
//     Adding both parts of a block into the same accumulator within a step keeps
//     the running sum small even when the two parts are individually large.
//
// Work split: grid.y = row tiles; a workgroup owns `wnc` column tiles and splits
// every 32-block K chunk `ksc` ways among its waves; partial tiles meet in LDS.
#include <algorithm>

#include "kernels_common.hip.h"

namespace mgn {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kChunkBlocks = 32;  // K blocks staged in LDS at a time (1024 k)
constexpr int kAhead = 3;         // weight blocks in flight per lane ahead of the one in use

__device__ __forceinline__ half8 as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const u32x4_t v = {a, b, c, d};
  return __builtin_bit_cast(half8, v);
}
__device__ __forceinline__ half8 as_half8(uint4 v) { return as_half8(v.x, v.y, v.z, v.w); }

__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ float half_lo(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[0]; }
__device__ __forceinline__ float half_hi(uint32_t p) { return (float)__builtin_bit_cast(half2_t, p)[1]; }

// exchange between lane l and lane l+32: a' = (a.lo | b.lo), b' = (a.hi | b.hi)
__device__ __forceinline__ void swap32(uint32_t& a, uint32_t& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}

template <int FMT>
struct RawBlk;
template <>
struct RawBlk<MGN_FMT_Q4> {
  uint4 q;
  uint32_t meta;
  __device__ __forceinline__ void load(const WeightView& w, size_t b) {
    q = stream_load_u128((const uint4*)w.quants + b);
    meta = stream_load_u32((const uint32_t*)w.meta + b);
  }
};
template <>
struct RawBlk<MGN_FMT_Q8> {
  uint4 q0, q1;
  uint32_t meta;
  __device__ __forceinline__ void load(const WeightView& w, size_t b) {
    q0 = stream_load_u128((const uint4*)w.quants + b * 2);
    q1 = stream_load_u128((const uint4*)w.quants + b * 2 + 1);
    meta = stream_load_u16((const uint16_t*)w.meta + b);
  }
};

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

// LDS per workgroup:
//   aimg[(lb * 2 + h) * 64 + lane]  (uint4): A operand of the MFMA that covers k = 16h..16h+15
//                                   of local block lb, for A lane `lane` = row + 32 * g
//   simg[(lb / 2) * 64 + lane]      (uint4): A operand of the step's additive MFMA; lanes < 32 hold
//                                   (mean_hi, mean_lo) of blocks 2p and 2p+1 in the first two dwords,
//                                   everything else stays zero
// The element order inside an A operand follows the B side: Q4 pairs k with k+4, Q8 is natural.
template <int FMT>
__device__ __forceinline__ void order_for_operand(const float (&x)[8], float (&p)[8]) {
  if constexpr (FMT == MGN_FMT_Q4) {
    p[0] = x[0], p[1] = x[4], p[2] = x[1], p[3] = x[5], p[4] = x[2], p[5] = x[6], p[6] = x[3], p[7] = x[7];
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) p[i] = x[i];
  }
}

// grid = (column-tile groups, row tiles).  blockDim.x = 64 * ksc * wnc.
// SPC = steps per chunk per wave = kChunkBlocks / (2 * ksc); a step is two K blocks.
template <int FMT, bool F32A, int SPC>
__global__ __launch_bounds__(1024) void gemm_mfma_kernel(WeightView w, const void* __restrict__ a_any,
                                                         const float* __restrict__ dres, float* __restrict__ c,
                                                         uint32_t m, uint32_t ksc) {
  constexpr int ROWS = F32A ? 16 : 32;           // real rows per tile
  constexpr int NI = F32A ? 8 : 16;              // result registers per lane
  constexpr int TPT = F32A ? 4 : 8;              // staging tasks per thread per chunk (>= 512 threads)
  constexpr int NTASK = ROWS * kChunkBlocks * 4;  // one task = 8 consecutive k of one row
  constexpr float kOpScale = FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f;
  extern __shared__ uint4 lds4[];
  uint4* aimg = lds4;
  uint4* simg = lds4 + kChunkBlocks * 2 * 64;
  float* red = (float*)lds4;  // reused after the K loop: [wave][NI][64]

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t nwaves = blockDim.x >> 6, wnc = nwaves / ksc;
  const uint32_t ks = wave % ksc, wn = wave / ksc;
  const uint32_t cl = lane & 31, g = lane >> 5;
  const uint32_t bpc = w.k / 32;
  const uint32_t n_tiles = (w.n + 31) / 32;
  const uint32_t col_tile = blockIdx.x * wnc + wn;
  const uint32_t n = col_tile * 32 + cl;
  const bool n_ok = col_tile < n_tiles && n < w.n;
  const uint32_t row0 = blockIdx.y * ROWS;
  const uint32_t zero_block = bpc * w.n;
  const uint32_t nchunks = (bpc + kChunkBlocks - 1) / kChunkBlocks;
  const uint32_t split_first = ks * (2 * SPC);  // this wave's first local block in every chunk

  // the additive operands' unused slots must read as zero for the whole kernel
  for (uint32_t t = tid; t < (kChunkBlocks / 2) * 64; t += blockDim.x) simg[t] = make_uint4(0, 0, 0, 0);
  lds_barrier();

  floatx16 acc;
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = 0.0f;

  for (uint32_t chunk = 0; chunk < nchunks; chunk++) {
    const uint32_t kb_chunk = chunk * kChunkBlocks;
    // ---- 1. activation loads for this thread's staging tasks (oldest in the queue) ----
    // task t = (lb * ROWS + r) * 4 + sub, sub = 2h + g: the four tasks of a (row, block) are a lane quad
    uint4 raw[TPT][F32A ? 2 : 1];
#pragma unroll
    for (int tt = 0; tt < TPT; tt++) {
      const uint32_t t = tid + tt * blockDim.x;
      const uint32_t sub = t & 3, r = (t >> 2) % ROWS, lb = (t >> 2) / ROWS;
      const uint32_t row = row0 + r, kb = kb_chunk + lb;
      const bool ok = t < NTASK && row < m && kb < bpc;
      const size_t off = ok ? (size_t)row * w.k + (size_t)kb * 32 + sub * 8 : (size_t)0;
      if constexpr (F32A) {
        const uint4* src = (const uint4*)((const float*)a_any + off);
        raw[tt][0] = src[0];
        raw[tt][1] = src[1];
      } else {
        raw[tt][0] = *(const uint4*)((const _Float16*)a_any + off);
      }
    }
    // ---- 2. first weight blocks of the chunk go out right behind them ----
    RawBlk<FMT> blk[SPC];
    const uint32_t kb_wave = kb_chunk + split_first + g;  // this lane's block in step 0
    const uint32_t wbase = n * bpc + kb_wave;
    auto fetch = [&](int s) {
      const bool ok = n_ok && kb_wave + 2 * s < bpc;
      blk[s].load(w, ok ? wbase + 2 * s : zero_block);
    };
#pragma unroll
    for (int s = 0; s < SPC && s < kAhead; s++) fetch(s);

    // ---- 3. stage the chunk's A operands ----
#pragma unroll
    for (int tt = 0; tt < TPT; tt++) {
      const uint32_t t = tid + tt * blockDim.x;
      if (t < NTASK) {  // whole waves together: NTASK and blockDim.x are multiples of 64
        const uint32_t sub = t & 3, r = (t >> 2) % ROWS, lb = (t >> 2) / ROWS;
        const uint32_t h = sub >> 1, gg = sub & 1;
        const bool ok = row0 + r < m && kb_chunk + lb < bpc;
        float x[8], p[8];
        if constexpr (F32A) {
          const uint4 v0 = raw[tt][0], v1 = raw[tt][1];
          const uint32_t bits[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
          for (int e = 0; e < 8; e++) x[e] = ok ? __builtin_bit_cast(float, bits[e]) : 0.0f;
        } else {
          const uint4 v = raw[tt][0];
          const uint32_t pr[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int e = 0; e < 4; e++) {
            x[2 * e] = ok ? half_lo(pr[e]) : 0.0f;
            x[2 * e + 1] = ok ? half_hi(pr[e]) : 0.0f;
          }
        }
        order_for_operand<FMT>(x, p);
        const uint32_t slot = (lb * 2 + h) * 64 + 32 * gg;
        float s_hi, s_lo = 0.0f;
        if constexpr (F32A) {
          const uint32_t hp[4] = {pack_rtz(p[0], p[1]), pack_rtz(p[2], p[3]), pack_rtz(p[4], p[5]), pack_rtz(p[6], p[7])};
          float res[8], hs = 0.0f;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float f0 = half_lo(hp[e]), f1 = half_hi(hp[e]);
            res[2 * e] = p[2 * e] - f0;
            res[2 * e + 1] = p[2 * e + 1] - f1;
            hs += f0 + f1;
            s_lo += res[2 * e] + res[2 * e + 1];
          }
          s_hi = hs;
          aimg[slot + r] = make_uint4(hp[0], hp[1], hp[2], hp[3]);
          aimg[slot + 16 + r] =
              make_uint4(pack_rtz(res[0], res[1]), pack_rtz(res[2], res[3]), pack_rtz(res[4], res[5]), pack_rtz(res[6], res[7]));
        } else {
          s_hi = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
          aimg[slot + r] = make_uint4(pack_rtz(p[0], p[1]), pack_rtz(p[2], p[3]), pack_rtz(p[4], p[5]), pack_rtz(p[6], p[7]));
        }
        // block mean (sum over the quad's 32 values / 32), split into two fp16
        s_hi += dpp_move<kDppQuadXor1>(s_hi);
        s_hi += dpp_move<kDppQuadXor2>(s_hi);
        if constexpr (F32A) {
          s_lo += dpp_move<kDppQuadXor1>(s_lo);
          s_lo += dpp_move<kDppQuadXor2>(s_lo);
        }
        if (sub == 0) {
          uint32_t* sdst = (uint32_t*)(simg + (lb >> 1) * 64) + (lb & 1);
          const float mean = s_hi * 0.03125f;
          const uint32_t mh = pack_rtz(mean, 0.0f);
          sdst[r * 4] = (mh & 0xFFFFu) | (pack_rtz(mean - half_lo(mh), 0.0f) << 16);
          if constexpr (F32A) {
            const float mean_l = s_lo * 0.03125f;
            const uint32_t ml = pack_rtz(mean_l, 0.0f);
            sdst[(16 + r) * 4] = (ml & 0xFFFFu) | (pack_rtz(mean_l - half_lo(ml), 0.0f) << 16);
          }
        }
      }
    }
    lds_barrier();

    // ---- 4. this wave's steps of the chunk ----
#pragma unroll
    for (int s = 0; s < SPC; s++) {
      if (s + kAhead < SPC) fetch(s + kAhead);
      const RawBlk<FMT>& cur = blk[s];
      const uint32_t lb0 = split_first + 2 * s;  // local index of the step's first block
      uint32_t meta0 = cur.meta, meta1 = cur.meta;
      swap32(meta0, meta1);  // meta0: block lb0 for every lane, meta1: block lb0 + 1
      half8 bop[2][2];       // [block][h]
      if constexpr (FMT == MGN_FMT_Q4) {
        uint32_t r0 = cur.q.x, r1 = cur.q.y, r2 = cur.q.z, r3 = cur.q.w;
        swap32(r0, r1);  // r0: block 0, k 0-7 | 8-15;   r1: block 1, same
        swap32(r2, r3);  // r2: block 0, k 16-23 | 24-31; r3: block 1, same
        bop[0][0] = nibbles_to_operand(r0);
        bop[1][0] = nibbles_to_operand(r1);
        bop[0][1] = nibbles_to_operand(r2);
        bop[1][1] = nibbles_to_operand(r3);
      } else {
        uint32_t r0 = cur.q0.x, r1 = cur.q0.y, r2 = cur.q0.z, r3 = cur.q0.w;
        uint32_t r4 = cur.q1.x, r5 = cur.q1.y, r6 = cur.q1.z, r7 = cur.q1.w;
        swap32(r0, r2);
        swap32(r1, r3);  // (r0, r1): block 0, k 0-7 | 8-15;   (r2, r3): block 1, same
        swap32(r4, r6);
        swap32(r5, r7);  // (r4, r5): block 0, k 16-23 | 24-31; (r6, r7): block 1, same
        bop[0][0] = bytes_to_operand(r0, r1);
        bop[1][0] = bytes_to_operand(r2, r3);
        bop[0][1] = bytes_to_operand(r4, r5);
        bop[1][1] = bytes_to_operand(r6, r7);
      }
#pragma unroll
      for (int t = 0; t < 2; t++) {
        floatx16 dsum;
#pragma unroll
        for (int i = 0; i < 16; i++) dsum[i] = 0.0f;
        const uint4* ap = aimg + ((lb0 + t) * 2) * 64 + lane;
        dsum = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(ap[0]), bop[t][0], dsum, 0, 0, 0);
        dsum = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(ap[64]), bop[t][1], dsum, 0, 0, 0);
        const float dq = half_bits_to_float((t == 0 ? meta0 : meta1) & 0xFFFFu) * kOpScale;
#pragma unroll
        for (int i = 0; i < 16; i++) acc[i] = __fmaf_rn(dq, dsum[i], acc[i]);
      }
      // additive part of both blocks: mean(x) * (32 * m), straight into acc
      uint32_t add0, add1;
      if constexpr (FMT == MGN_FMT_Q4) {
        add0 = __builtin_amdgcn_perm(meta0, meta0, 0x07060706u);  // (m, m) of block 0
        add1 = __builtin_amdgcn_perm(meta1, meta1, 0x07060706u);
        const half2_t k32 = {(_Float16)32.0f, (_Float16)32.0f};
        add0 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, add0) * k32);
        add1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, add1) * k32);
      } else {
        // bytes carry q + 128: take 128 * scale * sum(x) back out
        add0 = __builtin_amdgcn_perm(meta0, meta0, 0x05040504u);  // (scale, scale)
        add1 = __builtin_amdgcn_perm(meta1, meta1, 0x05040504u);
        const half2_t kb = {(_Float16)-4096.0f, (_Float16)-4096.0f};
        add0 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, add0) * kb);
        add1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, add1) * kb);
      }
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(simg[(lb0 >> 1) * 64 + lane]),
                                                    as_half8(add0, add1, add0, add1), acc, 0, 0, 0);
    }
    lds_barrier();  // the next chunk's staging overwrites aimg
  }

  // ---- combine the K splits through LDS, add the residual, store ----
  // D layout: lane -> column lane%32; register i -> tile row 8*(i/4) + 4*(lane/32) + i%4.
  // With f32 activations rows r and r+16 (registers i and i+8) are the hi and lo parts.
  float outv[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) outv[i] = F32A ? acc[i] + acc[i + 8] : acc[i];
#pragma unroll
  for (int i = 0; i < NI; i++) red[(wave * NI + i) * 64 + lane] = outv[i];
  lds_barrier();
  for (uint32_t idx = tid; idx < wnc * NI * 64; idx += blockDim.x) {
    const uint32_t ln = idx & 63, i = (idx >> 6) % NI, tile = idx / (64 * NI);
    const uint32_t row = row0 + 8 * (i >> 2) + 4 * (ln >> 5) + (i & 3);
    const uint32_t col = (blockIdx.x * wnc + tile) * 32 + (ln & 31);
    if (row < m && col < w.n) {
      float v = 0.0f;
      for (uint32_t s = 0; s < ksc; s++) v += red[((tile * ksc + s) * NI + i) * 64 + ln];
      const size_t o = (size_t)row * w.n + col;
      c[o] = dres ? v + dres[o] : v;
    }
  }
}

struct GemmPlan {
  uint32_t ksc, wnc, spc, grid_x, grid_y;
  size_t lds;
};

bool plan_gemm(uint32_t m, uint32_t n, bool f32a, int num_cus, GemmPlan* out) {
  const uint32_t rows = f32a ? 16 : 32;
  GemmPlan p{};
  p.grid_y = (m + rows - 1) / rows;
  if (p.grid_y > 65535) return false;
  const uint32_t n_tiles = (n + 31) / 32;
  // K splits: enough waves for ~8 per CU, in powers of two up to 16
  const uint64_t tiles = (uint64_t)p.grid_y * n_tiles;
  uint32_t ksc = 1;
  while (ksc < 16 && tiles * ksc < (uint64_t)num_cus * 8) ksc *= 2;
  p.ksc = ksc;
  p.spc = kChunkBlocks / (2 * ksc);
  // column tiles per workgroup: as many as fit (the activations are staged once per workgroup),
  // fewer only if that would leave a fifth of the CUs without a workgroup
  uint32_t wnc = std::min<uint32_t>(16 / ksc, n_tiles);
  auto groups = [&](uint32_t v) { return (uint64_t)p.grid_y * ((n_tiles + v - 1) / v); };
  while (wnc > 1 && groups(wnc) * 5 < (uint64_t)num_cus * 4) wnc--;
  // staging assumes at least 512 threads; waves without a column tile only help staging
  wnc = std::max<uint32_t>(wnc, (8 + ksc - 1) / ksc);
  p.wnc = wnc;
  p.grid_x = (n_tiles + wnc - 1) / wnc;
  p.lds = (size_t)(kChunkBlocks * 2 * 64 + (kChunkBlocks / 2) * 64) * 16;
  *out = p;
  return true;
}

template <int FMT, bool F32A, int SPC>
int launch_spc(ihipStream_t* s, const LaunchArgs& x, const GemmPlan& p) {
  auto kern = gemm_mfma_kernel<FMT, F32A, SPC>;
  static bool big_lds_enabled = false;
  if (!big_lds_enabled) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return (int)e;
    big_lds_enabled = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.grid_x, p.grid_y), dim3(64 * p.ksc * p.wnc), p.lds, s, x.w, x.a, x.d, x.c, x.m, p.ksc);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

template <int FMT, bool F32A>
int launch_fa(ihipStream_t* s, const LaunchArgs& x) {
  GemmPlan p;
  if (!plan_gemm(x.m, x.w.n, F32A, x.num_cus, &p)) return (int)hipErrorInvalidValue;
  switch (p.spc) {
    case 16: return launch_spc<FMT, F32A, 16>(s, x, p);
    case 8: return launch_spc<FMT, F32A, 8>(s, x, p);
    case 4: return launch_spc<FMT, F32A, 4>(s, x, p);
    case 2: return launch_spc<FMT, F32A, 2>(s, x, p);
    case 1: return launch_spc<FMT, F32A, 1>(s, x, p);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace

bool gemm_mfma_supported(const LaunchArgs& x) {
  if (x.m == 0) return false;
  GemmPlan p;
  return plan_gemm(x.m, x.w.n, !x.a_is_f16, x.num_cus, &p);
}

int launch_matmul_gemm_mfma(ihipStream_t* s, const LaunchArgs& x) {
  if (x.w.fmt == MGN_FMT_Q4) return x.a_is_f16 ? launch_fa<MGN_FMT_Q4, false>(s, x) : launch_fa<MGN_FMT_Q4, true>(s, x);
  return x.a_is_f16 ? launch_fa<MGN_FMT_Q8, false>(s, x) : launch_fa<MGN_FMT_Q8, true>(s, x);
}

}  // namespace mgn
