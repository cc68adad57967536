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
//   B operand: lane (c, g), c = lane%32, g = lane/32, holds 8 weights of column c.
//     The quants come from memory as whole runs of a column's blocks, are parked in a
//     wave-private LDS slice, and each lane reads back one whole block (column c, K
//     block 2s+g); v_permlane32_swap hands the partner lane the half it needs, so
//     after two swaps the wave holds, for both K blocks of a step, the k-slices the
//     instruction wants.  Nibbles are masked to fp16 bits 4-7 (n * 2^-20, exact; see
//     the GEMV kernel for why not bits 0-3), Q8 bytes (q + 128) to bits 0-7.
//   A operand: the activations, re-laid once per workgroup and K chunk into LDS in
//     exactly the per-lane order the instruction reads (consecutive lanes read
//     consecutive 16 bytes), double-buffered so the next chunk is staged while this
//     one is multiplied.  f32 activations are split hi + lo into two fp16 rows
//     (rows r and r+16 of the tile; the two partial results sit in the same lane
//     and are added at the end), so a tile carries 16 real rows; fp16 activations
//     fill all 32 rows.  f32 activations are not rescaled: |x| must stay below 65504.
//   Per quant block: two MFMAs (K = 32) into a fresh accumulator D, then
//     acc += d * D on the vector ALU (16 FMAs per lane).  The format's additive part
//     (m * sum(x) for Q4, -128 * scale * sum(x) for Q8's byte bias) is one more MFMA
//     per step into a second accumulator: its A operand is the block's activation sum
//     as (mean, sum - 32 mean), its B operand (32 m, m) (or (-4096, -128) * scale) taken
//     from the scale word, so |m| < 2048 and scale < 16 are required.  Both accumulators
//     are f32; their sum is taken once at the end.
//
// Work split: grid.y = row tiles; a workgroup owns `wnc` column tiles; K is cut into
// chunks of 8*ksc blocks which the workgroup walks in order (ksc waves share a chunk),
// and, when there are too few tiles to fill the chip, into `parts` ranges handled by
// different workgroups whose partial tiles the last one to finish adds up in part
// order (deterministic).
#include <algorithm>

#include "kernels_common.hip.h"

namespace mgn {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));


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

// LDS per workgroup, two buffers b = chunk parity (CB = 8 * ksc K blocks per chunk):
//   aimg[b][(lb * 2 + h) * 64 + lane]  (uint4): A operand of the MFMA that covers k = 16h..16h+15
//                                      of local block lb, for A lane `lane` = row + 32 * g
//   simg[b][(lb / 2) * 64 + lane]      (uint4): A operand of a step's additive MFMA; lanes < 32 hold
//                                      (mean, sum - 32 mean) of blocks 2p and 2p+1 in the first two
//                                      dwords, everything else stays zero
// The element order inside an A operand follows the B side: Q4 pairs k with k+4, Q8 is natural.
constexpr int kSteps = 4;  // steps per wave per chunk; a step is two K blocks
// bytes per column of a parked weight slice: 8 blocks + 16 bytes of padding
constexpr int slice_stride(int fmt) { return fmt == MGN_FMT_Q4 ? 8 * 16 + 16 : 8 * 32 + 16; }
typedef uint32_t u32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2_unaligned __attribute__((ext_vector_type(2), aligned(2)));

struct GemmTail {  // arguments first needed in the epilogue
  const float* dres;
  float* c;
  float* scratch;      // [parts][row tiles * ROWS][n] partial results when parts > 1
  uint32_t* counters;  // one arrival counter per (row tile, column group), zero between launches
  uint32_t* range_flag;  // host-visible: set when an f32 activation does not fit the fp16 pair
  uint32_t row_tiles;
  uint32_t epilogue;  // unary operations on the output (apply_epilogue)
};

// B operand pair of a block's additive part from its scale word: (32 c, c) with c = m (Q4: the
// word's high half) or -128 scale (Q8: the low half).  The A side pairs them with the block's mean
// activation and with what the sum has beyond 32 * mean.
template <int FMT>
__device__ __forceinline__ uint32_t additive_pair(uint32_t w) {
  const half2_t h = __builtin_bit_cast(half2_t, w);
  const _Float16 c = h[FMT == MGN_FMT_Q4 ? 1 : 0];
  const half2_t pair = {c, c};
  const half2_t weights = FMT == MGN_FMT_Q4 ? half2_t{(_Float16)32.0f, (_Float16)1.0f} : half2_t{(_Float16)-4096.0f, (_Float16)-128.0f};
  return __builtin_bit_cast(uint32_t, pair * weights);
}

template <int FMT>
__device__ __forceinline__ uint4 f16_operand(uint4 v) {
  if constexpr (FMT == MGN_FMT_Q4) {
    return make_uint4(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                      __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
  } else {
    return v;
  }
}

// grid = (parts, column groups, row tiles); blockDim.x = 64 * ksc * wnc, ksc in {1, 2}.
// A workgroup owns wnc column tiles of one row tile and K blocks
// [part * nch * CB, (part + 1) * nch * CB); within a chunk wave (ks, wn) takes the
// 8 blocks starting at 8 * ks.  While a chunk is being multiplied, the next chunk's
// activations are in flight to registers and the weight ring is refilled one chunk ahead.
// TPT = staging tasks per thread per chunk (one task = 8 consecutive k of one row).
// The leading scalar arguments are the ones a wave needs before its first loads; as plain
// scalars (not struct members) they can be handed over in registers at wave launch.
// AM: how the activations arrive and sit in the tile.  0: fp16, 32 rows per tile.  1: f32 split
// hi + lo into two fp16 rows of the tile (rows r and r + 16): 16 real rows per tile, one MFMA
// pair per block -- the form for M <= 16.  2: f32 split hi + lo into two A operands that are
// multiplied into the same accumulator: 32 real rows per tile at twice the MFMAs per block but
// the same vector-ALU work, which is what the kernel is bound by -- the form for M > 16.
template <int FMT, int AM, int TPT>
__global__ __launch_bounds__(512) void gemm_mfma_kernel(const void* __restrict__ a_arg, const void* __restrict__ meta_arg,
                                                        const void* __restrict__ quants_arg, uint32_t m_arg, uint32_t ksc_arg,
                                                        uint32_t wnc_arg, uint32_t nch_arg, uint32_t k_arg, uint32_t n_arg,
                                                        uint32_t parts_arg, uint32_t colgroups_arg, GemmTail tail) {
  // one view over both argument groups (the compiler keeps it in scalar registers)
  struct {
    WeightView w;
    const void* a;
    const float* dres;
    float* c;
    float* scratch;
    uint32_t* counters;
    uint32_t m, ksc, wnc, nch, parts, colgroups;
  } g;
  g.w.meta = meta_arg, g.w.quants = quants_arg, g.w.k = k_arg, g.w.n = n_arg, g.w.fmt = FMT;
  g.a = a_arg, g.m = m_arg, g.ksc = ksc_arg, g.wnc = wnc_arg, g.nch = nch_arg;
  g.parts = parts_arg, g.colgroups = colgroups_arg;
  g.dres = tail.dres, g.c = tail.c, g.scratch = tail.scratch, g.counters = tail.counters;
  constexpr bool F32A = AM != 0;
  constexpr bool CHAIN = AM == 2;
  constexpr int ROWS = AM == 1 ? 16 : 32;  // real rows per tile
  constexpr int NI = AM == 1 ? 8 : 16;     // result registers per lane
  constexpr int HL = CHAIN ? 2 : 1;        // A operands per (block, k half): hi and lo
  constexpr float kOpScale = FMT == MGN_FMT_Q4 ? 1048576.0f : 16777216.0f;
  extern __shared__ uint4 lds4[];
  const WeightView& w = g.w;
  const uint32_t ksc = g.ksc, wnc = g.wnc;
  const uint32_t cb = 8 * ksc;                  // blocks per chunk
  const uint32_t a_stride = cb * 2 * HL * 64;   // uint4 per aimg buffer
  const uint32_t s_stride = (cb / 2) * 64;      // uint4 per simg buffer
  uint4* const aimg = lds4;
  uint4* const simg = lds4 + 2 * a_stride;
  float* const red = (float*)lds4;  // reused after the K loop: [wn][NI][64]

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t ks = wave & (ksc - 1), wn = wave >> (ksc - 1);  // ksc is 1 or 2
  const uint32_t cl = lane & 31, gh = lane >> 5;
  const uint32_t bpc = w.k / 32;
  const uint32_t n_tiles = (w.n + 31) / 32;
  const uint32_t cg = blockIdx.y, part = blockIdx.x;
  const uint32_t nthreads = 64 * ksc * wnc;  // = blockDim.x
  const uint32_t col_tile = cg * wnc + wn;
  const uint32_t n = col_tile * 32 + cl;
  const bool n_ok = col_tile < n_tiles && n < w.n;
  const uint32_t row0 = blockIdx.z * ROWS;
  const uint32_t zero_block = bpc * w.n;
  const uint32_t chunk0 = part * g.nch;  // first chunk of this workgroup

  // ---- per-thread staging tasks: task t = (lb * ROWS + r) * 4 + sub, sub = 2h + g ----
  uint32_t t_lb[TPT], t_slot[TPT], t_r[TPT];
  size_t t_off[TPT];
  bool t_rowok[TPT], t_live[TPT];
#pragma unroll
  for (int tt = 0; tt < TPT; tt++) {
    const uint32_t t = tid + tt * nthreads;
    const uint32_t sub = t & 3, r = (t >> 2) % ROWS, lb = (t >> 2) / ROWS;
    t_lb[tt] = lb;
    t_r[tt] = r;
    t_live[tt] = lb < cb;
    t_rowok[tt] = t_live[tt] && row0 + r < g.m;
    t_off[tt] = t_rowok[tt] ? (size_t)(row0 + r) * w.k + (size_t)lb * 32 + sub * 8 : (size_t)0;
    t_slot[tt] = (lb * 2 + (sub >> 1)) * HL * 64 + 32 * (sub & 1) + r;
  }
  uint4 raw[TPT][F32A ? 2 : 1];
  auto load_a = [&](uint32_t chunk) {  // unconditional loads; dead tasks re-read element 0
    const uint32_t kb_chunk = chunk * cb;
#pragma unroll
    for (int tt = 0; tt < TPT; tt++) {
      const bool ok = t_rowok[tt] && kb_chunk + t_lb[tt] < bpc;
      const size_t off = ok ? t_off[tt] + (size_t)kb_chunk * 32 : (size_t)0;
      if constexpr (F32A) {
        const uint4* src = (const uint4*)((const float*)g.a + off);
        raw[tt][0] = src[0];
        raw[tt][1] = src[1];
      } else {
        raw[tt][0] = *(const uint4*)((const _Float16*)g.a + off);
      }
    }
  };
  auto stage = [&](uint32_t chunk, uint32_t buf) {
    const uint32_t kb_chunk = chunk * cb;
    uint4* const ab = aimg + buf * a_stride;
    uint32_t* const sb = (uint32_t*)(simg + buf * s_stride);
#pragma unroll
    for (int tt = 0; tt < TPT; tt++) {
      const bool ok = t_rowok[tt] && kb_chunk + t_lb[tt] < bpc;
      const uint32_t lb = t_lb[tt], r = t_r[tt];
      float s_hi, s_lo = 0.0f;
      uint4 op_hi, op_lo;
      if constexpr (F32A) {
        const uint4 v0 = raw[tt][0], v1 = raw[tt][1];
        const uint32_t bits[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
        float x[8], p[8];
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = ok ? __builtin_bit_cast(float, bits[e]) : 0.0f;
        if constexpr (FMT == MGN_FMT_Q4) {
          p[0] = x[0], p[1] = x[4], p[2] = x[1], p[3] = x[5], p[4] = x[2], p[5] = x[6], p[6] = x[3], p[7] = x[7];
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++) p[e] = x[e];
        }
        // hi + lo covers |x| < 65504 only (the conversion saturates silently beyond): say so
        const float amax = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                                 fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
        if (!(amax < 65504.0f) && tail.range_flag) *tail.range_flag = 1u;
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
        op_hi = make_uint4(hp[0], hp[1], hp[2], hp[3]);
        op_lo = make_uint4(pack_rtz(res[0], res[1]), pack_rtz(res[2], res[3]), pack_rtz(res[4], res[5]), pack_rtz(res[6], res[7]));
      } else {
        uint4 v = raw[tt][0];
        if (!ok) v = make_uint4(0, 0, 0, 0);
        const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
        s_hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v.x), ones, 0.0f, false);
        s_hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v.y), ones, s_hi, false);
        s_hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v.z), ones, s_hi, false);
        s_hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, v.w), ones, s_hi, false);
        op_hi = f16_operand<FMT>(v);
      }
      // block sum (over the lane quad's 32 values)
      s_hi += dpp_move<kDppQuadXor1>(s_hi);
      s_hi += dpp_move<kDppQuadXor2>(s_hi);
      if constexpr (F32A) {
        s_lo += dpp_move<kDppQuadXor1>(s_lo);
        s_lo += dpp_move<kDppQuadXor2>(s_lo);
      }
      if (t_live[tt]) {
        ab[t_slot[tt]] = op_hi;
        if constexpr (F32A) ab[t_slot[tt] + (CHAIN ? 64 : 16)] = op_lo;  // lo: an operand of its own, or rows 16-31
        if ((tid & 3) == 0) {
          uint32_t* sdst = sb + (lb >> 1) * 256 + (lb & 1);
          // the sum as 32 * mean + rest: the mean alone, as hi + lo, would lose the sum's low bits
          // where fp16 runs out of exponent (activations around 1e-3 and below)
          const float sum = CHAIN ? s_hi + s_lo : s_hi;
          const uint32_t mh = pack_rtz(sum * 0.03125f, 0.0f);
          sdst[r * 4] = (mh & 0xFFFFu) | (pack_rtz(sum - 32.0f * half_lo(mh), 0.0f) << 16);
          if constexpr (AM == 1) {
            const uint32_t ml = pack_rtz(s_lo * 0.03125f, 0.0f);
            sdst[(16 + r) * 4] = (ml & 0xFFFFu) | (pack_rtz(s_lo - 32.0f * half_lo(ml), 0.0f) << 16);
          }
        }
      }
    }
  };

  const uint32_t lb_wave = ks * (2 * kSteps);  // this wave's first local block in every chunk
  // ---- weight slices: a wave's 8 blocks x 32 columns of a chunk ----
  // Loaded as whole runs of a column's blocks (128 bytes of nibbles or 256 bytes of
  // int8: 8 or 16 lanes per column, NL loads), parked in a wave-private LDS area with
  // a padded column stride, and read back one block per lane (column lane%32, block
  // 2s + lane/32) for step s.  Loading in the operand's own lane order instead would
  // take 32 bytes from each cache line at a time and fetch every line several times.
  // The scale words of the slice are one load per lane (4 blocks), broadcast across
  // the wave halves.
  constexpr int QB = FMT == MGN_FMT_Q4 ? 16 : 32;  // quant bytes per block
  constexpr int NL = QB / 4;                       // 16-byte loads per lane per slice
  constexpr int LPC = QB / 2;                      // lanes per column in one load
  constexpr int CPL = 64 / LPC;                    // columns per load
  constexpr int kStride = slice_stride(FMT);
  uint4 wq[NL];
  uint4 wm;  // Q4: scale|min words of 4 blocks; Q8: x, y = four fp16 scales
  uint8_t* const wbuf = (uint8_t*)(lds4 + 2 * a_stride + 2 * s_stride) + wave * (32 * kStride);
  auto fetch_slice = [&](uint32_t chunk, bool chunk_ok) {
    const uint32_t kb0 = chunk * cb + lb_wave;
    const bool tile_ok = chunk_ok && col_tile < n_tiles;
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const uint32_t nn = col_tile * 32 + CPL * j + lane / LPC, piece = lane % LPC;
      const uint32_t kb = kb0 + piece / (QB / 16);
      const bool ok = tile_ok && nn < w.n && kb < bpc;
      const size_t idx = ok ? ((size_t)nn * bpc + kb0) * (QB / 16) + piece : (size_t)zero_block * (QB / 16);
      wq[j] = stream_load_u128((const uint4*)w.quants + idx);
    }
    // blocks past the end of the column carry zero quants; their scale words must be zero too
    const uint32_t kbm = kb0 + 4 * gh;
    const bool okm = tile_ok && n_ok && kbm < bpc;
    const bool ok1 = okm && kbm + 1 < bpc, ok2 = okm && kbm + 2 < bpc, ok3 = okm && kbm + 3 < bpc;
    if constexpr (FMT == MGN_FMT_Q4) {
      const u32x4_unaligned v =
          __builtin_nontemporal_load((const u32x4_unaligned*)((const uint32_t*)w.meta + (okm ? n * bpc + kbm : zero_block)));
      wm = make_uint4(okm ? v.x : 0u, ok1 ? v.y : 0u, ok2 ? v.z : 0u, ok3 ? v.w : 0u);
    } else {
      const u32x2_unaligned v =
          __builtin_nontemporal_load((const u32x2_unaligned*)((const uint16_t*)w.meta + (okm ? n * bpc + kbm : zero_block)));
      wm = make_uint4(okm ? v.x & 0xFFFFu : 0u, ok1 ? v.x >> 16 : 0u, ok2 ? v.y & 0xFFFFu : 0u, ok3 ? v.y >> 16 : 0u);
    }
  };
  uint32_t mb[8];  // scale words of the slice's 8 blocks, the same in every lane
  auto park_slice = [&]() {
#pragma unroll
    for (int j = 0; j < NL; j++) *(uint4*)(wbuf + (CPL * j + lane / LPC) * kStride + (lane % LPC) * 16) = wq[j];
    const uint32_t mm[4] = {wm.x, wm.y, wm.z, wm.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
      uint32_t lo = mm[e], hi = mm[e];
      swap32(lo, hi);  // lo: lower half's word (block e) in every lane, hi: upper half's (block 4 + e)
      mb[e] = lo;
      mb[4 + e] = hi;
    }
  };

  load_a(chunk0);
  fetch_slice(chunk0, true);
  // the additive operands' unused slots must read as zero for the whole kernel
  for (uint32_t t = tid; t < 2 * s_stride; t += nthreads) simg[t] = make_uint4(0, 0, 0, 0);
  lds_barrier();
  stage(chunk0, 0);
  lds_barrier();

  floatx16 acc, acc2;  // scaled quant sums (vector ALU), additive parts (MFMA)
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = acc2[i] = 0.0f;

  for (uint32_t c = 0; c < g.nch; c++) {
    const uint32_t chunk = chunk0 + c, buf = c & 1;
    const bool more = c + 1 < g.nch;
    load_a(more ? chunk + 1 : chunk);  // next chunk's activations travel while this one is multiplied
    const uint4* const ab = aimg + buf * a_stride;
    const uint4* const sb = simg + buf * s_stride;
    park_slice();
    fetch_slice(chunk + 1, more);
    // Software pipeline over the steps: the MFMAs of step s + 1 are issued before the vector
    // ALU scales the results of step s, so the matrix cores work through one step while the
    // ALU finishes the previous one.  The scheduling fences keep the compiler from undoing it.
    floatx16 dsum[2][2];  // [step parity][block]
    auto issue_step = [&](int s) {
      const uint32_t lb0 = lb_wave + 2 * s;  // local index of the step's first block
      const uint32_t meta0 = mb[2 * s], meta1 = mb[2 * s + 1];  // block lb0, block lb0 + 1
      half8 bop[2][2];                                            // [block][h]
      const uint4* const wsrc = (const uint4*)(wbuf + cl * kStride + (2 * s + gh) * QB);
      if constexpr (FMT == MGN_FMT_Q4) {
        const uint4 q = wsrc[0];
        uint32_t r0 = q.x, r1 = q.y, r2 = q.z, r3 = q.w;
        swap32(r0, r1);  // r0: block 0, k 0-7 | 8-15;   r1: block 1, same
        swap32(r2, r3);  // r2: block 0, k 16-23 | 24-31; r3: block 1, same
        bop[0][0] = nibbles_to_operand(r0);
        bop[1][0] = nibbles_to_operand(r1);
        bop[0][1] = nibbles_to_operand(r2);
        bop[1][1] = nibbles_to_operand(r3);
      } else {
        const uint4 q0 = wsrc[0], q1 = wsrc[1];
        uint32_t r0 = q0.x, r1 = q0.y, r2 = q0.z, r3 = q0.w;
        uint32_t r4 = q1.x, r5 = q1.y, r6 = q1.z, r7 = q1.w;
        swap32(r0, r2);
        swap32(r1, r3);  // (r0, r1): block 0, k 0-7 | 8-15;   (r2, r3): block 1, same
        swap32(r4, r6);
        swap32(r5, r7);  // (r4, r5): block 0, k 16-23 | 24-31; (r6, r7): block 1, same
        bop[0][0] = bytes_to_operand(r0, r1);
        bop[1][0] = bytes_to_operand(r2, r3);
        bop[0][1] = bytes_to_operand(r4, r5);
        bop[1][1] = bytes_to_operand(r6, r7);
      }
      // additive part of both blocks: (mean(x), sum(x) - 32 mean(x)) x (32 m, m), into its own
      // accumulator so that this MFMA chain and the vector ALU's chain never wait for each other
      // (Q8: bytes carry q + 128, so 128 * scale * sum(x) is taken back out)
      const uint32_t add0 = additive_pair<FMT>(meta0), add1 = additive_pair<FMT>(meta1);
      uint4 aop[2][2], lop[2][2];  // [block][k half]; lop: the low halves' operands (CHAIN)
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const uint4* ap = ab + ((lb0 + t) * 2) * HL * 64 + lane;
        aop[t][0] = ap[0];
        aop[t][1] = ap[HL * 64];
        if constexpr (CHAIN) {
          lop[t][0] = ap[64];
          lop[t][1] = ap[HL * 64 + 64];
        }
      }
      const uint4 sop = sb[(lb0 >> 1) * 64 + lane];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 2; t++) {
        floatx16 z;
#pragma unroll
        for (int i = 0; i < 16; i++) z[i] = 0.0f;
        z = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(aop[t][0]), bop[t][0], z, 0, 0, 0);
        if constexpr (CHAIN) {
          z = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(lop[t][0]), bop[t][0], z, 0, 0, 0);
          z = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(lop[t][1]), bop[t][1], z, 0, 0, 0);
        }
        dsum[s & 1][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(aop[t][1]), bop[t][1], z, 0, 0, 0);
      }
      acc2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(sop), as_half8(add0, add1, add0, add1), acc2, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    };
    auto scale_step = [&](int s) {
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const float dq = half_bits_to_float(mb[2 * s + t] & 0xFFFFu) * kOpScale;
#pragma unroll
        for (int i = 0; i < 16; i++) acc[i] = __fmaf_rn(dq, dsum[s & 1][t][i], acc[i]);
      }
    };
    issue_step(0);
#pragma unroll
    for (int s = 0; s < kSteps; s++) {
      if (s + 1 < kSteps) issue_step(s + 1);
      scale_step(s);
      asm volatile("" : "+v"(acc));  // the scaling stays here, between the two MFMA groups
    }
    if (more) stage(chunk + 1, buf ^ 1);  // the other buffer was last read before the previous barrier
    lds_barrier();
  }

  // ---- combine the two K halves of the workgroup ----
  // D layout: lane -> column lane%32; register i -> tile row 8*(i/4) + 4*(lane/32) + i%4.
  // In the 16-row f32 form rows r and r+16 (registers i and i+8) are the hi and lo parts.
  float outv[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) outv[i] = AM == 1 ? (acc[i] + acc2[i]) + (acc[i + 8] + acc2[i + 8]) : acc[i] + acc2[i];
  if (ksc == 2) {
    if (ks == 1) {
#pragma unroll
      for (int i = 0; i < NI; i++) red[(wn * NI + i) * 64 + lane] = outv[i];
    }
    lds_barrier();
    if (ks == 0) {
#pragma unroll
      for (int i = 0; i < NI; i++) outv[i] += red[(wn * NI + i) * 64 + lane];
    }
  }
  const bool writer = ks == 0 && n_ok;

  if (g.parts > 1) {
    // ---- K parts of other workgroups: the last one to arrive adds them up in part order ----
    // Each XCD has its own L2, so partial tiles travel as device-scope relaxed atomics:
    // write-through stores, complete (in memory) once acknowledged, and L2-coherent loads.
    // No release fence: it would write back this XCD's whole L2 (4 us measured) for the
    // sake of stores that have been written through already.
    const size_t plane = (size_t)tail.row_tiles * ROWS * w.n;  // floats per part
    float* const mine = g.scratch + (size_t)part * plane + (size_t)row0 * w.n + n;
    if (writer) {
#pragma unroll
      for (int i = 0; i < NI; i++)
        __hip_atomic_store(mine + (size_t)(8 * (i >> 2) + 4 * gh + (i & 3)) * w.n, outv[i], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    // every wave waits until its write-through stores have been acknowledged, i.e. have
    // reached memory; the barrier then orders all of them before the count
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t* const flag = (uint32_t*)lds4;
    if (tid == 0) {
      uint32_t* ctr = g.counters + blockIdx.z * g.colgroups + cg;
      const uint32_t seen = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = seen == g.parts - 1;
      if (last) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
      *flag = last ? 1u : 0u;
    }
    __syncthreads();
    if (*flag == 0u) return;
    if (writer) {
      // every part comes from memory, this workgroup's own included: NI loads of a part in
      // flight together, parts added in order
      const float* const base = g.scratch + (size_t)row0 * w.n + n;
      float sum[NI];
#pragma unroll
      for (int i = 0; i < NI; i++) sum[i] = 0.0f;
      constexpr int PB = AM == 1 ? 4 : 2;  // parts in flight together
      for (uint32_t p0 = 0; p0 < g.parts; p0 += PB) {
        float tmp[PB][NI];
#pragma unroll
        for (int j = 0; j < PB; j++) {
          const uint32_t p = p0 + j < g.parts ? p0 + j : g.parts - 1;
#pragma unroll
          for (int i = 0; i < NI; i++)
            tmp[j][i] = __hip_atomic_load(base + p * plane + (size_t)(8 * (i >> 2) + 4 * gh + (i & 3)) * w.n,
                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int j = 0; j < PB; j++) {
          if (p0 + j < g.parts) {
#pragma unroll
            for (int i = 0; i < NI; i++) sum[i] += tmp[j][i];
          }
        }
      }
#pragma unroll
      for (int i = 0; i < NI; i++) outv[i] = sum[i];
    }
  }
  if (writer) {
    if (row0 + 8 * ((NI - 1) >> 2) + 8 <= g.m && !g.dres && tail.epilogue == 0) {  // (uniform) whole rows, nothing to add or apply
      float* const dst = g.c + (size_t)(row0 + 4 * gh) * w.n + n;
#pragma unroll
      for (int i = 0; i < NI; i++) dst[(size_t)(8 * (i >> 2) + (i & 3)) * w.n] = outv[i];
      return;
    }
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const uint32_t row = row0 + 8 * (i >> 2) + 4 * gh + (i & 3);
      if (row < g.m) {
        const size_t o = (size_t)row * w.n + n;
        g.c[o] = apply_epilogue(g.dres ? outv[i] + g.dres[o] : outv[i], tail.epilogue);
      }
    }
  }
}

size_t gemm_lds_bytes(int fmt, uint32_t ksc, uint32_t wnc, bool chain) {
  const uint32_t cb = 8 * ksc, hl = chain ? 2 : 1;
  return std::max<size_t>((size_t)2 * (cb * 2 * hl * 64 + (cb / 2) * 64) * 16 + (size_t)ksc * wnc * 32 * slice_stride(fmt),
                          (size_t)wnc * 16 * 64 * 4);
}

struct GemmPlan {
  uint32_t am;  // the kernel's AM: 0 fp16 activations, 1 f32 in 16-row tiles (M <= 16), 2 f32 in 32-row tiles
  uint32_t ksc, wnc, tpt, nch, parts, colgroups, grid_y;
  size_t lds, scratch_bytes;
};

// Picks the workgroup shape and the K split.  The kernel is bound by what a compute
// unit has to pull in (weights for its columns, activations for its K range), so the
// model is: rounds of workgroups over the CUs x bytes per workgroup.
bool plan_gemm(const LaunchArgs& x, GemmPlan* out) {
  const bool f32a = !x.a_is_f16;
  const uint32_t am = !f32a ? 0 : x.m > 16 ? 2 : 1;
  const uint32_t rows = am == 1 ? 16 : 32;
  const uint32_t bpc = x.w.k / 32, n_tiles = (x.w.n + 31) / 32;
  const uint32_t grid_y = (x.m + rows - 1) / rows;
  if (x.m == 0 || bpc == 0 || grid_y > 65535) return false;
  const double wblock = x.w.fmt == MGN_FMT_Q4 ? 20.0 * 32 : 34.0 * 32;  // bytes per K block of a column tile
  const double ablock = rows * 32.0 * (f32a ? 4 : 2);
  const uint32_t max_tasks = am == 1 ? 8 : 16;  // staging tasks per chunk per ksc, in units of 64 threads
  double best = 0;
  GemmPlan bp{};
  for (uint32_t ksc = 1; ksc <= 2; ksc++) {
    const uint32_t cb = 8 * ksc, chunks = (bpc + cb - 1) / cb;
    // at most 8 waves: each gets 256 registers, and Q8 slices of more would not fit the LDS
    for (uint32_t wnc = 8 / ksc; wnc >= 1; wnc--) {
      const uint32_t tpt = (max_tasks + wnc - 1) / wnc;
      if (tpt > 4) break;
      if (gemm_lds_bytes(x.w.fmt, ksc, wnc, am == 2) > 160 * 1024) continue;
      if (wnc > n_tiles && wnc * ksc > 8 && wnc > 4) continue;  // idle waves only help staging up to a point
      const uint32_t colgroups = (n_tiles + wnc - 1) / wnc;
      if (colgroups > 65535) continue;  // grid.y
      for (uint32_t nch = chunks; nch >= 1; nch--) {
        const uint32_t parts = (chunks + nch - 1) / nch;
        if ((chunks + parts - 1) / parts != nch) continue;  // same split, already seen
        const uint64_t wgs = (uint64_t)grid_y * colgroups * parts;
        const size_t scratch = parts > 1 ? (size_t)parts * grid_y * rows * x.w.n * 4 : 0;
        if (scratch > x.scratch_bytes || (parts > 1 && (uint64_t)grid_y * colgroups > x.n_counters)) break;
        if (wgs * 64 * ksc * wnc > (uint64_t)x.num_cus * 4096 && parts > 1) break;  // far more than enough already
        const double rounds = (double)((wgs + x.num_cus - 1) / x.num_cus);
        // K parts: a workgroup writes its partial tiles, and the last one of a column group,
        // which the launch ends with, reads all parts back behind a round trip for the count
        const double tile_bytes = wnc * 32.0 * rows * 4;
        const double per_wg = nch * cb * (std::min(wnc, n_tiles) * wblock + ablock) + 32768.0 +
                              (parts > 1 ? (1.0 + parts) * tile_bytes + 16384.0 : 0.0);
        // few waves hide little latency; a task count that does not divide over the threads
        // leaves part of the workgroup idle while the rest stages twice
        const double cost = rounds * per_wg * (ksc * wnc < 8 ? 1.5 : 1.0) * (max_tasks % wnc ? 1.15 : 1.0) * (tpt > 2 ? 1.1 : 1.0);
        if (best == 0 || cost < best) {
          best = cost;
          bp.ksc = ksc, bp.wnc = wnc, bp.tpt = tpt <= 1 ? 1 : tpt <= 2 ? 2 : 4;
          bp.nch = nch, bp.parts = parts, bp.colgroups = colgroups, bp.grid_y = grid_y;
          bp.scratch_bytes = scratch;
        }
      }
    }
  }
  if (best == 0 || (uint64_t)bp.colgroups * bp.parts > 0x7fffffffu) return false;
  bp.lds = gemm_lds_bytes(x.w.fmt, bp.ksc, bp.wnc, am == 2);
  bp.am = am;
  *out = bp;
  return true;
}

template <int FMT, int AM, int TPT>
int launch_tpt(ihipStream_t* s, const LaunchArgs& x, const GemmPlan& p) {
  auto kern = gemm_mfma_kernel<FMT, AM, TPT>;
  static std::atomic<uint64_t> big_lds_done{0};
  if (int e = enable_big_lds(kern, x.device, big_lds_done)) return e;
  GemmTail tail{x.d, x.c, (float*)x.scratch, x.counters, x.range_flag, p.grid_y, x.epilogue};
  if (p.colgroups > 65535 || p.grid_y > 65535) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(kern, dim3(p.parts, p.colgroups, p.grid_y), dim3(64 * p.ksc * p.wnc), p.lds, s, x.a, x.w.meta, x.w.quants,
                     x.m, p.ksc, p.wnc, p.nch, x.w.k, x.w.n, p.parts, p.colgroups, tail);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

template <int FMT, int AM>
int launch_am(ihipStream_t* s, const LaunchArgs& x, const GemmPlan& p) {
  switch (p.tpt) {
    case 1: return launch_tpt<FMT, AM, 1>(s, x, p);
    case 2: return launch_tpt<FMT, AM, 2>(s, x, p);
    default: return launch_tpt<FMT, AM, 4>(s, x, p);
  }
}

template <int FMT>
int launch_fmt(ihipStream_t* s, const LaunchArgs& x) {
  GemmPlan p;
  if (!plan_gemm(x, &p)) return (int)hipErrorInvalidValue;
  return p.am == 0 ? launch_am<FMT, 0>(s, x, p) : p.am == 1 ? launch_am<FMT, 1>(s, x, p) : launch_am<FMT, 2>(s, x, p);
}

}  // namespace

bool gemm_mfma_supported(const LaunchArgs& x) {
  if (!x.w.mfma_gemm_range_ok) return false;  // a block minimum or scale too large for the fp16 operand
  GemmPlan p;
  return plan_gemm(x, &p);
}

bool describe_gemm_mfma(const LaunchArgs& x, mgn_plan_info* out) {
  GemmPlan p;
  if (!gemm_mfma_supported(x) || !plan_gemm(x, &p)) return false;
  out->route = MGN_ROUTE_GEMM_MFMA;
  out->grid[0] = p.parts, out->grid[1] = p.colgroups, out->grid[2] = p.grid_y;
  out->threads = 64 * p.ksc * p.wnc;
  out->lds_bytes = (uint32_t)p.lds;
  out->waves_n = p.wnc, out->k_splits = p.ksc, out->k_parts = p.parts, out->steps = p.nch;
  out->quads_per_wave = 0, out->full_steps = 0, out->tail_blocks = 0;
  out->workspace_bytes = p.scratch_bytes;
  return true;
}

int launch_matmul_gemm_mfma(ihipStream_t* s, const LaunchArgs& x) {
  return x.w.fmt == MGN_FMT_Q4 ? launch_fmt<MGN_FMT_Q4>(s, x) : launch_fmt<MGN_FMT_Q8>(s, x);
}

}  // namespace mgn
