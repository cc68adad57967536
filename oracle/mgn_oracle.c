/*
 * CPU ORACLE — TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's block quantizers and of the f32
 * matmul its own tests use as ground truth.  Nothing in the shipped library
 * links or calls this file; only tests, the smoke check and the CPU leg of the
 * benchmark may load it, and only as the checker.
 *
 * Every function cites the reference lines it follows (paths are relative to
 * the reference checkout).  Compile with -ffp-contract=off: the reference is
 * Rust, which never fuses a*b+c, so a contracted FMA here would change bits.
 *
 * What pins each function (none of these is a retyped formula):
 *   orc_f32_to_f16 / orc_f16_to_f32  exhaustive sweep against numpy float16
 *                                    (all 65536 half patterns + tie cases),
 *                                    and the six bit patterns of the
 *                                    reference's q4_decode_f16 unit test.
 *   orc_quantize_q4 / dequantize_q4  hand-derived known-answer bytes on the
 *                                    reference's own unit-test ramp, tie
 *                                    vectors that separate half-away from
 *                                    half-even, constant-block and layout
 *                                    invariants, the reference's two
 *                                    round-trip tests (err < 0.3).
 *   orc_quantize_q8 / dequantize_q8  the reference holds NO test for Q8, so
 *                                    parity rests on hand-derived known-answer
 *                                    bytes, tie vectors and invariants only.
 *   orc_matmul_f32 / _f64            known-answer matmuls from the reference's
 *                                    gpu_smoke tests, brute force on tiny
 *                                    shapes, f32-vs-f64 agreement.
 *   orc_matmul_q_tiled               must equal orc_matmul_f32 on dequantized
 *                                    weights bit for bit (same k order).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_OK 0
#define ORC_EINVAL 1

/* ---- IEEE-754 binary16 <-> binary32, as the `half` crate does it ----------
 * (src/runtime.rs:2074-2075,2122-2123,2172,2204 call half::f16::from_f32 and
 * from_bits().to_f32(): round-to-nearest-even, overflow to inf, gradual
 * underflow, NaN kept as quiet NaN.)  Written with integer arithmetic so that
 * it does not depend on the compiler's _Float16 support. */
uint16_t orc_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t exp = (x >> 23) & 0xFFu;
  uint32_t man = x & 0x7FFFFFu;
  if (exp == 0xFF) { /* inf / NaN */
    if (man == 0) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | 0x7C00u | 0x0200u | (man >> 13)); /* quiet NaN */
  }
  int32_t e = (int32_t)exp - 127 + 15; /* rebias */
  if (e >= 31) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
  if (e <= 0) { /* subnormal half or zero */
    if (e < -10) return (uint16_t)sign; /* below half of the smallest subnormal */
    man |= 0x800000u; /* hidden bit */
    uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
    uint32_t half_man = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
    return (uint16_t)(sign | half_man); /* a carry lands on exponent 1: correct */
  }
  uint32_t half_man = man >> 13;
  uint32_t rem = man & 0x1FFFu;
  uint32_t out = sign | ((uint32_t)e << 10) | half_man;
  if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1u))) out++; /* may carry to inf */
  return (uint16_t)out;
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t x;
  if (exp == 0) {
    if (man == 0) {
      x = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        e++;
        man <<= 1;
      } while ((man & 0x400u) == 0);
      man &= 0x3FFu;
      x = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    x = sign | 0x7F800000u | (man << 13);
  } else {
    x = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

/* Rust `f32::clamp(lo, hi)` keeps NaN; `as u8` / `as i8` then saturate and map
 * NaN to 0 (src/runtime.rs:2088,2182). */
static inline float orc_clamp(float v, float lo, float hi) {
  if (v < lo) return lo;
  if (v > hi) return hi;
  return v;
}

size_t orc_packed_size_q4(size_t rows, size_t cols) { return (rows / 32) * cols * 20; }
size_t orc_packed_size_q8(size_t rows, size_t cols) { return (rows / 32) * cols * 36; }

/* ---- Q4 ("Q4_0" in the enum, asymmetric scale+min in fact) ----------------
 * src/runtime.rs:2035-2102.  w is f32 [rows, cols] row-major; blocks are 32
 * consecutive rows of one column; block id = col * (rows/32) + blk.  Output:
 * nb little-endian u32 words (d_f16 | m_f16 << 16), then nb * 16 nibble bytes.
 */
int orc_quantize_q4(const float* w, size_t rows, size_t cols, uint8_t* out) {
  if (rows % 32 != 0) return ORC_EINVAL; /* reference asserts (2037-2040) */
  size_t bpc = rows / 32, nb = bpc * cols;
  memset(out, 0, nb * 20); /* zero-initialised before OR-ing nibbles (2047) */
  for (size_t col = 0; col < cols; col++) {
    for (size_t blk = 0; blk < bpc; blk++) {
      size_t b = col * bpc + blk;
      float bmin = INFINITY, bmax = -INFINITY; /* 2054-2065 */
      for (int i = 0; i < 32; i++) {
        float v = w[(blk * 32 + i) * cols + col];
        if (v < bmin) bmin = v;
        if (v > bmax) bmax = v;
      }
      float d = (bmax > bmin) ? (bmax - bmin) / 15.0f : 1.0f; /* 2068-2072 */
      float m = bmin;
      uint32_t dm = (uint32_t)orc_f32_to_f16(d) | ((uint32_t)orc_f32_to_f16(m) << 16);
      out[b * 4 + 0] = (uint8_t)(dm);
      out[b * 4 + 1] = (uint8_t)(dm >> 8);
      out[b * 4 + 2] = (uint8_t)(dm >> 16);
      out[b * 4 + 3] = (uint8_t)(dm >> 24);
      uint8_t* q = out + nb * 4 + b * 16;            /* 2083 */
      float d_inv = (d > 0.0f) ? 1.0f / d : 0.0f;    /* 2084: unrounded f32 d */
      for (int i = 0; i < 32; i++) {
        float v = w[(blk * 32 + i) * cols + col];
        float t = orc_clamp(roundf((v - m) * d_inv), 0.0f, 15.0f); /* 2088 */
        uint8_t nib = (t != t) ? 0 : (uint8_t)t;
        q[i / 2] |= (i % 2 == 0) ? nib : (uint8_t)(nib << 4);       /* 2090-2096 */
      }
    }
  }
  return ORC_OK;
}

/* src/runtime.rs:2105-2138: out[row*cols+col] = nibble as f32 * d + m. */
int orc_dequantize_q4(const uint8_t* in, size_t rows, size_t cols, float* out) {
  if (rows % 32 != 0) return ORC_EINVAL;
  size_t bpc = rows / 32, nb = bpc * cols;
  for (size_t col = 0; col < cols; col++) {
    for (size_t blk = 0; blk < bpc; blk++) {
      size_t b = col * bpc + blk;
      const uint8_t* p = in + b * 4;
      float d = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
      float m = orc_f16_to_f32((uint16_t)(p[2] | (p[3] << 8)));
      const uint8_t* q = in + nb * 4 + b * 16;
      for (int i = 0; i < 32; i++) {
        uint32_t nib = (i % 2 == 0) ? (q[i / 2] & 0xFu) : (q[i / 2] >> 4);
        out[(blk * 32 + i) * cols + col] = (float)nib * d + m;
      }
    }
  }
  return ORC_OK;
}

/* ---- Q8_0 ------------------------------------------------------------------
 * src/runtime.rs:2143-2188.  36 bytes per block at b*36: f16 scale, two zero
 * pad bytes, 32 int8. */
int orc_quantize_q8(const float* w, size_t rows, size_t cols, uint8_t* out) {
  if (rows % 32 != 0) return ORC_EINVAL;
  size_t bpc = rows / 32, nb = bpc * cols;
  memset(out, 0, nb * 36);
  for (size_t col = 0; col < cols; col++) {
    for (size_t blk = 0; blk < bpc; blk++) {
      uint8_t* p = out + (col * bpc + blk) * 36;
      float amax = 0.0f; /* 2162-2169 */
      for (int i = 0; i < 32; i++) {
        float a = fabsf(w[(blk * 32 + i) * cols + col]);
        if (a > amax) amax = a;
      }
      float scale = (amax > 0.0f) ? amax / 127.0f : 1.0f; /* 2171 */
      uint16_t s16 = orc_f32_to_f16(scale);
      p[0] = (uint8_t)s16;
      p[1] = (uint8_t)(s16 >> 8);
      float inv = (scale > 0.0f) ? 1.0f / scale : 0.0f;   /* 2178 */
      for (int i = 0; i < 32; i++) {
        float v = w[(blk * 32 + i) * cols + col];
        float t = orc_clamp(roundf(v * inv), -128.0f, 127.0f); /* 2182 */
        int8_t q = (t != t) ? 0 : (int8_t)t;
        p[4 + i] = (uint8_t)q;
      }
    }
  }
  return ORC_OK;
}

/* src/runtime.rs:2191-2215. */
int orc_dequantize_q8(const uint8_t* in, size_t rows, size_t cols, float* out) {
  if (rows % 32 != 0) return ORC_EINVAL;
  size_t bpc = rows / 32;
  for (size_t col = 0; col < cols; col++) {
    for (size_t blk = 0; blk < bpc; blk++) {
      const uint8_t* p = in + (col * bpc + blk) * 36;
      float scale = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
      for (int i = 0; i < 32; i++)
        out[(blk * 32 + i) * cols + col] = (float)(int8_t)p[4 + i] * scale;
    }
  }
  return ORC_OK;
}

/* ---- matmul ground truth ---------------------------------------------------
 * tests/gpu_smoke.rs:2732-2741 and tests/gemv_parity.rs:11-21: C[M,N] = A[M,K] x
 * B[K,N] (+ D[M,N]), f32, k ascending, one rounding per multiply and per add.
 * The residual is added once after the k loop (src/shaders/matmul.wgsl store,
 * src/shaders/matmul_gemv_add.wgsl:49). */
void orc_matmul_f32(const float* a, const float* b, const float* d, float* c, size_t m,
                    size_t k, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t col = 0; col < n; col++) {
    for (size_t row = 0; row < m; row++) {
      float sum = 0.0f;
      for (size_t kk = 0; kk < k; kk++) sum += a[row * k + kk] * b[kk * n + col];
      c[row * n + col] = d ? sum + d[row * n + col] : sum;
    }
  }
}

/* f64-accumulated variant, the precedent of tests/gemv_parity.rs:207-217: used
 * to budget how far any f32 summation order may drift. */
void orc_matmul_f64(const float* a, const float* b, const float* d, float* c, size_t m,
                    size_t k, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t col = 0; col < n; col++) {
    for (size_t row = 0; row < m; row++) {
      double sum = 0.0;
      for (size_t kk = 0; kk < k; kk++) sum += (double)a[row * k + kk] * (double)b[kk * n + col];
      if (d) sum += (double)d[row * n + col];
      c[row * n + col] = (float)sum;
    }
  }
}

/* The same, reading B straight from packed bytes in column order so that the
 * [K,N] f32 matrix never has to exist: what a full-size check at K*N = 58.7 M
 * needs.  fmt: 0 = Q4, 1 = Q8.  Per element it decodes exactly as
 * orc_dequantize_q4/q8 and sums in the same k order as orc_matmul_f32. */
int orc_matmul_packed_f32(int fmt, const float* a, const uint8_t* packed, const float* d,
                          float* c, size_t m, size_t k, size_t n) {
  if (k % 32 != 0 || (fmt != 0 && fmt != 1)) return ORC_EINVAL;
  size_t bpc = k / 32, nb = bpc * n;
#pragma omp parallel for schedule(static)
  for (size_t col = 0; col < n; col++) {
    float* wcol = (float*)malloc(k * sizeof(float));
    for (size_t blk = 0; blk < bpc; blk++) {
      size_t b = col * bpc + blk;
      if (fmt == 0) {
        const uint8_t* p = packed + b * 4;
        float dd = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
        float mm = orc_f16_to_f32((uint16_t)(p[2] | (p[3] << 8)));
        const uint8_t* q = packed + nb * 4 + b * 16;
        for (int i = 0; i < 32; i++) {
          uint32_t nib = (i % 2 == 0) ? (q[i / 2] & 0xFu) : (q[i / 2] >> 4);
          wcol[blk * 32 + i] = (float)nib * dd + mm;
        }
      } else {
        const uint8_t* p = packed + b * 36;
        float s = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
        for (int i = 0; i < 32; i++) wcol[blk * 32 + i] = (float)(int8_t)p[4 + i] * s;
      }
    }
    for (size_t row = 0; row < m; row++) {
      float sum = 0.0f;
      for (size_t kk = 0; kk < k; kk++) sum += a[row * k + kk] * wcol[kk];
      c[row * n + col] = d ? sum + d[row * n + col] : sum;
    }
    free(wcol);
  }
  return ORC_OK;
}

/* ---- the reference's GPU algorithm, restated for the CPU timing leg --------
 * src/shaders/matmul.wgsl:1-109 with $B_LOAD_EXPR = dequant_q4 / dequant_q8
 * (src/codegen.rs:748-769, 785-805): grid [ceil(N/64), ceil(M/64)], 64x64
 * output tile per workgroup, K walked in tiles of 32, B dequantized ELEMENT BY
 * ELEMENT on load (two word reads + f16 decode per element, no reuse of the
 * block's scale), 256 threads each owning a 4x4 patch.  One OpenMP task per
 * workgroup stands in for how a CPU Vulkan driver runs workgroups on cores.
 * The f16 decode here keeps subnormals (the CPU definition); for the weight
 * ranges used they never occur, so this matches the shader's flush-to-zero
 * decoder too.  Result is bit-identical to orc_matmul_f32 on dequantized
 * weights because each output still sums k ascending with separate mul/add. */
static inline float orc_deq_elem(int fmt, const uint8_t* packed, size_t nb, size_t bpc,
                                 size_t krow, size_t ncol) {
  size_t b = ncol * bpc + krow / 32;
  size_t i = krow % 32;
  if (fmt == 0) {
    const uint8_t* p = packed + b * 4;
    float d = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
    float m = orc_f16_to_f32((uint16_t)(p[2] | (p[3] << 8)));
    uint8_t byte = packed[nb * 4 + b * 16 + i / 2];
    uint32_t nib = (i & 1) ? (byte >> 4) : (byte & 0xFu);
    return (float)nib * d + m;
  }
  const uint8_t* p = packed + b * 36;
  float s = orc_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
  return (float)(int8_t)p[4 + i] * s;
}

int orc_matmul_q_tiled(int fmt, const float* a, const uint8_t* packed, const float* d,
                       float* c, size_t m, size_t k, size_t n) {
  if (k % 32 != 0 || (fmt != 0 && fmt != 1)) return ORC_EINVAL;
  size_t bpc = k / 32, nb = bpc * n;
  size_t gx = (n + 63) / 64, gy = (m + 63) / 64;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (size_t wy = 0; wy < gy; wy++) {
    for (size_t wx = 0; wx < gx; wx++) {
      float sa[64 * 33], sb[32 * 65], acc[64][64];
      memset(acc, 0, sizeof acc);
      size_t tile_row = wy * 64, tile_col = wx * 64;
      for (size_t t = 0; t < k; t += 32) {
        for (size_t r = 0; r < 64; r++)
          for (size_t cc = 0; cc < 32; cc++) {
            size_t ar = tile_row + r, ac = t + cc;
            sa[r * 33 + cc] = (ar < m && ac < k) ? a[ar * k + ac] : 0.0f;
          }
        for (size_t r = 0; r < 32; r++)
          for (size_t cc = 0; cc < 64; cc++) {
            size_t br = t + r, bc = tile_col + cc;
            sb[r * 65 + cc] = (br < k && bc < n) ? orc_deq_elem(fmt, packed, nb, bpc, br, bc) : 0.0f;
          }
        for (size_t kk = 0; kk < 32; kk++)
          for (size_t r = 0; r < 64; r++) {
            float av = sa[r * 33 + kk];
            for (size_t cc = 0; cc < 64; cc++) acc[r][cc] += av * sb[kk * 65 + cc];
          }
      }
      for (size_t r = 0; r < 64; r++)
        for (size_t cc = 0; cc < 64; cc++) {
          size_t row = tile_row + r, col = tile_col + cc;
          if (row < m && col < n) {
            size_t idx = row * n + col;
            c[idx] = d ? acc[r][cc] + d[idx] : acc[r][cc];
          }
        }
    }
  }
  return ORC_OK;
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
