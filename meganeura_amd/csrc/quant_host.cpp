// Host-side block quantizers of the shipped library (reference byte layout).
//
// quantize_q4_0 / quantize_q8_0 / dequantize_q4_0 / dequantize_q8_0 of the
// reference (src/runtime.rs:2035-2215) are single-threaded and walk the f32
// matrix column by column.  These produce the same bytes from a row-blocked,
// multi-threaded walk: one task per block row (32 rows of W), columns in
// order, so every cache line of W is read once.
//
// Built with -ffp-contract=off: the byte-exactness rests on each f32 operation
// rounding separately, as it does in the reference.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "mgn_internal.h"

namespace mgn {

// IEEE binary32 -> binary16, round to nearest even, overflow to infinity,
// gradual underflow (what half::f16::from_f32 does, src/runtime.rs:2074-2075).
uint16_t f32_to_f16_bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  const uint32_t sign = (u >> 16) & 0x8000u;
  u &= 0x7FFFFFFFu;
  if (u >= 0x7F800000u) return uint16_t(sign | (u > 0x7F800000u ? 0x7E00u | ((u >> 13) & 0x3FFu) : 0x7C00u));
  if (u >= 0x477FF000u) return uint16_t(sign | 0x7C00u);  // >= 65520 rounds to inf
  if (u < 0x33000001u) return uint16_t(sign);              // <= 2^-25 rounds to zero
  if (u < 0x38800000u) {
    // subnormal half: add the hidden bit and shift so that one unit = 2^-24
    const uint32_t shift = 126u - (u >> 23);  // 14..24
    const uint32_t man = (u & 0x7FFFFFu) | 0x800000u;
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    q += (rem > half) | ((rem == half) & (q & 1u));
    return uint16_t(sign | q);
  }
  // normal: rebias exponent, round mantissa at bit 13 (carry may bump the exponent)
  uint32_t v = u - 0x38000000u;
  const uint32_t rem = v & 0x1FFFu;
  v >>= 13;
  v += (rem > 0x1000u) | ((rem == 0x1000u) & (v & 1u));
  return uint16_t(sign | v);
}

float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = uint32_t(h & 0x8000u) << 16;
  uint32_t em = h & 0x7FFFu;
  uint32_t u;
  if (em >= 0x7C00u) {
    u = sign | 0x7F800000u | ((em & 0x3FFu) << 13);
  } else if (em >= 0x0400u) {
    u = sign | ((em << 13) + 0x38000000u);
  } else {
    // zero or subnormal: value = em * 2^-24 exactly
    float f = float(em) * 5.9604644775390625e-08f;
    std::memcpy(&u, &f, 4);
    u |= sign;
  }
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

static inline float clamp_keep_nan(float v, float lo, float hi) {
  // Rust's f32::clamp: NaN passes through (and then casts to 0)
  return v < lo ? lo : (v > hi ? hi : v);
}

template <class F>
static void parallel_rows(size_t count, F&& body) {
  unsigned hw = std::thread::hardware_concurrency();
  size_t nthreads = std::min<size_t>(std::min<size_t>(hw ? hw : 1, 16), count);
  if (nthreads <= 1) {
    for (size_t i = 0; i < count; i++) body(i);
    return;
  }
  std::atomic<size_t> next{0};
  std::vector<std::thread> pool;
  pool.reserve(nthreads);
  for (size_t t = 0; t < nthreads; t++)
    pool.emplace_back([&] {
      for (size_t i; (i = next.fetch_add(1)) < count;) body(i);
    });
  for (auto& th : pool) th.join();
}

static constexpr size_t kColTile = 64;

void quantize_q4_host(const float* w, size_t rows, size_t cols, uint8_t* out) {
  const size_t bpc = rows / 32, nb = bpc * cols;
  uint8_t* dm_base = out;
  uint8_t* q_base = out + nb * 4;
  parallel_rows(bpc, [&](size_t blk) {
    float tile[kColTile][32];
    for (size_t c0 = 0; c0 < cols; c0 += kColTile) {
      const size_t cn = std::min(kColTile, cols - c0);
      for (int i = 0; i < 32; i++) {
        const float* src = w + (blk * 32 + i) * cols + c0;
        for (size_t c = 0; c < cn; c++) tile[c][i] = src[c];
      }
      for (size_t c = 0; c < cn; c++) {
        const float* v = tile[c];
        float bmin = INFINITY, bmax = -INFINITY;
        for (int i = 0; i < 32; i++) {
          if (v[i] < bmin) bmin = v[i];
          if (v[i] > bmax) bmax = v[i];
        }
        const float d = bmax > bmin ? (bmax - bmin) / 15.0f : 1.0f;
        const float m = bmin;
        const float d_inv = d > 0.0f ? 1.0f / d : 0.0f;
        const size_t b = (c0 + c) * bpc + blk;
        const uint32_t dm = uint32_t(f32_to_f16_bits(d)) | (uint32_t(f32_to_f16_bits(m)) << 16);
        std::memcpy(dm_base + b * 4, &dm, 4);
        uint8_t* q = q_base + b * 16;
        for (int j = 0; j < 16; j++) {
          float t0 = clamp_keep_nan(std::round((v[2 * j] - m) * d_inv), 0.0f, 15.0f);
          float t1 = clamp_keep_nan(std::round((v[2 * j + 1] - m) * d_inv), 0.0f, 15.0f);
          uint8_t n0 = t0 != t0 ? 0 : uint8_t(t0), n1 = t1 != t1 ? 0 : uint8_t(t1);
          q[j] = uint8_t(n0 | (n1 << 4));
        }
      }
    }
  });
}

// The same encoders for a weight stored [N, K] row-major (the B operand of matmul_bt,
// src/graph.rs:809-817): block (n, kb) covers w_nk[n][kb*32 .. kb*32+31], contiguous in
// memory, and lands where quantizing the transposed [K, N] matrix would put it.
void quantize_q4_host_nk(const float* w_nk, size_t n_rows, size_t k_cols, uint8_t* out) {
  const size_t bpc = k_cols / 32, nb = bpc * n_rows;
  uint8_t* dm_base = out;
  uint8_t* q_base = out + nb * 4;
  parallel_rows(n_rows, [&](size_t n) {
    for (size_t blk = 0; blk < bpc; blk++) {
      const float* v = w_nk + n * k_cols + blk * 32;
      float bmin = INFINITY, bmax = -INFINITY;
      for (int i = 0; i < 32; i++) {
        if (v[i] < bmin) bmin = v[i];
        if (v[i] > bmax) bmax = v[i];
      }
      const float d = bmax > bmin ? (bmax - bmin) / 15.0f : 1.0f;
      const float m = bmin;
      const float d_inv = d > 0.0f ? 1.0f / d : 0.0f;
      const size_t b = n * bpc + blk;
      const uint32_t dm = uint32_t(f32_to_f16_bits(d)) | (uint32_t(f32_to_f16_bits(m)) << 16);
      std::memcpy(dm_base + b * 4, &dm, 4);
      uint8_t* q = q_base + b * 16;
      for (int j = 0; j < 16; j++) {
        float t0 = clamp_keep_nan(std::round((v[2 * j] - m) * d_inv), 0.0f, 15.0f);
        float t1 = clamp_keep_nan(std::round((v[2 * j + 1] - m) * d_inv), 0.0f, 15.0f);
        uint8_t n0 = t0 != t0 ? 0 : uint8_t(t0), n1 = t1 != t1 ? 0 : uint8_t(t1);
        q[j] = uint8_t(n0 | (n1 << 4));
      }
    }
  });
}

void quantize_q8_host_nk(const float* w_nk, size_t n_rows, size_t k_cols, uint8_t* out) {
  const size_t bpc = k_cols / 32;
  parallel_rows(n_rows, [&](size_t n) {
    for (size_t blk = 0; blk < bpc; blk++) {
      const float* v = w_nk + n * k_cols + blk * 32;
      float amax = 0.0f;
      for (int i = 0; i < 32; i++) {
        float a = std::fabs(v[i]);
        if (a > amax) amax = a;
      }
      const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
      const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
      uint8_t* p = out + (n * bpc + blk) * 36;
      const uint32_t head = f32_to_f16_bits(scale);  // pad bytes 2..3 stay zero
      std::memcpy(p, &head, 4);
      for (int i = 0; i < 32; i++) {
        float t = clamp_keep_nan(std::round(v[i] * inv), -128.0f, 127.0f);
        p[4 + i] = uint8_t(int8_t(t != t ? 0 : int(t)));
      }
    }
  });
}

void quantize_q8_host(const float* w, size_t rows, size_t cols, uint8_t* out) {
  const size_t bpc = rows / 32;
  parallel_rows(bpc, [&](size_t blk) {
    float tile[kColTile][32];
    for (size_t c0 = 0; c0 < cols; c0 += kColTile) {
      const size_t cn = std::min(kColTile, cols - c0);
      for (int i = 0; i < 32; i++) {
        const float* src = w + (blk * 32 + i) * cols + c0;
        for (size_t c = 0; c < cn; c++) tile[c][i] = src[c];
      }
      for (size_t c = 0; c < cn; c++) {
        const float* v = tile[c];
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
          float a = std::fabs(v[i]);
          if (a > amax) amax = a;
        }
        const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
        const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        uint8_t* p = out + ((c0 + c) * bpc + blk) * 36;
        const uint32_t head = f32_to_f16_bits(scale);  // pad bytes 2..3 stay zero
        std::memcpy(p, &head, 4);
        for (int i = 0; i < 32; i++) {
          float t = clamp_keep_nan(std::round(v[i] * inv), -128.0f, 127.0f);
          p[4 + i] = uint8_t(int8_t(t != t ? 0 : int(t)));
        }
      }
    }
  });
}

void dequantize_q4_host(const uint8_t* in, size_t rows, size_t cols, float* out) {
  const size_t bpc = rows / 32, nb = bpc * cols;
  parallel_rows(bpc, [&](size_t blk) {
    for (size_t col = 0; col < cols; col++) {
      const size_t b = col * bpc + blk;
      uint32_t dm;
      std::memcpy(&dm, in + b * 4, 4);
      const float d = f16_bits_to_f32(uint16_t(dm & 0xFFFFu));
      const float m = f16_bits_to_f32(uint16_t(dm >> 16));
      const uint8_t* q = in + nb * 4 + b * 16;
      for (int j = 0; j < 16; j++) {
        out[(blk * 32 + 2 * j) * cols + col] = float(q[j] & 0xFu) * d + m;
        out[(blk * 32 + 2 * j + 1) * cols + col] = float(q[j] >> 4) * d + m;
      }
    }
  });
}

void dequantize_q8_host(const uint8_t* in, size_t rows, size_t cols, float* out) {
  const size_t bpc = rows / 32;
  parallel_rows(bpc, [&](size_t blk) {
    for (size_t col = 0; col < cols; col++) {
      const uint8_t* p = in + (col * bpc + blk) * 36;
      uint16_t s16;
      std::memcpy(&s16, p, 2);
      const float scale = f16_bits_to_f32(s16);
      for (int i = 0; i < 32; i++) out[(blk * 32 + i) * cols + col] = float(int8_t(p[4 + i])) * scale;
    }
  });
}

}  // namespace mgn
