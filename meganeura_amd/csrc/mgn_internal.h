// Internal declarations shared by the translation units of libmgn_hip.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "../../include/mgn_hip.h"
#include "../../include/mgn_bench.h"

struct ihipStream_t;
struct ihipEvent_t;

namespace mgn {

// ---- host quantizers (quant_host.cpp) ----
uint16_t f32_to_f16_bits(float f);
float f16_bits_to_f32(uint16_t h);
void quantize_q4_host(const float* w, size_t rows, size_t cols, uint8_t* out);
void quantize_q8_host(const float* w, size_t rows, size_t cols, uint8_t* out);
void quantize_q4_host_nk(const float* w_nk, size_t n_rows, size_t k_cols, uint8_t* out);
void quantize_q8_host_nk(const float* w_nk, size_t n_rows, size_t k_cols, uint8_t* out);
void dequantize_q4_host(const uint8_t* in, size_t rows, size_t cols, float* out);
void dequantize_q8_host(const uint8_t* in, size_t rows, size_t cols, float* out);

// ---- device view of a quantized weight ----
// Blocks are numbered b = n * (K/32) + kb, as in the reference, so one output
// column's blocks are contiguous.  Scales and quants live in separate arrays:
//   Q4: meta[b] = u32 (d_f16 | m_f16 << 16), quants[b] = 16 bytes of nibbles
//       -> byte for byte the reference layout, split at nb*4;
//   Q8: meta[b] = u16 scale_f16,             quants[b] = 32 int8
//       -> the reference's 36-byte blocks with the pad dropped and scales
//          gathered, so quants are 32-byte aligned for 128-bit loads.
// Both arrays carry 256 extra all-zero blocks from index nb = (K/32)*N on.
struct WeightView {
  const void* meta;
  const void* quants;
  uint32_t k, n;  // rows, cols
  int fmt;        // mgn_fmt
  // The tiled MFMA kernel feeds 32 * min (Q4) or 4096 * scale (Q8) to the matrix cores as
  // fp16: true when every block of this weight keeps that finite (|min| < 2047, scale < 15.99).
  bool mfma_gemm_range_ok = true;
  // The 16x16 tiled kernels multiply every block's additive constant (Q4: min, Q8: scale) by 2^additive_lift
  // on its way into the matrix cores, which lose low product bits on fp16 subnormals: the largest
  // power of two up to 2^15 that keeps the weight's largest such constant below 32768.
  uint32_t additive_lift = 0;
};

enum { kProNone = 0, kProRmsNorm = 1, kProSwiglu = 2 };

struct LaunchArgs {
  WeightView w;
  const void* a;   // [m, k] f32 or f16
  const float* d;  // [m, n] or null
  float* c;        // [m, n]
  uint32_t m;
  bool a_is_f16;
  int num_cus;
  int device = 0;  // HIP device ordinal of the context
  // other work may run on the device beside this launch: no plan whose workgroups all wait for
  // each other (they would have to be resident together, and a second such kernel can take their CUs)
  bool shared_device = false;
  // further weights served by the same launch (GEMV-MFMA route only): same K, format and
  // activations, each with its own output and optional residual
  struct More {
    WeightView w;
    const float* d;
    float* c;
  };
  More more[2] = {};
  int n_more = 0;
  uint32_t epilogue = 0;  // unary operations on the output, four bits each, first in the low bits
  // fused prologue (GEMV-MFMA route only): what `a` goes through before the matmul
  int pro_kind = 0;                   // kProNone / kProRmsNorm / kProSwiglu
  const float* pro_weight = nullptr;  // norm weight [K]
  float pro_eps = 0.0f;
  // context-owned workspace for kernels that split K across workgroups
  void* scratch = nullptr;
  size_t scratch_bytes = 0;
  uint32_t* counters = nullptr;  // all zero between launches
  uint32_t n_counters = 0;
  size_t scratch_capacity = 0;   // bytes really behind `scratch` when that is less than the planners are shown (0: scratch_bytes)
  // Second workspace, for kernels whose K parts meet without counters: every word is kHandoverEmpty
  // between launches; a part's partial sums are stored over it and the reading workgroup, which
  // polls until none of the words it needs is empty any more, puts the pattern back.
  void* handover = nullptr;
  size_t handover_bytes = 0;
  uint32_t spin_limit = 1u << 20;  // polls after which a reading wave gives up and sets fault_flag
  // host-visible word a kernel sets when f32 activations leave the range it can represent
  uint32_t* range_flag = nullptr;
  // host-visible word set by a wave that gave up waiting for another workgroup's partial sums
  uint32_t* fault_flag = nullptr;
};

// the bit pattern of a word of the hand-over workspace that holds nothing (a NaN no arithmetic
// produces; a partial sum that happens to carry it is stored as the default NaN instead)
constexpr uint32_t kHandoverEmpty = 0xFFFFFFFFu;

// kernels.hip
int launch_dequantize(ihipStream_t* s, const WeightView& w, float* out_dev);  // out [k, n] f32
int launch_export_q8(ihipStream_t* s, const WeightView& w, uint8_t* out_dev);  // 36-byte blocks
// range2_dev / out2_dev: two words, zero before the launch, that receive the bits of the largest
// |scale| and the largest |min| (as f32) over the blocks the kernel writes or reads
int launch_import_q8(ihipStream_t* s, const uint8_t* ref_dev, size_t nb, void* meta, void* quants, uint32_t* range2_dev);
int launch_scale_range(ihipStream_t* s, const WeightView& w, uint32_t* out2_dev);
int launch_quantize(ihipStream_t* s, int fmt, const float* w_dev, uint32_t k, uint32_t n, void* meta,
                    void* quants, uint32_t* range2_dev);
// the same from a matrix stored [n, k] row-major (16-byte aligned)
int launch_quantize_nk(ihipStream_t* s, int fmt, const float* w_nk_dev, uint32_t k, uint32_t n, void* meta, void* quants,
                       uint32_t* range2_dev);
// in[rows][cols] -> out[cols][rows] (f32); cols at most 65535 * 32
int launch_transpose(ihipStream_t* s, const float* in, float* out, uint32_t rows, uint32_t cols);
// measurement aid: one pass of plain reads over the weight's quants and scales
// two words: shader-clock ticks and 100 MHz ticks over the same ~20 us
// (num_cus_loaded > 0: that many workgroups of matrix-instruction work run meanwhile; out2_dev then
// needs 64 + 4096 bytes)
int launch_clock_probe(ihipStream_t* s, uint64_t* out2_dev, int num_cus_loaded);
// pattern 0: contiguous shares per workgroup; 1: the decode kernel's lane -> address map
int launch_read_probe(ihipStream_t* s, const WeightView& w, int num_cus, uint32_t* sink, int pattern);
int launch_matmul_generic(ihipStream_t* s, const LaunchArgs& a);
bool gemv_supported(const LaunchArgs& a);
int launch_matmul_gemv(ihipStream_t* s, const LaunchArgs& a);
bool gemv_mfma_supported(const LaunchArgs& a);
int launch_matmul_gemv_mfma(ihipStream_t* s, const LaunchArgs& a);
bool gemm_mfma_supported(const LaunchArgs& a);
// launch geometry of the two MFMA routes (false: the route does not take the shape)
bool describe_gemv_mfma(const LaunchArgs& a, mgn_plan_info* out);
bool describe_gemm_mfma(const LaunchArgs& a, mgn_plan_info* out);
// the workspace every context owns: partial sums of K parts, then arrival counters
constexpr size_t kWorkspaceBytes = (size_t)16 << 20;
constexpr uint32_t kWorkspaceCounters = 4096;
constexpr size_t kHandoverBytes = (size_t)16 << 20;  // the counter-free hand-over workspace of a context
int launch_matmul_gemm_mfma(ihipStream_t* s, const LaunchArgs& a);
// kernels_chain.hip: a chain of dependent one-row matmuls in one launch.  One stage as the kernel
// reads it from its table in device memory.
struct ChainStageDev {
  const void* meta;
  const void* quants;
  const float* a;       // activations [K] (kProSwiglu: [2K] = gate | up); a slot of the chain's workspace when made in the chain
  const float* d;       // residual [N] or null; likewise
  const float* norm_w;  // [K] (kProRmsNorm)
  float* c;             // [N]: the caller's buffer
  float* c_slot;        // the workspace slot later stages read this output from, or null
  uint32_t k, n;
  uint32_t pro, epilogue;
  float eps;
  uint32_t a_poll, d_poll;  // that operand is made in the chain: poll until none of its words is empty
  // plan: workgroups that take part, column quads per workgroup, K splits across waves (log2),
  // 16-block steps per split, quad slots (waves per K split that take quads)
  uint32_t wgs, qpw_wg, ksc_log2, steps, nslots;
  uint32_t wg_first;  // the first of the `wgs` consecutive workgroups that serve this stage
};
bool plan_chain_stage(int fmt, int num_cus, ChainStageDev* st, size_t* lds);
int launch_chain(ihipStream_t* s, int device, int fmt, const ChainStageDev* stages_dev, uint32_t nstages, uint32_t grid, size_t lds,
                 uint32_t* clear_ptr, uint32_t clear_words, uint32_t spin_limit, uint32_t* fault_flag);
// kernels_tile.hip: the 16x16x32 tiled kernel (activation image + weight streaming)
bool tile_mfma_supported(const LaunchArgs& a);
// shapes on which the automatic route takes this kernel ahead of the 32x32 tiled one
bool tile_mfma_preferred(const LaunchArgs& a);
bool describe_tile_mfma(const LaunchArgs& a, mgn_plan_info* out);
int launch_matmul_tile_mfma(ihipStream_t* s, const LaunchArgs& a);

}  // namespace mgn

struct mgn_ctx {
  int device = 0;
  int num_cus = 0;
  ihipStream_t* stream = nullptr;
  ihipEvent_t* ev_start = nullptr;
  ihipEvent_t* ev_stop = nullptr;
  mgn_route route = MGN_ROUTE_AUTO;
  bool any_magnitude = true;  // f32 activations of M >= 5 may have any magnitude (mgn_ctx_set_activation_range)
  void* scratch = nullptr;  // split-K partial results + arrival counters, one allocation
  size_t scratch_bytes = 0;
  uint32_t* counters = nullptr;
  uint32_t n_counters = 0;
  void* handover = nullptr;  // counter-free hand-over workspace (LaunchArgs::handover), kHandoverEmpty between launches
  size_t handover_bytes = 0;
  uint32_t spin_limit = 1u << 20;
  bool shared_device = false;  // mgn_ctx_set_shared_device
  uint32_t* range_flag_host = nullptr;  // pinned, mapped, two words: [0] range, [1] hand-over gave up; written by kernels, read at sync points
  uint32_t* range_flag_dev = nullptr;   // the same words as the device sees them
  void* static_scratch = nullptr;       // this device's copy of the library's static workspace (mgn_matmul_q_static)
  void* at_stage = nullptr;             // transposed activations of the A^T matmul forms, grown on demand
  size_t at_stage_bytes = 0;
  std::vector<struct mgn_chain*> chains;  // live chains: their workspaces are emptied again after a fault
  std::string err;
};

// A chain of dependent one-row matmuls served by one launch (mgn_chain_create).
struct mgn_chain {
  int fmt = 0;
  uint32_t nstages = 0, grid = 0;
  size_t lds = 0;
  void* dev = nullptr;  // one allocation: two stage tables, then two sets of slots
  mgn::ChainStageDev* tables[2] = {nullptr, nullptr};
  uint32_t* slots[2] = {nullptr, nullptr};
  uint32_t slot_words = 0;  // per set
  uint32_t runs = 0;        // launches so far: run r works on set r % 2 and empties the other
};

namespace mgn {
mgn_status reserve_at_stage(mgn_ctx* ctx, size_t bytes);
// whether mgn_matmul_q_batch would take these weights in one launch (same K and format assumed checked)
bool batch_plans(const mgn_ctx* ctx, const mgn_weight* const* ws, size_t count, uint32_t m, int pro_kind);
}  // namespace mgn

struct mgn_buf {
  void* ptr = nullptr;
  size_t bytes = 0;
};

struct mgn_weight {
  mgn_fmt fmt;
  size_t rows = 0, cols = 0, nb = 0;
  void* base = nullptr;    // one allocation
  void* meta = nullptr;    // into base
  void* quants = nullptr;  // into base, 256-byte aligned
  size_t meta_bytes = 0, quant_bytes = 0;
  bool mfma_gemm_range_ok = true;  // see WeightView
  uint32_t additive_lift = 0;      // see WeightView
};
