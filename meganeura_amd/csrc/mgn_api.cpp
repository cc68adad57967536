// C ABI of libmgn_hip: contexts, buffers, quantized weights, matmul dispatch.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <algorithm>
#include <vector>

#include "mgn_internal.h"

// ---- split-K workspace in the library's own image, for callers that cannot allocate ----
// mgn_matmul_q_static hands this array to the kernels in place of the context's workspace.
// The name below is a host-side stand-in: the device address comes from hipGetSymbolAddress,
// once per device (every device holds its own copy), and only that pointer is passed on.
constexpr size_t kStaticPartialBytes = MGN_STATIC_WORKSPACE_BYTES;  // partial sums of K parts
constexpr uint32_t kStaticCounters = mgn::kWorkspaceCounters;      // arrival counters behind them
// ... and, behind the counters, as many bytes again for the kernels whose K parts meet without counters
constexpr size_t kStaticHandoverOffset = kStaticPartialBytes + kStaticCounters * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[kStaticHandoverOffset + kStaticPartialBytes];

__global__ void fill_words_kernel(uint32_t* p, uint32_t n, uint32_t value) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void* g_static_scratch[kMaxDevices] = {};  // device address of `scratch`, per device ordinal

// With `device` current: the address of this device's copy of `scratch` (looked up once).
hipError_t static_scratch_for(int device, void** out) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_scratch[device]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_static_scratch[device] = p;
  }
  *out = g_static_scratch[device];
  return hipSuccess;
}

thread_local std::string g_create_error;

mgn_status fail(mgn_ctx* ctx, mgn_status st, const std::string& msg) {
  if (ctx) ctx->err = msg; else g_create_error = msg;
  return st;
}

mgn_status hip_fail(mgn_ctx* ctx, const char* what, hipError_t e) {
  return fail(ctx, MGN_EHIP, std::string(what) + ": " + hipGetErrorString(e));
}

#define MGN_HIP(ctx, call)                                   \
  do {                                                       \
    hipError_t e_ = (call);                                  \
    if (e_ != hipSuccess) return hip_fail(ctx, #call, e_);   \
  } while (0)

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

size_t meta_elem(mgn_fmt fmt) { return fmt == MGN_FMT_Q4 ? 4 : 2; }
size_t quant_elem(mgn_fmt fmt) { return fmt == MGN_FMT_Q4 ? 16 : 32; }

bool valid_fmt(mgn_fmt fmt) { return fmt == MGN_FMT_Q4 || fmt == MGN_FMT_Q8; }

mgn::WeightView view_of(const mgn_weight* w) {
  return mgn::WeightView{w->meta, w->quants, (uint32_t)w->rows, (uint32_t)w->cols, (int)w->fmt, w->mfma_gemm_range_ok, w->additive_lift};
}

// Device storage for a [rows, cols] weight, contents undefined.
mgn_status weight_alloc(mgn_ctx* ctx, mgn_fmt fmt, size_t rows, size_t cols, mgn_weight** out) {
  if (!ctx || !out) return fail(ctx, MGN_EINVAL, "null argument");
  *out = nullptr;
  if (!valid_fmt(fmt)) return fail(ctx, MGN_EINVAL, "unknown weight format");
  if (rows == 0 || cols == 0) return fail(ctx, MGN_EINVAL, "empty weight");
  if (rows % 32 != 0) return fail(ctx, MGN_EINVAL, "quantized weights require rows (K dim) to be a multiple of 32");
  if (rows > 0xFFFFFFE0ull || cols > 0xFFFFFFFFull || (rows / 32) * cols >= 0x7FFFFFFFull)
    return fail(ctx, MGN_EINVAL, "weight too large: block count must stay below 2^31");
  auto* w = new (std::nothrow) mgn_weight();
  if (!w) return fail(ctx, MGN_ENOMEM, "out of host memory");
  w->fmt = fmt;
  w->rows = rows;
  w->cols = cols;
  w->nb = (rows / 32) * cols;
  w->meta_bytes = w->nb * meta_elem(fmt);
  w->quant_bytes = w->nb * quant_elem(fmt);
  // 256 all-zero blocks follow the real ones in both arrays: lanes that have no block of
  // their own load block nb and contribute exactly zero, and the GEMV kernels' last K steps of
  // the last column may read past the end of K (up to 15 blocks; up to 8 x 16 + 15 when K is
  // cut into parts of whole steps for different workgroups).
  constexpr size_t kMetaPad = 1024, kQuantPad = 8192;
  const size_t q_off = align_up(w->meta_bytes + kMetaPad, 256);
  hipError_t e = hipMalloc(&w->base, q_off + w->quant_bytes + kQuantPad);
  if (e != hipSuccess) {
    delete w;
    return e == hipErrorOutOfMemory ? fail(ctx, MGN_ENOMEM, "out of device memory") : hip_fail(ctx, "hipMalloc", e);
  }
  w->meta = w->base;
  w->quants = (char*)w->base + q_off;
  e = hipMemsetAsync((char*)w->meta + w->meta_bytes, 0, kMetaPad, ctx->stream);
  if (e == hipSuccess) e = hipMemsetAsync((char*)w->quants + w->quant_bytes, 0, kQuantPad, ctx->stream);
  if (e != hipSuccess) {
    (void)hipFree(w->base);
    delete w;
    return hip_fail(ctx, "hipMemsetAsync", e);
  }
  *out = w;
  return MGN_OK;
}

// The automatic choice of a kernel family.  M <= 4: the MFMA GEMV.  Larger M: the resident
// 16x16x32 kernel where it measured faster; the 32x32 tiled kernel for fp16 activations and
// for f32 activations the caller has promised to keep in the fp16 range (it splits them
// without rescaling), if the weight's block constants are in its range too; the rescaling
// 16x16x32 kernels for everything else.
mgn_route auto_route(const mgn::LaunchArgs& x, bool any_magnitude) {
  if (mgn::gemv_mfma_supported(x)) return MGN_ROUTE_GEMV_MFMA;
  if (mgn::tile_mfma_preferred(x)) return MGN_ROUTE_TILE_MFMA;
  if ((x.a_is_f16 || !any_magnitude) && mgn::gemm_mfma_supported(x)) return MGN_ROUTE_GEMM_MFMA;
  if (mgn::tile_mfma_supported(x)) return MGN_ROUTE_TILE_MFMA;
  if (mgn::gemv_supported(x)) return MGN_ROUTE_GEMV_VALU;
  return MGN_ROUTE_GENERIC;
}

// After the stream has been synchronised: did a wave give up waiting for another workgroup's
// partial sums, or did a kernel meet activations outside its range?
mgn_status check_range_flag(mgn_ctx* ctx) {
  if (!ctx->range_flag_host) return MGN_OK;
  volatile uint32_t* const flags = (volatile uint32_t*)ctx->range_flag_host;
  if (flags[1] != 0) {
    // what the parts of that launch stored after the reader had given up is still in the hand-over
    // workspace (and in the slots of the chains): make it empty again before anything else runs
    flags[0] = flags[1] = 0;
    hipError_t e = ctx->handover ? hipMemsetAsync(ctx->handover, 0xFF, ctx->handover_bytes, ctx->stream) : hipSuccess;
    for (mgn_chain* ch : ctx->chains)
      if (e == hipSuccess && ch->slot_words) e = hipMemsetAsync(ch->slots[0], 0xFF, (size_t)2 * ch->slot_words * 4, ctx->stream);
    if (e == hipSuccess && ctx->static_scratch)
      e = hipMemsetAsync((char*)ctx->static_scratch + kStaticHandoverOffset, 0xFF, kStaticPartialBytes, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, "hand-over workspace reset", e);
    return fail(ctx, MGN_ETIMEOUT,
                "a workgroup gave up waiting for the partial sums of the other K parts of its matmul (spin limit reached): "
                "outputs of the matmuls since the last synchronisation are not valid");
  }
  if (flags[0] == 0) return MGN_OK;
  flags[0] = 0;
  return fail(ctx, MGN_ERANGE,
              "an f32 activation of magnitude >= 65504 reached the tiled MFMA kernel (M >= 5), which splits activations "
              "into fp16 pairs without rescaling: the affected outputs are wrong (the context was set to MGN_ACT_FP16_RANGE, or the route was forced)");
}

// Whether the 32x32 MFMA kernel may take a weight depends on the largest |scale| and |min| over
// its blocks.  The kernels that put the blocks on the device reduce them on the way into two spare
// words of the context (range_words), which are zeroed before and read back after, in stream
// order; the one synchronisation a weight's creation needs anyway then covers the read-back.
uint32_t* range_words(mgn_ctx* ctx) { return (uint32_t*)((char*)ctx->scratch + ctx->scratch_bytes) + ctx->n_counters; }

hipError_t clear_range_words(mgn_ctx* ctx) { return hipMemsetAsync(range_words(ctx), 0, 8, ctx->stream); }

// Enqueues the read-back, synchronises and records the verdict in the weight.
mgn_status finish_weight_range(mgn_ctx* ctx, mgn_weight* w, const char* what) {
  uint32_t host[2] = {0, 0};
  hipError_t e = hipMemcpyAsync(host, range_words(ctx), 8, hipMemcpyDeviceToHost, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) return hip_fail(ctx, what, e);
  float smax, mmax;
  std::memcpy(&smax, &host[0], 4);
  std::memcpy(&mmax, &host[1], 4);
  w->mfma_gemm_range_ok = w->fmt == MGN_FMT_Q4 ? (mmax < 2047.0f && std::isfinite(smax)) : smax < 15.99f;
  // the constant the additive part multiplies by: every block's minimum (Q4) or scale (Q8)
  const float amax = w->fmt == MGN_FMT_Q4 ? mmax : smax;
  w->additive_lift = 0;
  if (std::isfinite(amax)) {
    while (w->additive_lift < 15 && std::ldexp(amax, (int)w->additive_lift + 1) < 32768.0f) w->additive_lift++;
  }
  return MGN_OK;
}

}  // namespace

namespace mgn {
// The staging area of the A^T matmul forms holds at least `bytes` afterwards (allocates or grows it;
// a session does this for its whole plan when it is built, so that no step allocates).
mgn_status reserve_at_stage(mgn_ctx* ctx, size_t bytes) {
  if (!ctx) return MGN_EINVAL;
  if (ctx->at_stage_bytes >= bytes) return MGN_OK;
  // earlier launches may still read the old area
  MGN_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (ctx->at_stage) (void)hipFree(ctx->at_stage);
  ctx->at_stage = nullptr;
  ctx->at_stage_bytes = 0;
  const size_t grown = align_up(bytes, (size_t)1 << 20);
  const hipError_t e = hipMalloc(&ctx->at_stage, grown);
  if (e != hipSuccess) {
    ctx->at_stage = nullptr;
    return e == hipErrorOutOfMemory ? fail(ctx, MGN_ENOMEM, "out of device memory") : hip_fail(ctx, "hipMalloc", e);
  }
  ctx->at_stage_bytes = grown;
  return MGN_OK;
}

// Would one launch serve these weights together (mgn_matmul_q_batch's own check)?  The plan
// depends on the column count of the whole batch, so a weight that plans alone need not plan
// next to its siblings.
bool batch_plans(const mgn_ctx* ctx, const mgn_weight* const* ws, size_t count, uint32_t m, int pro_kind) {
  if (!ctx || !ws || count == 0 || count > 3 || m == 0) return false;
  if (ctx->route != MGN_ROUTE_AUTO && ctx->route != MGN_ROUTE_GEMV_MFMA) return false;
  LaunchArgs x{view_of(ws[0]), nullptr, nullptr, nullptr, m, false, ctx->num_cus};
  for (size_t j = 1; j < count; j++) x.more[j - 1] = {view_of(ws[j]), nullptr, nullptr};
  x.n_more = (int)count - 1;
  x.scratch = ctx->scratch;
  x.scratch_bytes = ctx->scratch_bytes;
  x.counters = ctx->counters;
  x.n_counters = ctx->n_counters;
  x.pro_kind = pro_kind;
  return gemv_mfma_supported(x);
}
}  // namespace mgn

extern "C" {

const char* mgn_version(void) { return "0.1.0"; }
const char* mgn_built_for(void) { return "gfx950"; }

mgn_status mgn_ctx_create(int device_id, mgn_ctx** out) {
  if (!out) return fail(nullptr, MGN_EINVAL, "null out pointer");
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0) return fail(nullptr, MGN_ENODEVICE, "no HIP device visible");
  if (device_id < 0 || device_id >= count) return fail(nullptr, MGN_EINVAL, "device_id out of range");
  hipDeviceProp_t prop;
  MGN_HIP(nullptr, hipGetDeviceProperties(&prop, device_id));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(nullptr, MGN_ENODEVICE, std::string("kernels are built for gfx950, device is ") + prop.gcnArchName);
  MGN_HIP(nullptr, hipSetDevice(device_id));
  auto* ctx = new (std::nothrow) mgn_ctx();
  if (!ctx) return fail(nullptr, MGN_ENOMEM, "out of host memory");
  ctx->device = device_id;
  ctx->num_cus = prop.multiProcessorCount;
  if ((e = static_scratch_for(device_id, &ctx->static_scratch)) != hipSuccess) {
    delete ctx;
    return hip_fail(nullptr, "hipGetSymbolAddress(static workspace)", e);
  }
  if ((e = hipStreamCreate(&ctx->stream)) != hipSuccess || (e = hipEventCreate(&ctx->ev_start)) != hipSuccess ||
      (e = hipEventCreate(&ctx->ev_stop)) != hipSuccess) {
    mgn_ctx_destroy(ctx);
    return hip_fail(nullptr, "stream/event creation", e);
  }
  // workspace of the split-K matmul kernels: partial tiles, then 4096 arrival counters
  constexpr size_t kScratchBytes = mgn::kWorkspaceBytes;
  constexpr uint32_t kCounters = mgn::kWorkspaceCounters;
  // (+ two words the weight range scan reduces into)
  if ((e = hipMalloc(&ctx->scratch, kScratchBytes + (kCounters + 2) * sizeof(uint32_t))) != hipSuccess ||
      (e = hipMemsetAsync((char*)ctx->scratch + kScratchBytes, 0, (kCounters + 2) * sizeof(uint32_t), ctx->stream)) != hipSuccess) {
    mgn_ctx_destroy(ctx);
    return hip_fail(nullptr, "workspace allocation", e);
  }
  ctx->scratch_bytes = kScratchBytes;
  ctx->counters = (uint32_t*)((char*)ctx->scratch + kScratchBytes);
  ctx->n_counters = kCounters;
  // the counter-free hand-over workspace: every word "empty" between launches.  The static array's
  // share is set up here too (once per context: cheap, and whatever an earlier process state left is gone)
  if ((e = hipMalloc(&ctx->handover, mgn::kHandoverBytes)) != hipSuccess ||
      (e = hipMemsetAsync(ctx->handover, 0xFF, mgn::kHandoverBytes, ctx->stream)) != hipSuccess ||
      (e = hipMemsetAsync((char*)ctx->static_scratch + kStaticHandoverOffset, 0xFF, kStaticPartialBytes, ctx->stream)) != hipSuccess) {
    mgn_ctx_destroy(ctx);
    return hip_fail(nullptr, "hand-over workspace allocation", e);
  }
  ctx->handover_bytes = mgn::kHandoverBytes;
  // one pinned, device-mapped word: a kernel that meets activations it cannot represent sets it
  // and the next synchronising call reports MGN_ERANGE
  if ((e = hipHostMalloc((void**)&ctx->range_flag_host, 2 * sizeof(uint32_t), hipHostMallocMapped)) != hipSuccess ||
      (e = hipHostGetDevicePointer((void**)&ctx->range_flag_dev, ctx->range_flag_host, 0)) != hipSuccess) {
    mgn_ctx_destroy(ctx);
    return hip_fail(nullptr, "pinned flag allocation", e);
  }
  ctx->range_flag_host[0] = ctx->range_flag_host[1] = 0;
  *out = ctx;
  return MGN_OK;
}

void mgn_ctx_destroy(mgn_ctx* ctx) {
  if (!ctx) return;
  if (ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamDestroy(ctx->stream);
  }
  if (ctx->scratch) (void)hipFree(ctx->scratch);
  if (ctx->handover) (void)hipFree(ctx->handover);
  if (ctx->at_stage) (void)hipFree(ctx->at_stage);
  if (ctx->range_flag_host) (void)hipHostFree(ctx->range_flag_host);
  if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
  if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
  delete ctx;
}

const char* mgn_last_error(const mgn_ctx* ctx) { return ctx ? ctx->err.c_str() : g_create_error.c_str(); }

mgn_status mgn_sync(mgn_ctx* ctx) {
  if (!ctx) return MGN_EINVAL;
  MGN_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return check_range_flag(ctx);
}

mgn_status mgn_ctx_set_activation_range(mgn_ctx* ctx, mgn_act_range range) {
  if (!ctx) return MGN_EINVAL;
  if (range != MGN_ACT_ANY && range != MGN_ACT_FP16_RANGE) return fail(ctx, MGN_EINVAL, "unknown activation range");
  ctx->any_magnitude = range == MGN_ACT_ANY;
  return MGN_OK;
}

mgn_status mgn_ctx_set_shared_device(mgn_ctx* ctx, int shared) {
  if (!ctx) return MGN_EINVAL;
  ctx->shared_device = shared != 0;
  return MGN_OK;
}

mgn_status mgn_ctx_set_spin_limit(mgn_ctx* ctx, uint32_t polls) {
  if (!ctx) return MGN_EINVAL;
  ctx->spin_limit = polls;
  return MGN_OK;
}

mgn_status mgn_ctx_set_route(mgn_ctx* ctx, mgn_route route) {
  if (!ctx) return MGN_EINVAL;
  if (route < MGN_ROUTE_AUTO || route > MGN_ROUTE_TILE_MFMA) return fail(ctx, MGN_EINVAL, "unknown route");
  ctx->route = route;
  return MGN_OK;
}

// ---- buffers ----

mgn_status mgn_buf_alloc(mgn_ctx* ctx, size_t bytes, mgn_buf** out) {
  if (!ctx || !out) return fail(ctx, MGN_EINVAL, "null argument");
  *out = nullptr;
  auto* b = new (std::nothrow) mgn_buf();
  if (!b) return fail(ctx, MGN_ENOMEM, "out of host memory");
  b->bytes = bytes;
  const size_t alloc = align_up(bytes < 4 ? 4 : bytes, 256);  // the reference's minimum is 4 bytes
  hipError_t e = hipMalloc(&b->ptr, alloc);
  if (e != hipSuccess) {
    delete b;
    return e == hipErrorOutOfMemory ? fail(ctx, MGN_ENOMEM, "out of device memory") : hip_fail(ctx, "hipMalloc", e);
  }
  e = hipMemsetAsync(b->ptr, 0, alloc, ctx->stream);
  if (e != hipSuccess) {
    (void)hipFree(b->ptr);
    delete b;
    return hip_fail(ctx, "hipMemsetAsync", e);
  }
  *out = b;
  return MGN_OK;
}

void mgn_buf_free(mgn_ctx* ctx, mgn_buf* buf) {
  if (!buf) return;
  if (ctx) (void)hipStreamSynchronize(ctx->stream);
  if (buf->ptr) (void)hipFree(buf->ptr);
  delete buf;
}

size_t mgn_buf_size(const mgn_buf* buf) { return buf ? buf->bytes : 0; }
void* mgn_buf_device_ptr(const mgn_buf* buf) { return buf ? buf->ptr : nullptr; }

mgn_status mgn_buf_upload(mgn_ctx* ctx, mgn_buf* buf, size_t offset, const void* src, size_t bytes) {
  if (!ctx || !buf || (!src && bytes)) return fail(ctx, MGN_EINVAL, "null argument");
  if (offset > buf->bytes || bytes > buf->bytes - offset) return fail(ctx, MGN_EINVAL, "upload exceeds buffer size");
  if (bytes == 0) return MGN_OK;
  MGN_HIP(ctx, hipMemcpyAsync((char*)buf->ptr + offset, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  MGN_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return MGN_OK;
}

mgn_status mgn_buf_download(mgn_ctx* ctx, const mgn_buf* buf, size_t offset, void* dst, size_t bytes) {
  if (!ctx || !buf || (!dst && bytes)) return fail(ctx, MGN_EINVAL, "null argument");
  if (offset > buf->bytes || bytes > buf->bytes - offset) return fail(ctx, MGN_EINVAL, "download exceeds buffer size");
  if (bytes == 0) return mgn_sync(ctx);
  MGN_HIP(ctx, hipMemcpyAsync(dst, (const char*)buf->ptr + offset, bytes, hipMemcpyDeviceToHost, ctx->stream));
  MGN_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return check_range_flag(ctx);
}

mgn_status mgn_buf_copy(mgn_ctx* ctx, mgn_buf* dst, const mgn_buf* src, size_t bytes) {
  if (!ctx || !dst || !src) return fail(ctx, MGN_EINVAL, "null argument");
  if (bytes > dst->bytes || bytes > src->bytes) return fail(ctx, MGN_EINVAL, "copy exceeds buffer size");
  if (bytes == 0) return MGN_OK;
  MGN_HIP(ctx, hipMemcpyAsync(dst->ptr, src->ptr, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return MGN_OK;
}

// ---- host quantizers ----

size_t mgn_packed_size(mgn_fmt fmt, size_t rows, size_t cols) {
  if (!valid_fmt(fmt)) return 0;
  return (rows / 32) * cols * (fmt == MGN_FMT_Q4 ? 20 : 36);
}

mgn_status mgn_quantize_ref(mgn_fmt fmt, const float* w, size_t rows, size_t cols, uint8_t* out) {
  if (!valid_fmt(fmt) || rows % 32 != 0) return MGN_EINVAL;
  if (rows == 0 || cols == 0) return MGN_OK;
  if (!w || !out) return MGN_EINVAL;
  if (fmt == MGN_FMT_Q4) mgn::quantize_q4_host(w, rows, cols, out);
  else mgn::quantize_q8_host(w, rows, cols, out);
  return MGN_OK;
}

mgn_status mgn_quantize_ref_nk(mgn_fmt fmt, const float* w_nk, size_t n_rows, size_t k_cols, uint8_t* out) {
  if (!valid_fmt(fmt) || k_cols % 32 != 0) return MGN_EINVAL;
  if (n_rows == 0 || k_cols == 0) return MGN_OK;
  if (!w_nk || !out) return MGN_EINVAL;
  if (fmt == MGN_FMT_Q4) mgn::quantize_q4_host_nk(w_nk, n_rows, k_cols, out);
  else mgn::quantize_q8_host_nk(w_nk, n_rows, k_cols, out);
  return MGN_OK;
}

mgn_status mgn_dequantize_ref(mgn_fmt fmt, const uint8_t* in, size_t rows, size_t cols, float* out) {
  if (!valid_fmt(fmt) || rows % 32 != 0) return MGN_EINVAL;
  if (rows == 0 || cols == 0) return MGN_OK;
  if (!in || !out) return MGN_EINVAL;
  if (fmt == MGN_FMT_Q4) mgn::dequantize_q4_host(in, rows, cols, out);
  else mgn::dequantize_q8_host(in, rows, cols, out);
  return MGN_OK;
}

// ---- weights ----

mgn_status mgn_weight_create_packed(mgn_ctx* ctx, mgn_fmt fmt, const uint8_t* packed, size_t rows, size_t cols,
                                    mgn_weight** out) {
  if (!packed) return fail(ctx, MGN_EINVAL, "null argument");
  mgn_weight* w = nullptr;
  mgn_status st = weight_alloc(ctx, fmt, rows, cols, &w);
  if (st != MGN_OK) return st;
  hipError_t e = clear_range_words(ctx);
  void* tmp = nullptr;
  if (fmt == MGN_FMT_Q4) {
    // the reference layout is already "all scale|min words, then all nibbles": plain copies, and
    // a pass over the scale words for their range
    if (e == hipSuccess) e = hipMemcpyAsync(w->meta, packed, w->meta_bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess)
      e = hipMemcpyAsync(w->quants, packed + w->meta_bytes, w->quant_bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = (hipError_t)mgn::launch_scale_range(ctx->stream, view_of(w), range_words(ctx));
  } else {
    const size_t bytes = w->nb * 36;
    if (e == hipSuccess) e = hipMalloc(&tmp, bytes);
    if (e == hipSuccess) e = hipMemcpyAsync(tmp, packed, bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess)
      e = (hipError_t)mgn::launch_import_q8(ctx->stream, (const uint8_t*)tmp, w->nb, w->meta, w->quants, range_words(ctx));
  }
  // one synchronisation: the caller's bytes are free again, tmp can go, the range is known
  if (e == hipSuccess) st = finish_weight_range(ctx, w, "weight upload");
  else (void)hipStreamSynchronize(ctx->stream);
  if (tmp) (void)hipFree(tmp);
  if (e != hipSuccess || st != MGN_OK) {
    mgn_weight_free(ctx, w);
    return e != hipSuccess ? hip_fail(ctx, "weight upload", e) : st;
  }
  *out = w;
  return MGN_OK;
}

// A weight from f32 values on the device, stored [rows, cols] (K major) or, nk, [cols, rows]: the
// quantizer kernel packs them and reduces the range of the block constants on the way.  Synchronises.
static mgn_status weight_from_device_f32(mgn_ctx* ctx, mgn_fmt fmt, const void* src, size_t src_bytes, size_t rows,
                                         size_t cols, bool nk, mgn_weight** out) {
  mgn_weight* w = nullptr;
  mgn_status st = weight_alloc(ctx, fmt, rows, cols, &w);
  if (st != MGN_OK) return st;
  if (src_bytes / sizeof(float) < rows * cols) {
    mgn_weight_free(ctx, w);
    return fail(ctx, MGN_EINVAL, "source buffer smaller than rows*cols floats");
  }
  hipError_t e = clear_range_words(ctx);
  if (e == hipSuccess)
    e = (hipError_t)(nk ? mgn::launch_quantize_nk : mgn::launch_quantize)(ctx->stream, (int)fmt, (const float*)src, (uint32_t)rows,
                                                                          (uint32_t)cols, w->meta, w->quants, range_words(ctx));
  if (e != hipSuccess) {
    mgn_weight_free(ctx, w);
    return hip_fail(ctx, "quantize kernel", e);
  }
  st = finish_weight_range(ctx, w, "quantize kernel");
  if (st != MGN_OK) {
    mgn_weight_free(ctx, w);
    return st;
  }
  *out = w;
  return MGN_OK;
}

// Uploads host f32 values into a staging buffer and packs them there (see mgn_weight_create).
// The staging copy costs 4 bytes per element of device memory until the call returns.  *no_staging
// is set when there was no room for it, or none for the weight while it was held: the caller then
// packs on the host, which needs the weight's own bytes only.
static mgn_status weight_from_host_f32(mgn_ctx* ctx, mgn_fmt fmt, const float* wdata, size_t rows, size_t cols, bool nk,
                                       mgn_weight** out, bool* no_staging) {
  *no_staging = false;
  void* staged = nullptr;
  const size_t bytes = rows * cols * sizeof(float);
  if (hipMalloc(&staged, bytes) != hipSuccess) {
    (void)hipGetLastError();  // out of device memory for the staging copy: not an error of the call
    *no_staging = true;
    return MGN_ENOMEM;
  }
  const hipError_t e = hipMemcpyAsync(staged, wdata, bytes, hipMemcpyHostToDevice, ctx->stream);
  const mgn_status st = e == hipSuccess ? weight_from_device_f32(ctx, fmt, staged, bytes, rows, cols, nk, out)
                                        : hip_fail(ctx, "weight upload", e);
  if (e != hipSuccess || st != MGN_OK) (void)hipStreamSynchronize(ctx->stream);
  (void)hipFree(staged);
  // the weight itself found no room while the staging copy was held: the host path, which holds
  // none, gets its try
  if (st == MGN_ENOMEM) *no_staging = true;
  return st;
}

mgn_status mgn_weight_create(mgn_ctx* ctx, mgn_fmt fmt, const float* wdata, size_t rows, size_t cols,
                             mgn_weight** out) {
  if (!ctx || !out || !wdata) return fail(ctx, MGN_EINVAL, "null argument");
  *out = nullptr;
  if (!valid_fmt(fmt)) return fail(ctx, MGN_EINVAL, "unknown weight format");
  if (rows % 32 != 0) return fail(ctx, MGN_EINVAL, "quantized weights require rows (K dim) to be a multiple of 32");
  if (rows == 0 || cols == 0) return fail(ctx, MGN_EINVAL, "empty weight");
  // The f32 values go up as they are and the device quantizer packs them (the same bytes as the
  // host quantizer's, three to four times sooner on a 4096 x 14336 weight: 9 ms against 28-35 ms)
  // when there is device memory for them; otherwise the host packs and the bytes go up.
  bool no_staging = false;
  const mgn_status direct = weight_from_host_f32(ctx, fmt, wdata, rows, cols, false, out, &no_staging);
  if (!no_staging) return direct;
  std::vector<uint8_t> packed;
  try {
    packed.resize(mgn_packed_size(fmt, rows, cols));
  } catch (const std::bad_alloc&) {
    return fail(ctx, MGN_ENOMEM, "out of host memory");
  }
  mgn_quantize_ref(fmt, wdata, rows, cols, packed.data());
  return mgn_weight_create_packed(ctx, fmt, packed.data(), rows, cols, out);
}

mgn_status mgn_weight_create_nk(mgn_ctx* ctx, mgn_fmt fmt, const float* w_nk, size_t n_rows, size_t k_cols,
                                mgn_weight** out) {
  if (!ctx || !out || !w_nk) return fail(ctx, MGN_EINVAL, "null argument");
  *out = nullptr;
  if (!valid_fmt(fmt)) return fail(ctx, MGN_EINVAL, "unknown weight format");
  if (k_cols % 32 != 0) return fail(ctx, MGN_EINVAL, "quantized weights require the K dim to be a multiple of 32");
  if (n_rows == 0 || k_cols == 0) return fail(ctx, MGN_EINVAL, "empty weight");
  bool no_staging = false;
  const mgn_status direct = weight_from_host_f32(ctx, fmt, w_nk, k_cols, n_rows, true, out, &no_staging);  // as mgn_weight_create
  if (!no_staging) return direct;
  std::vector<uint8_t> packed;
  try {
    packed.resize(mgn_packed_size(fmt, k_cols, n_rows));
  } catch (const std::bad_alloc&) {
    return fail(ctx, MGN_ENOMEM, "out of host memory");
  }
  mgn_quantize_ref_nk(fmt, w_nk, n_rows, k_cols, packed.data());
  return mgn_weight_create_packed(ctx, fmt, packed.data(), k_cols, n_rows, out);
}

mgn_status mgn_weight_create_device(mgn_ctx* ctx, mgn_fmt fmt, const mgn_buf* w_f32, size_t rows, size_t cols,
                                    mgn_weight** out) {
  if (!w_f32) return fail(ctx, MGN_EINVAL, "null argument");
  return weight_from_device_f32(ctx, fmt, w_f32->ptr, w_f32->bytes, rows, cols, false, out);
}

void mgn_weight_free(mgn_ctx* ctx, mgn_weight* w) {
  if (!w) return;
  if (ctx) (void)hipStreamSynchronize(ctx->stream);
  if (w->base) (void)hipFree(w->base);
  delete w;
}

mgn_status mgn_weight_info(const mgn_weight* w, mgn_fmt* fmt, size_t* rows, size_t* cols) {
  if (!w) return MGN_EINVAL;
  if (fmt) *fmt = w->fmt;
  if (rows) *rows = w->rows;
  if (cols) *cols = w->cols;
  return MGN_OK;
}

mgn_status mgn_weight_dequantize(mgn_ctx* ctx, const mgn_weight* w, float* out_host) {
  if (!ctx || !w || !out_host) return fail(ctx, MGN_EINVAL, "null argument");
  const size_t bytes = w->rows * w->cols * sizeof(float);
  float* tmp = nullptr;
  hipError_t e = hipMalloc((void**)&tmp, bytes);
  if (e != hipSuccess) return e == hipErrorOutOfMemory ? fail(ctx, MGN_ENOMEM, "out of device memory") : hip_fail(ctx, "hipMalloc", e);
  e = (hipError_t)mgn::launch_dequantize(ctx->stream, view_of(w), tmp);
  if (e == hipSuccess) e = hipMemcpyAsync(out_host, tmp, bytes, hipMemcpyDeviceToHost, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  (void)hipFree(tmp);
  if (e != hipSuccess) return hip_fail(ctx, "dequantize", e);
  return MGN_OK;
}

mgn_status mgn_weight_export_ref(mgn_ctx* ctx, const mgn_weight* w, uint8_t* out_packed) {
  if (!ctx || !w || !out_packed) return fail(ctx, MGN_EINVAL, "null argument");
  hipError_t e = hipSuccess;
  void* tmp = nullptr;
  if (w->fmt == MGN_FMT_Q4) {
    e = hipMemcpyAsync(out_packed, w->meta, w->meta_bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess)
      e = hipMemcpyAsync(out_packed + w->meta_bytes, w->quants, w->quant_bytes, hipMemcpyDeviceToHost, ctx->stream);
  } else {
    const size_t bytes = w->nb * 36;
    e = hipMalloc(&tmp, bytes);
    if (e == hipSuccess) e = (hipError_t)mgn::launch_export_q8(ctx->stream, view_of(w), (uint8_t*)tmp);
    if (e == hipSuccess) e = hipMemcpyAsync(out_packed, tmp, bytes, hipMemcpyDeviceToHost, ctx->stream);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (tmp) (void)hipFree(tmp);
  if (e != hipSuccess) return hip_fail(ctx, "weight export", e);
  return MGN_OK;
}

// ---- pre-quantized weights on disk ----
// Header, little-endian: "MGNQ" | u32 version (1) | u32 fmt | u32 reserved (0) | u64 rows | u64 cols
// | u64 payload bytes; then the reference-layout packed bytes (mgn_packed_size of them).

namespace {
struct QFileHeader {
  char magic[4];
  uint32_t version, fmt, reserved;
  uint64_t rows, cols, payload;
};
static_assert(sizeof(QFileHeader) == 40, "header is 40 bytes, no padding");
}  // namespace

mgn_status mgn_weight_save(mgn_ctx* ctx, const mgn_weight* w, const char* path) {
  if (!ctx || !w || !path) return fail(ctx, MGN_EINVAL, "null argument");
  std::vector<uint8_t> packed;
  try {
    packed.resize(mgn_packed_size(w->fmt, w->rows, w->cols));
  } catch (const std::bad_alloc&) {
    return fail(ctx, MGN_ENOMEM, "out of host memory");
  }
  mgn_status st = mgn_weight_export_ref(ctx, w, packed.data());
  if (st != MGN_OK) return st;
  QFileHeader h{{'M', 'G', 'N', 'Q'}, 1u, (uint32_t)w->fmt, 0u, (uint64_t)w->rows, (uint64_t)w->cols, (uint64_t)packed.size()};
  FILE* f = std::fopen(path, "wb");
  if (!f) return fail(ctx, MGN_EINVAL, std::string("cannot open for writing: ") + path);
  const bool ok = std::fwrite(&h, sizeof(h), 1, f) == 1 && std::fwrite(packed.data(), 1, packed.size(), f) == packed.size();
  const bool closed = std::fclose(f) == 0;
  if (!ok || !closed) return fail(ctx, MGN_EINVAL, std::string("short write: ") + path);
  return MGN_OK;
}

mgn_status mgn_weight_load(mgn_ctx* ctx, const char* path, mgn_weight** out) {
  if (!ctx || !path || !out) return fail(ctx, MGN_EINVAL, "null argument");
  *out = nullptr;
  FILE* f = std::fopen(path, "rb");
  if (!f) return fail(ctx, MGN_ENOTFOUND, std::string("cannot open: ") + path);
  QFileHeader h{};
  mgn_status st = MGN_OK;
  std::vector<uint8_t> packed;
  if (std::fread(&h, sizeof(h), 1, f) != 1 || std::memcmp(h.magic, "MGNQ", 4) != 0) {
    st = fail(ctx, MGN_EINVAL, std::string("not a quantized-weight file: ") + path);
  } else if (h.version != 1) {
    st = fail(ctx, MGN_EINVAL, "unknown quantized-weight file version " + std::to_string(h.version));
  } else if (!valid_fmt((mgn_fmt)h.fmt) || h.rows == 0 || h.cols == 0 || h.rows % 32 != 0 ||
             h.rows > 0xFFFFFFE0ull || h.cols > 0xFFFFFFFFull || (h.rows / 32) * h.cols >= 0x7FFFFFFFull ||
             h.payload != mgn_packed_size((mgn_fmt)h.fmt, h.rows, h.cols)) {
    st = fail(ctx, MGN_EINVAL, std::string("inconsistent header in ") + path);
  } else {
    try {
      packed.resize(h.payload);
    } catch (const std::bad_alloc&) {
      st = fail(ctx, MGN_ENOMEM, "out of host memory");
    }
    if (st == MGN_OK && std::fread(packed.data(), 1, packed.size(), f) != packed.size())
      st = fail(ctx, MGN_EINVAL, std::string("truncated file: ") + path);
  }
  std::fclose(f);
  if (st != MGN_OK) return st;
  return mgn_weight_create_packed(ctx, (mgn_fmt)h.fmt, packed.data(), h.rows, h.cols, out);
}

// ---- matmul ----

static mgn_status matmul_impl(mgn_ctx* ctx, const mgn_buf* a, bool a_is_f16, const mgn_weight* w, const mgn_buf* d,
                              mgn_buf* c, uint32_t m, int pro_kind = mgn::kProNone, const mgn_buf* norm_weight = nullptr,
                              float eps = 0.0f, uint32_t epilogue = 0, bool static_workspace = false) {
  if (!ctx || !a || !w || !c) return fail(ctx, MGN_EINVAL, "null argument");
  if (m == 0) return MGN_OK;
  const size_t k = w->rows, n = w->cols;
  const size_t a_elem = a_is_f16 ? 2 : 4;
  const size_t a_cols = pro_kind == mgn::kProSwiglu ? 2 * k : k;
  if (a->bytes / a_elem < (size_t)m * a_cols) return fail(ctx, MGN_EINVAL, "A is smaller than its m rows");
  if (pro_kind == mgn::kProRmsNorm && (!norm_weight || norm_weight->bytes / 4 < k))
    return fail(ctx, MGN_EINVAL, "norm weight is missing or shorter than K floats");
  if (c->bytes / 4 < (size_t)m * n) return fail(ctx, MGN_EINVAL, "C is smaller than m*N floats");
  if (d && d->bytes / 4 < (size_t)m * n) return fail(ctx, MGN_EINVAL, "D is smaller than m*N floats");
  if (c->ptr == a->ptr) return fail(ctx, MGN_EINVAL, "C must not alias A");
  mgn::LaunchArgs x{view_of(w), a->ptr, d ? (const float*)d->ptr : nullptr, (float*)c->ptr, m, a_is_f16, ctx->num_cus};
  x.device = ctx->device;
  x.shared_device = ctx->shared_device;
  x.range_flag = ctx->range_flag_dev;
  x.fault_flag = ctx->range_flag_dev + 1;
  x.spin_limit = ctx->spin_limit;
  x.scratch = ctx->scratch;
  x.scratch_bytes = ctx->scratch_bytes;
  x.counters = ctx->counters;
  x.n_counters = ctx->n_counters;
  x.handover = ctx->handover;
  x.handover_bytes = ctx->handover_bytes;
  x.pro_kind = pro_kind;
  x.pro_weight = norm_weight ? (const float*)norm_weight->ptr : nullptr;
  x.pro_eps = eps;
  x.epilogue = epilogue;
  mgn_route route = ctx->route;
  if (pro_kind != mgn::kProNone) {
    // only the MFMA GEMV stages its activations in a way a prologue can ride on
    if (a_is_f16 || !mgn::gemv_mfma_supported(x) || (route != MGN_ROUTE_AUTO && route != MGN_ROUTE_GEMV_MFMA))
      return fail(ctx, MGN_EUNSUPPORTED, "fused prologue needs the GEMV_MFMA route (f32 activations, M <= 4)");
    route = MGN_ROUTE_GEMV_MFMA;
  }
  if (route == MGN_ROUTE_AUTO) route = auto_route(x, ctx->any_magnitude);
  if (static_workspace) {
    // Same plan as the allocating entry point (the planners see the same workspace limits), run
    // on the library's static array if the plan's partial sums fit it; refused otherwise.
    mgn_plan_info plan{};
    const bool parts = route == MGN_ROUTE_GEMV_MFMA   ? mgn::describe_gemv_mfma(x, &plan)
                       : route == MGN_ROUTE_GEMM_MFMA ? mgn::describe_gemm_mfma(x, &plan)
                       : route == MGN_ROUTE_TILE_MFMA ? mgn::describe_tile_mfma(x, &plan)
                                                      : false;
    const uint64_t need = parts ? plan.workspace_bytes : 0;
    if (need > kStaticPartialBytes)
      return fail(ctx, MGN_EUNSUPPORTED,
                  "mgn_matmul_q_static: this shape's K parts need " + std::to_string(need) +
                      " bytes of workspace, the static one holds " + std::to_string(kStaticPartialBytes) +
                      "; use mgn_matmul_q");
    x.scratch = ctx->static_scratch;
    x.scratch_capacity = kStaticPartialBytes;  // a launch that would need more than was checked above is refused, not run
    x.counters = (uint32_t*)((char*)ctx->static_scratch + kStaticPartialBytes);
    x.handover = (char*)ctx->static_scratch + kStaticHandoverOffset;
    if (need > 0) {
      // every call on this device shares the array: the arrival counters must start at zero and
      // the hand-over words the plan uses must be empty, whatever an earlier call left (fill
      // kernels, not memset nodes: safe under graph capture)
      hipLaunchKernelGGL(fill_words_kernel, dim3((kStaticCounters + 255) / 256), dim3(256), 0, ctx->stream, x.counters,
                         kStaticCounters, 0u);
      const uint32_t words = (uint32_t)((need + 3) / 4);
      hipLaunchKernelGGL(fill_words_kernel, dim3((words + 255) / 256), dim3(256), 0, ctx->stream, (uint32_t*)x.handover, words,
                         mgn::kHandoverEmpty);
      const hipError_t le = hipGetLastError();
      if (le != hipSuccess) return hip_fail(ctx, "workspace fill launch", le);
    }
  }
  int rc;
  switch (route) {
    case MGN_ROUTE_GEMV_VALU:
      if (!mgn::gemv_supported(x)) return fail(ctx, MGN_EINVAL, "GEMV_VALU route does not support this shape");
      rc = mgn::launch_matmul_gemv(ctx->stream, x);
      break;
    case MGN_ROUTE_GEMV_MFMA:
      if (!mgn::gemv_mfma_supported(x)) return fail(ctx, MGN_EINVAL, "GEMV_MFMA route does not support this shape");
      rc = mgn::launch_matmul_gemv_mfma(ctx->stream, x);
      break;
    case MGN_ROUTE_TILE_MFMA:
      if (!mgn::tile_mfma_supported(x)) return fail(ctx, MGN_EINVAL, "TILE_MFMA route does not support this shape");
      rc = mgn::launch_matmul_tile_mfma(ctx->stream, x);
      break;
    case MGN_ROUTE_GEMM_MFMA:
      if (!mgn::gemm_mfma_supported(x)) return fail(ctx, MGN_EINVAL, "GEMM_MFMA route does not support this shape");
      rc = mgn::launch_matmul_gemm_mfma(ctx->stream, x);
      break;
    default:
      rc = mgn::launch_matmul_generic(ctx->stream, x);
      break;
  }
  if (rc != 0) return hip_fail(ctx, "kernel launch", (hipError_t)rc);
  return MGN_OK;
}

mgn_status mgn_matmul_q(mgn_ctx* ctx, const mgn_buf* a, const mgn_weight* w, const mgn_buf* d, mgn_buf* c,
                        uint32_t m) {
  return matmul_impl(ctx, a, false, w, d, c, m);
}

mgn_status mgn_matmul_q_static(mgn_ctx* ctx, const mgn_buf* a, const mgn_weight* w, const mgn_buf* d, mgn_buf* c,
                               uint32_t m) {
  return matmul_impl(ctx, a, false, w, d, c, m, mgn::kProNone, nullptr, 0.0f, 0, true);
}

mgn_status mgn_matmul_q_epilogue(mgn_ctx* ctx, const mgn_buf* a, const mgn_weight* w, const mgn_buf* d, mgn_buf* c,
                                 uint32_t m, const mgn_unary* ops, size_t n_ops) {
  if (n_ops > 8 || (n_ops > 0 && !ops)) return fail(ctx, MGN_EINVAL, "an epilogue has at most 8 operations");
  uint32_t packed = 0;
  for (size_t i = 0; i < n_ops; i++) {
    if (ops[i] < MGN_UNARY_RELU || ops[i] > MGN_UNARY_SILU) return fail(ctx, MGN_EINVAL, "unknown unary operation in the epilogue");
    packed |= (uint32_t)ops[i] << (4 * i);
  }
  return matmul_impl(ctx, a, false, w, d, c, m, mgn::kProNone, nullptr, 0.0f, packed);
}

mgn_status mgn_matmul_q_rms_norm(mgn_ctx* ctx, const mgn_buf* x, const mgn_buf* norm_weight, float eps,
                                 const mgn_weight* w, const mgn_buf* d, mgn_buf* c, uint32_t m) {
  return matmul_impl(ctx, x, false, w, d, c, m, mgn::kProRmsNorm, norm_weight, eps);
}

mgn_status mgn_matmul_q_swiglu(mgn_ctx* ctx, const mgn_buf* gate_up, const mgn_weight* w, const mgn_buf* d, mgn_buf* c,
                               uint32_t m) {
  return matmul_impl(ctx, gate_up, false, w, d, c, m, mgn::kProSwiglu);
}

mgn_status mgn_matmul_q_batch(mgn_ctx* ctx, const mgn_buf* a, mgn_prologue prologue, const mgn_buf* norm_weight, float eps,
                              const mgn_matmul_item* items, size_t count, uint32_t m) {
  if (!ctx || !a || !items) return fail(ctx, MGN_EINVAL, "null argument");
  if (count == 0 || count > 3) return fail(ctx, MGN_EINVAL, "a batch holds 1 to 3 matmuls");
  if (prologue < MGN_PROLOGUE_NONE || prologue > MGN_PROLOGUE_SWIGLU) return fail(ctx, MGN_EINVAL, "unknown prologue");
  if (m == 0) return MGN_OK;
  for (size_t j = 0; j < count; j++)
    if (!items[j].w || !items[j].c) return fail(ctx, MGN_EINVAL, "null weight or output in the batch");
  const mgn_weight* w0 = items[0].w;
  const size_t k = w0->rows;
  const size_t a_cols = prologue == MGN_PROLOGUE_SWIGLU ? 2 * k : k;
  if (a->bytes / 4 < (size_t)m * a_cols) return fail(ctx, MGN_EINVAL, "A is smaller than its m rows");
  if (prologue == MGN_PROLOGUE_RMS_NORM && (!norm_weight || norm_weight->bytes / 4 < k))
    return fail(ctx, MGN_EINVAL, "norm weight is missing or shorter than K floats");
  mgn::LaunchArgs x{view_of(w0), a->ptr, items[0].d ? (const float*)items[0].d->ptr : nullptr, (float*)items[0].c->ptr, m,
                    false, ctx->num_cus};
  for (size_t j = 0; j < count; j++) {
    const mgn_matmul_item& it = items[j];
    if (it.w->rows != k || it.w->fmt != w0->fmt) return fail(ctx, MGN_EINVAL, "batched weights must share K and the format");
    if (it.c->bytes / 4 < (size_t)m * it.w->cols) return fail(ctx, MGN_EINVAL, "C is smaller than m*N floats");
    if (it.d && it.d->bytes / 4 < (size_t)m * it.w->cols) return fail(ctx, MGN_EINVAL, "D is smaller than m*N floats");
    if (it.c->ptr == a->ptr) return fail(ctx, MGN_EINVAL, "C must not alias A");
    if (j > 0) x.more[j - 1] = {view_of(it.w), it.d ? (const float*)it.d->ptr : nullptr, (float*)it.c->ptr};
  }
  x.n_more = (int)count - 1;
  x.device = ctx->device;
  x.fault_flag = ctx->range_flag_dev + 1;
  x.spin_limit = ctx->spin_limit;
  x.handover = ctx->handover;
  x.handover_bytes = ctx->handover_bytes;
  x.scratch = ctx->scratch;
  x.scratch_bytes = ctx->scratch_bytes;
  x.counters = ctx->counters;
  x.n_counters = ctx->n_counters;
  x.pro_kind = (int)prologue;
  x.pro_weight = norm_weight ? (const float*)norm_weight->ptr : nullptr;
  x.pro_eps = eps;
  if ((ctx->route != MGN_ROUTE_AUTO && ctx->route != MGN_ROUTE_GEMV_MFMA) || !mgn::gemv_mfma_supported(x))
    return fail(ctx, MGN_EUNSUPPORTED, "batched matmul needs the GEMV_MFMA route (f32 activations, M <= 4)");
  const int rc = mgn::launch_matmul_gemv_mfma(ctx->stream, x);
  if (rc != 0) return hip_fail(ctx, "kernel launch", (hipError_t)rc);
  return MGN_OK;
}

int mgn_matmul_q_can_fuse(mgn_ctx* ctx, const mgn_weight* w, uint32_t m) {
  if (!ctx || !w || m == 0) return 0;
  mgn::LaunchArgs x{view_of(w), nullptr, nullptr, nullptr, m, false, ctx->num_cus};
  x.pro_kind = mgn::kProRmsNorm;
  return (ctx->route == MGN_ROUTE_AUTO || ctx->route == MGN_ROUTE_GEMV_MFMA) && mgn::gemv_mfma_supported(x) ? 1 : 0;
}

mgn_status mgn_matmul_q_at(mgn_ctx* ctx, const mgn_buf* a_t, const mgn_weight* w, const mgn_buf* d, mgn_buf* c, uint32_t m,
                           const mgn_unary* ops, size_t n_ops) {
  if (!ctx || !a_t || !w || !c) return fail(ctx, MGN_EINVAL, "null argument");
  if (n_ops > 8 || (n_ops > 0 && !ops)) return fail(ctx, MGN_EINVAL, "an epilogue has at most 8 operations");
  uint32_t packed = 0;
  for (size_t i = 0; i < n_ops; i++) {
    if (ops[i] < MGN_UNARY_RELU || ops[i] > MGN_UNARY_SILU) return fail(ctx, MGN_EINVAL, "unknown unary operation in the epilogue");
    packed |= (uint32_t)ops[i] << (4 * i);
  }
  if (m == 0) return MGN_OK;
  const size_t k = w->rows, need = (size_t)m * k * sizeof(float);
  if (a_t->bytes < need) return fail(ctx, MGN_EINVAL, "A^T is smaller than K rows of m floats");
  if (c->ptr == a_t->ptr) return fail(ctx, MGN_EINVAL, "C must not alias A");
  if (((size_t)m + 31) / 32 > 65535) return fail(ctx, MGN_EINVAL, "m is too large for the transposed form");
  if (const mgn_status st = mgn::reserve_at_stage(ctx, need)) return st;
  const int rc = mgn::launch_transpose(ctx->stream, (const float*)a_t->ptr, (float*)ctx->at_stage, (uint32_t)k, m);
  if (rc != 0) return hip_fail(ctx, "transpose launch", (hipError_t)rc);
  const mgn_buf staged{ctx->at_stage, need};
  return matmul_impl(ctx, &staged, false, w, d, c, m, mgn::kProNone, nullptr, 0.0f, packed);
}

mgn_status mgn_matmul_q_f16a(mgn_ctx* ctx, const mgn_buf* a_f16, const mgn_weight* w, const mgn_buf* d, mgn_buf* c,
                             uint32_t m) {
  return matmul_impl(ctx, a_f16, true, w, d, c, m);
}

mgn_status mgn_matmul_q_plan(mgn_fmt fmt, uint32_t m, uint64_t k, uint64_t n, int a_is_f16, int num_cus, mgn_plan_info* out) {
  if (!out || !valid_fmt(fmt) || m == 0 || k == 0 || n == 0 || k % 32 != 0 || num_cus <= 0) return MGN_EINVAL;
  if (k > 0xFFFFFFE0ull || n > 0xFFFFFFFFull || (k / 32) * n >= 0x7FFFFFFFull) return MGN_EINVAL;
  *out = mgn_plan_info{};
  mgn::LaunchArgs x{};
  x.w = mgn::WeightView{nullptr, nullptr, (uint32_t)k, (uint32_t)n, (int)fmt, true};
  x.m = m;
  x.a_is_f16 = a_is_f16 == 1;
  x.num_cus = num_cus;
  // the planners only look at whether a workspace exists, never through the pointers
  static char workspace_stand_in;
  x.scratch = &workspace_stand_in;
  x.scratch_bytes = mgn::kWorkspaceBytes;
  x.counters = (uint32_t*)&workspace_stand_in;
  x.n_counters = mgn::kWorkspaceCounters;
  x.handover = &workspace_stand_in;
  x.handover_bytes = mgn::kHandoverBytes;
  if (a_is_f16 < 0 || a_is_f16 > 2) return MGN_EINVAL;
  const mgn_route route = auto_route(x, a_is_f16 == 0);
  if (route == MGN_ROUTE_GEMV_MFMA && mgn::describe_gemv_mfma(x, out)) return MGN_OK;
  if (route == MGN_ROUTE_GEMM_MFMA && mgn::describe_gemm_mfma(x, out)) return MGN_OK;
  if (route == MGN_ROUTE_TILE_MFMA && mgn::describe_tile_mfma(x, out)) return MGN_OK;
  out->route = route;
  return MGN_OK;
}

mgn_status mgn_matmul_q_loop(mgn_ctx* ctx, const mgn_buf* a, int a_is_f16, const mgn_weight* const* weights, size_t count,
                             const mgn_buf* d, mgn_buf* c, uint32_t m, uint32_t steps) {
  if (!ctx || !weights || count == 0) return fail(ctx, MGN_EINVAL, "null argument or no weights");
  for (uint32_t i = 0; i < steps; i++) {
    const mgn_status st = matmul_impl(ctx, a, a_is_f16 != 0, weights[i % count], d, c, m);
    if (st != MGN_OK) return st;
  }
  return MGN_OK;
}

mgn_status mgn_weight_read_loop(mgn_ctx* ctx, const mgn_weight* const* weights, size_t count, uint32_t steps, int pattern) {
  if (!ctx || !weights || count == 0) return fail(ctx, MGN_EINVAL, "null argument or no weights");
  if (pattern != 0 && pattern != 1) return fail(ctx, MGN_EINVAL, "unknown read pattern");
  for (size_t i = 0; i < count; i++)
    if (!weights[i]) return fail(ctx, MGN_EINVAL, "null weight");
  for (uint32_t i = 0; i < steps; i++) {
    // the sink is the first word of the split-K workspace, which holds nothing between launches
    const int e = mgn::launch_read_probe(ctx->stream, view_of(weights[i % count]), ctx->num_cus, (uint32_t*)ctx->scratch, pattern);
    if (e != 0) return fail(ctx, MGN_EHIP, hipGetErrorString((hipError_t)e));
  }
  return MGN_OK;
}

mgn_status mgn_engine_clock_mhz(mgn_ctx* ctx, int loaded, float* mhz, float* cycles_per_round) {
  if (!ctx || !mhz) return fail(ctx, MGN_EINVAL, "null argument");
  // (the first bytes of the split-K workspace hold nothing between launches)
  const int rc = mgn::launch_clock_probe(ctx->stream, (uint64_t*)ctx->scratch, loaded ? ctx->num_cus : 0);
  if (rc != 0) return hip_fail(ctx, "clock probe launch", (hipError_t)rc);
  uint64_t host[3] = {0, 0, 0};
  MGN_HIP(ctx, hipMemcpyAsync(host, ctx->scratch, sizeof(host), hipMemcpyDeviceToHost, ctx->stream));
  MGN_HIP(ctx, hipStreamSynchronize(ctx->stream));
  *mhz = host[1] ? 100.0f * (float)host[0] / (float)host[1] : 0.0f;
  if (cycles_per_round) *cycles_per_round = loaded && host[2] ? (float)host[0] / (float)host[2] : 0.0f;
  return MGN_OK;
}

// ---- chains ----

mgn_status mgn_chain_create(mgn_ctx* ctx, const mgn_chain_stage* stages, size_t count, uint32_t m, mgn_chain** out) {
  if (!ctx || !stages || !out) return fail(ctx, MGN_EINVAL, "null argument");
  *out = nullptr;
  if (count == 0 || count > 4096) return fail(ctx, MGN_EINVAL, "a chain holds 1 to 4096 stages");
  if (m != 1) return fail(ctx, MGN_EUNSUPPORTED, "chains serve one activation row (M = 1)");
  if (ctx->shared_device) return fail(ctx, MGN_EUNSUPPORTED, "chains need the device to themselves (mgn_ctx_set_shared_device)");
  const int chain_cus = ctx->num_cus;
  std::vector<mgn::ChainStageDev> dev(count);
  std::vector<int> a_from(count, -1), d_from(count, -1);
  std::vector<char> has_reader(count, 0);
  size_t lds = 0;
  uint32_t grid = 1;
  const mgn_fmt fmt = stages[0].w ? stages[0].w->fmt : MGN_FMT_Q4;
  for (size_t j = 0; j < count; j++) {
    const mgn_chain_stage& st = stages[j];
    if (!st.w || !st.a || !st.c) return fail(ctx, MGN_EINVAL, "a stage lacks its weight, activations or output");
    if (st.prologue < MGN_PROLOGUE_NONE || st.prologue > MGN_PROLOGUE_SWIGLU) return fail(ctx, MGN_EINVAL, "unknown prologue");
    if (st.n_ops > 8 || (st.n_ops > 0 && !st.ops)) return fail(ctx, MGN_EINVAL, "an epilogue has at most 8 operations");
    const size_t k = st.w->rows, n = st.w->cols;
    if (st.a->bytes / 4 < (st.prologue == MGN_PROLOGUE_SWIGLU ? 2 * k : k)) return fail(ctx, MGN_EINVAL, "A is smaller than its row");
    if (st.prologue == MGN_PROLOGUE_RMS_NORM && (!st.norm_weight || st.norm_weight->bytes / 4 < k))
      return fail(ctx, MGN_EINVAL, "norm weight is missing or shorter than K floats");
    if (st.c->bytes / 4 < n) return fail(ctx, MGN_EINVAL, "C is smaller than N floats");
    if (st.d && st.d->bytes / 4 < n) return fail(ctx, MGN_EINVAL, "D is smaller than N floats");
    if (st.c == st.a || st.c->ptr == st.a->ptr) return fail(ctx, MGN_EINVAL, "C must not alias A");
    if (st.w->fmt != fmt) return fail(ctx, MGN_EUNSUPPORTED, "the stages of a chain share one weight format");
    mgn::ChainStageDev& d = dev[j];
    d = mgn::ChainStageDev{};
    d.meta = st.w->meta, d.quants = st.w->quants, d.k = (uint32_t)k, d.n = (uint32_t)n;
    d.pro = (uint32_t)st.prologue, d.eps = st.eps;
    d.norm_w = st.prologue == MGN_PROLOGUE_RMS_NORM ? (const float*)st.norm_weight->ptr : nullptr;
    for (size_t i = 0; i < st.n_ops; i++) {
      if (st.ops[i] < MGN_UNARY_RELU || st.ops[i] > MGN_UNARY_SILU) return fail(ctx, MGN_EINVAL, "unknown unary operation in the epilogue");
      d.epilogue |= (uint32_t)st.ops[i] << (4 * i);
    }
    d.c = (float*)st.c->ptr;
    // the latest earlier stage that writes what this one reads
    for (size_t p = 0; p < j; p++) {
      if (stages[p].c->ptr == st.a->ptr) a_from[j] = (int)p;
      if (st.d && stages[p].c->ptr == st.d->ptr) d_from[j] = (int)p;
      if (stages[p].c->ptr == st.c->ptr) return fail(ctx, MGN_EUNSUPPORTED, "two stages of a chain write the same buffer");
    }
    if (a_from[j] >= 0) has_reader[a_from[j]] = 1;
    if (d_from[j] >= 0) has_reader[d_from[j]] = 1;
  }
  // Phases: consecutive stages that read nothing from each other share the workgroups between
  // them (in proportion to their column quads), so a workgroup serves one stage per phase and the
  // chain's length in hand-overs is its number of phases (a decode layer: q, k, v and o together,
  // then gate | up, then down).
  for (size_t p0 = 0; p0 < count;) {
    size_t p1 = p0 + 1;
    while (p1 < count && a_from[p1] < (int)p0 && d_from[p1] < (int)p0 && (int)(p1 - p0) < chain_cus) p1++;
    uint64_t quads = 0;
    for (size_t j = p0; j < p1; j++) quads += (dev[j].n + 3) / 4;
    uint32_t first = 0;
    for (size_t j = p0; j < p1; j++) {
      const uint64_t mine = (dev[j].n + 3) / 4;
      const uint32_t left_stages = (uint32_t)(p1 - j - 1);
      uint32_t share = (uint32_t)std::max<uint64_t>(1, (uint64_t)chain_cus * mine / quads);
      share = std::min<uint32_t>(share, (uint32_t)chain_cus - first - left_stages);  // every later stage of the phase keeps at least one
      size_t need = 0;
      if (!mgn::plan_chain_stage((int)fmt, (int)share, &dev[j], &need))
        return fail(ctx, MGN_EUNSUPPORTED, "stage " + std::to_string(j) + " is not served by the chain kernel (Q4, K <= 16384)");
      dev[j].wg_first = first;
      first += dev[j].wgs;
      lds = std::max(lds, need);
      grid = std::max(grid, first);
    }
    p0 = p1;
  }
  // A buffer that some stage reads as written before the launch must not be written by any stage:
  // the workgroups are not in step, and one that is ahead would overwrite what another still reads.
  for (size_t j = 0; j < count; j++) {
    const void* ext[3] = {a_from[j] < 0 ? stages[j].a->ptr : nullptr, (stages[j].d && d_from[j] < 0) ? stages[j].d->ptr : nullptr,
                          stages[j].norm_weight ? stages[j].norm_weight->ptr : nullptr};
    for (size_t p = 0; p < count; p++)
      for (const void* e : ext)
        if (e && stages[p].c->ptr == e) return fail(ctx, MGN_EUNSUPPORTED, "a stage writes a buffer that the chain reads as its input");
  }
  // slots for the outputs that later stages read
  std::vector<size_t> slot_at(count, 0);
  size_t slot_words = 0;
  for (size_t j = 0; j < count; j++)
    if (has_reader[j]) {
      slot_at[j] = slot_words;
      slot_words += align_up(dev[j].n, 64);
    }
  if (slot_words > 0x3FFFFFFFu) return fail(ctx, MGN_EUNSUPPORTED, "chain workspace too large");
  auto* ch = new (std::nothrow) mgn_chain();
  if (!ch) return fail(ctx, MGN_ENOMEM, "out of host memory");
  ch->fmt = (int)fmt, ch->nstages = (uint32_t)count, ch->grid = grid, ch->lds = lds, ch->slot_words = (uint32_t)slot_words;
  const size_t table_bytes = align_up(count * sizeof(mgn::ChainStageDev), 256);
  const size_t total = 2 * table_bytes + 2 * slot_words * 4 + 256;
  hipError_t e = hipMalloc(&ch->dev, total);
  if (e != hipSuccess) {
    delete ch;
    return e == hipErrorOutOfMemory ? fail(ctx, MGN_ENOMEM, "out of device memory") : hip_fail(ctx, "hipMalloc", e);
  }
  ch->tables[0] = (mgn::ChainStageDev*)ch->dev;
  ch->tables[1] = (mgn::ChainStageDev*)((char*)ch->dev + table_bytes);
  ch->slots[0] = (uint32_t*)((char*)ch->dev + 2 * table_bytes);
  ch->slots[1] = ch->slots[0] + slot_words;
  std::vector<mgn::ChainStageDev> both(2 * count);
  for (int set = 0; set < 2; set++)
    for (size_t j = 0; j < count; j++) {
      mgn::ChainStageDev d = dev[j];
      const mgn_chain_stage& st = stages[j];
      float* const base = (float*)ch->slots[set];
      d.a = a_from[j] >= 0 ? base + slot_at[a_from[j]] : (const float*)st.a->ptr;
      d.a_poll = a_from[j] >= 0;
      d.d = !st.d ? nullptr : d_from[j] >= 0 ? base + slot_at[d_from[j]] : (const float*)st.d->ptr;
      d.d_poll = st.d && d_from[j] >= 0;
      d.c_slot = has_reader[j] ? base + slot_at[j] : nullptr;
      both[set * count + j] = d;
    }
  e = hipMemcpyAsync(ch->tables[0], both.data(), count * sizeof(mgn::ChainStageDev), hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess)
    e = hipMemcpyAsync(ch->tables[1], both.data() + count, count * sizeof(mgn::ChainStageDev), hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess && slot_words) e = hipMemsetAsync(ch->slots[0], 0xFF, 2 * slot_words * 4, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);  // `both` goes out of scope
  if (e != hipSuccess) {
    (void)hipFree(ch->dev);
    delete ch;
    return hip_fail(ctx, "chain upload", e);
  }
  ctx->chains.push_back(ch);
  *out = ch;
  return MGN_OK;
}

mgn_status mgn_chain_run(mgn_ctx* ctx, mgn_chain* chain) {
  if (!ctx || !chain) return fail(ctx, MGN_EINVAL, "null argument");
  const uint32_t set = chain->runs & 1u;
  const int rc = mgn::launch_chain(ctx->stream, ctx->device, chain->fmt, chain->tables[set], chain->nstages, chain->grid, chain->lds,
                                   chain->slots[set ^ 1u], chain->slot_words, ctx->spin_limit, ctx->range_flag_dev + 1);
  if (rc != 0) return hip_fail(ctx, "chain launch", (hipError_t)rc);
  chain->runs++;
  return MGN_OK;
}

void mgn_chain_free(mgn_ctx* ctx, mgn_chain* chain) {
  if (!chain) return;
  if (ctx) {
    (void)hipStreamSynchronize(ctx->stream);
    for (size_t i = 0; i < ctx->chains.size(); i++)
      if (ctx->chains[i] == chain) {
        ctx->chains.erase(ctx->chains.begin() + (long)i);
        break;
      }
  }
  if (chain->dev) (void)hipFree(chain->dev);
  delete chain;
}

// ---- timing ----

mgn_status mgn_timer_start(mgn_ctx* ctx) {
  if (!ctx) return MGN_EINVAL;
  MGN_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
  return MGN_OK;
}

mgn_status mgn_timer_stop(mgn_ctx* ctx, float* elapsed_ms) {
  if (!ctx || !elapsed_ms) return fail(ctx, MGN_EINVAL, "null argument");
  MGN_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
  MGN_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
  MGN_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
  return check_range_flag(ctx);
}

}  // extern "C"
