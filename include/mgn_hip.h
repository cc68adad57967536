/*
 * mgn_hip.h — C ABI of libmgn_hip: MI355X (gfx950) kernels for meganeura's
 * quantized matmul path, i.e. `matmul` nodes whose B operand is a
 * `parameter_q4` / `parameter_q8` weight.
 *
 * This is the boundary a host runtime binds in place of its own GPU dispatch
 * for those nodes.  Each entry point names the reference interface it stands
 * in for (paths relative to the reference checkout, kvark/meganeura v0.2.0).
 *
 * Conventions
 *   - every call returns an mgn_status; nothing throws or aborts across the ABI
 *     (the reference panics: `unknown parameter`, `rows % 32`; here those are
 *     MGN_EINVAL / MGN_ENOTFOUND and mgn_last_error() holds the message);
 *   - handles are opaque and owned by the caller, who frees them with the
 *     matching *_free / *_destroy before destroying the context;
 *   - one HIP stream per context; matmul calls are asynchronous on it, like
 *     Session::step (src/runtime.rs:2843), and mgn_sync is Session::wait
 *     (src/runtime.rs:2835);
 *   - a context is thread-compatible, not thread-safe (the reference's Session
 *     is `&mut self` everywhere);
 *   - matrices are row-major; a weight is W[K,N] with K = rows = the reduction
 *     dimension, which must be a multiple of 32 (src/runtime.rs:2037-2040).
 */
#ifndef MGN_HIP_H
#define MGN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mgn_status {
  MGN_OK = 0,
  MGN_EINVAL = 1,    /* bad argument: null handle, rows % 32 != 0, size mismatch */
  MGN_ENOMEM = 2,    /* host or device allocation failed */
  MGN_EHIP = 3,      /* a HIP runtime call failed; see mgn_last_error */
  MGN_ENOTFOUND = 4, /* unknown name (session layer) */
  MGN_ENODEVICE = 5, /* no usable gfx950 device */
  MGN_EUNSUPPORTED = 6, /* a fused entry point asked for a shape its kernel does not serve */
  MGN_ERANGE = 7, /* reported by the next synchronising call: an f32 activation too large for the kernel
                    that ran (|x| >= 65504 on MGN_ROUTE_GEMM_MFMA, M >= 5, which only a context set to
                    MGN_ACT_FP16_RANGE or a forced route uses for f32); outputs of that call are wrong */
  MGN_ETIMEOUT = 8 /* reported by the next synchronising call: a workgroup that adds up the partial sums of a
                    matmul whose K is cut into parts gave up waiting for another part (its wait is bounded, so
                    every kernel ends); outputs since the last synchronisation are not valid.  The library
                    has emptied its hand-over workspace again when the call returns. */
} mgn_status;

/* compile::WeightFormat::{Q4,Q8} (src/compile.rs:8-29), graph::DType::{Q4_0,Q8_0}
 * (src/graph.rs:6-27).  Q4 is the asymmetric scale+min format the reference
 * stores under the name Q4_0. */
typedef enum mgn_fmt { MGN_FMT_Q4 = 0, MGN_FMT_Q8 = 1 } mgn_fmt;

/* Which kernel family serves a matmul; MGN_ROUTE_AUTO is what a runtime uses.
 * The others exist so that tests can drive every kernel at every shape. */
typedef enum mgn_route {
  MGN_ROUTE_AUTO = 0,
  MGN_ROUTE_GENERIC = 1,   /* scalar f32 fallback, any M */
  MGN_ROUTE_GEMV_VALU = 2, /* streaming dequant-GEMV on the vector ALU, M <= 4 */
  MGN_ROUTE_GEMV_MFMA = 3, /* streaming dequant-GEMV, raw quants x split-fp16 activations on MFMA, M <= 4 */
  MGN_ROUTE_GEMM_MFMA = 4, /* tiled dequant-GEMM on MFMA (32x32x16 tiles), larger M: the fast form, for weights whose
                              block minima stay below 2047 (Q8: scales below 15.99) and f32 activations below 65504 */
  MGN_ROUTE_TILE_MFMA = 5  /* tiled dequant-GEMM on MFMA (16x16x32 tiles, activations rescaled per row and 256-element
                              K slice): any finite weight, activations below 2^100 in magnitude (a slice that holds a
                              larger one gives its row non-finite results), larger M; the automatic choice for weights
                              outside the range of the form above */
} mgn_route;

typedef struct mgn_ctx mgn_ctx;
typedef struct mgn_buf mgn_buf;
typedef struct mgn_weight mgn_weight;

/* ---- context: blade_graphics::Context::init + Session::new
 *      (src/runtime.rs:1513-1524, 2012-2024; device chosen by index as
 *      MEGANEURA_DEVICE_ID does). */
mgn_status mgn_ctx_create(int device_id, mgn_ctx** out);
void mgn_ctx_destroy(mgn_ctx* ctx);
/* Message of the last failed call on this context ("" if none).  With a null
 * ctx: the message of the last failed mgn_ctx_create on this thread. */
const char* mgn_last_error(const mgn_ctx* ctx);
/* Session::wait (src/runtime.rs:2835-2841). */
mgn_status mgn_sync(mgn_ctx* ctx);
/* What the context may assume about f32 activations of matmuls with M >= 5.
 *   MGN_ACT_ANY (default): nothing.  Those matmuls run on the kernels that rescale every
 *     256-element slice of a row by a power of two before splitting it into fp16 pairs (hi + lo:
 *     22 significant bits relative to the slice's largest magnitude, products with the quants
 *     exact on those): f32 of any magnitude below 2^100 is served with the same relative accuracy,
 *     inf and NaN stay in their rows, and a slice holding a magnitude of 2^100 or more makes its
 *     row's results non-finite (never a finite wrong number) -- in effect what the reference's f32
 *     arithmetic on the scalar ALUs gives (src/shaders/matmul.wgsl:43-90) up to that magnitude.
 *   MGN_ACT_FP16_RANGE: the caller promises |x| < 65504 and accepts that values below 2^-4 are
 *     carried with an absolute step of 2^-25 instead of a relative one.  The matmuls may then run
 *     on the 32x32 tiled kernel, which splits without rescaling and is faster on some shapes
 *     (up to 1.3x, mostly long K at many rows); an activation that breaks the promise is
 *     detected while it is staged and the next synchronising call returns MGN_ERANGE.
 * fp16 activations (mgn_matmul_q_f16a) and M <= 4 never depend on this. */
typedef enum mgn_act_range { MGN_ACT_ANY = 0, MGN_ACT_FP16_RANGE = 1 } mgn_act_range;
/* Whether other work runs on the device beside this context's launches (other contexts, other
 * processes).  Two kinds of launch let all their workgroups wait for each other, which needs them
 * resident on the device together: a chain (mgn_chain_*), and a matmul whose K parts are added up
 * by all parts, a share each.  Two such kernels at once can take each other's compute units and
 * both stall until their bounded waits give up (MGN_ETIMEOUT at the next synchronising call, no
 * hang, results not to be used).  shared = 0 (default): the context has the device to itself while
 * it computes, and both are used.  shared != 0: neither is; chains are refused with
 * MGN_EUNSUPPORTED and K parts are added up by the part that is dispatched last, which waits only
 * for workgroups dispatched before it.  No counterpart in the reference (one Session per device). */
mgn_status mgn_ctx_set_shared_device(mgn_ctx* ctx, int shared);
mgn_status mgn_ctx_set_activation_range(mgn_ctx* ctx, mgn_act_range range);
/* ---- plain device buffers: the reference allocates every plan buffer
 *      zero-filled (src/runtime.rs:1737-1755) and moves data with memcpy
 *      through mapped memory (upload_buffer 2552-2558, read_buffer 2623-2629). */
mgn_status mgn_buf_alloc(mgn_ctx* ctx, size_t bytes, mgn_buf** out); /* zero-filled */
void mgn_buf_free(mgn_ctx* ctx, mgn_buf* buf);
size_t mgn_buf_size(const mgn_buf* buf);
/* Raw device address, for callers that share the buffer with their own kernels. */
void* mgn_buf_device_ptr(const mgn_buf* buf);
/* Session::set_input / f32 set_parameter (src/runtime.rs:2496-2504, 2344).
 * Ordered after earlier work on the context's stream; returns when src may be reused. */
mgn_status mgn_buf_upload(mgn_ctx* ctx, mgn_buf* buf, size_t offset, const void* src, size_t bytes);
/* Session::read_output / read_buffer (src/runtime.rs:2612-2629); waits for the stream. */
mgn_status mgn_buf_download(mgn_ctx* ctx, const mgn_buf* buf, size_t offset, void* dst, size_t bytes);

/* Device-to-device copy on the context's stream (asynchronous).  The reference has no
 * such call (its buffers are host-mapped); it is here for callers that stage data on
 * the device, and it gives profilers a copy of known size to calibrate byte counters. */
mgn_status mgn_buf_copy(mgn_ctx* ctx, mgn_buf* dst, const mgn_buf* src, size_t bytes);

/* ---- block quantizers on the host, reference byte layout
 *      TensorType::size_bytes (src/graph.rs:52-68): 20 or 36 bytes per 32-element block. */
size_t mgn_packed_size(mgn_fmt fmt, size_t rows, size_t cols);
/* quantize_q4_0 / quantize_q8_0 (src/runtime.rs:2035-2102, 2143-2188), bit-exact.
 * w: f32 [rows, cols] row-major.  out: mgn_packed_size bytes. */
mgn_status mgn_quantize_ref(mgn_fmt fmt, const float* w, size_t rows, size_t cols, uint8_t* out);
/* dequantize_q4_0 / dequantize_q8_0 (src/runtime.rs:2105-2138, 2191-2215), bit-exact. */
mgn_status mgn_dequantize_ref(mgn_fmt fmt, const uint8_t* in, size_t rows, size_t cols, float* out);

/* ---- quantized weights on the device
 * Session::set_parameter for a Q4/Q8 parameter (src/runtime.rs:2327-2345):
 * quantize f32 [rows, cols] and place it in device memory.  The device layout
 * is private; mgn_weight_export_ref gives back the reference's bytes.  (The values are
 * uploaded and packed by the device quantizer, whose bytes equal mgn_quantize_ref's; when the
 * device has no room for the f32 copy, the host packs and the bytes are uploaded.) */
mgn_status mgn_weight_create(mgn_ctx* ctx, mgn_fmt fmt, const float* w, size_t rows, size_t cols,
                             mgn_weight** out);
/* Same from bytes already in the reference layout (what load_checkpoint copies
 * back into a Q4/Q8 buffer, src/runtime.rs:4256-4265). */
mgn_status mgn_weight_create_packed(mgn_ctx* ctx, mgn_fmt fmt, const uint8_t* packed, size_t rows,
                                    size_t cols, mgn_weight** out);
/* A weight stored [N, K] row-major: the B operand of Graph::matmul_bt (src/graph.rs:809-817,
 * lowering src/compile.rs:1447-1485), which is how weight-tied lm_heads keep their embedding
 * table (models/smollm2.rs:413-414).  Blocks run along K -- contiguous in this storage -- so
 * the result is the same weight, byte for byte, as mgn_weight_create on the transposed [K, N]
 * matrix, and C = A x B^T is then mgn_matmul_q with it.  (The reference's set_parameter blocks
 * such a parameter along shape[0] = N while its shader reads it along K, src/compile.rs:1233-1239;
 * that inconsistency is not reproduced.)  mgn_quantize_ref_nk is the host-only form; its
 * output has the reference byte layout for rows = K, cols = N. */
mgn_status mgn_quantize_ref_nk(mgn_fmt fmt, const float* w_nk, size_t n_rows, size_t k_cols, uint8_t* out);
mgn_status mgn_weight_create_nk(mgn_ctx* ctx, mgn_fmt fmt, const float* w_nk, size_t n_rows, size_t k_cols,
                                mgn_weight** out);
/* Same from an f32 [rows, cols] matrix already on the device: the block
 * quantizer runs as a kernel, bit-exact with mgn_quantize_ref. */
mgn_status mgn_weight_create_device(mgn_ctx* ctx, mgn_fmt fmt, const mgn_buf* w_f32, size_t rows,
                                    size_t cols, mgn_weight** out);
void mgn_weight_free(mgn_ctx* ctx, mgn_weight* w);
mgn_status mgn_weight_info(const mgn_weight* w, mgn_fmt* fmt, size_t* rows, size_t* cols);
/* Device-side dequantization to host f32 [rows, cols]; must equal
 * mgn_dequantize_ref(mgn_quantize_ref(w)) bit for bit. */
mgn_status mgn_weight_dequantize(mgn_ctx* ctx, const mgn_weight* w, float* out_host);
/* Device weight back to the reference byte layout (save_checkpoint's dump of a
 * packed buffer, src/runtime.rs:4218-4226). */
mgn_status mgn_weight_export_ref(mgn_ctx* ctx, const mgn_weight* w, uint8_t* out_packed);

/* Pre-quantized weights on disk.  The reference's save_checkpoint writes a quantized
 * parameter's packed bytes under an F32 label and load_checkpoint copies them back blindly
 * (src/runtime.rs:4218-4226, 4256-4265); this is a tagged container instead: 40-byte
 * little-endian header "MGNQ", version 1, format, rows, cols, payload size, then the
 * reference-layout packed bytes, so a file is independent of the private device layout and a
 * weight never has to be re-quantized at start-up.  Load: MGN_ENOTFOUND if the file cannot be
 * opened, MGN_EINVAL for a foreign, truncated or inconsistent file. */
mgn_status mgn_weight_save(mgn_ctx* ctx, const mgn_weight* w, const char* path);
mgn_status mgn_weight_load(mgn_ctx* ctx, const char* path, mgn_weight** out);

/* ---- the matmul itself
 * C[M,N] = A[M,K] x W (+ D[M,N] when d is not null).  A, C, D: f32 row-major
 * device buffers.  Stands in for the ShaderEntry::{MatMul, MatMulGemv,
 * FusedMatMulAdd, MatMulGemvAdd} dispatches whose weight_format is Q4/Q8
 * (src/compile.rs:1381-1421, 1486-1524; bind_dispatch src/runtime.rs:3073-3122).
 * The kernel family is chosen from (M, K, N) inside, as compile.rs:1390 and
 * runtime.rs:1634 do for the reference.  Asynchronous on the context's stream.
 * c must not alias a; c may alias d. */
mgn_status mgn_matmul_q(mgn_ctx* ctx, const mgn_buf* a, const mgn_weight* w, const mgn_buf* d,
                        mgn_buf* c, uint32_t m);
/* The same with fp16 activations A[M,K] (prefill): fp16 operands on MFMA with
 * f32 accumulation, the role matmul_coop.wgsl plays for unquantized weights
 * (src/codegen.rs:1168-1176; quantized weights are excluded from it in the
 * reference, src/runtime.rs:1634).  At M <= 4 the decode kernel takes it and
 * widens the halves while it stages the activations. */
mgn_status mgn_matmul_q_f16a(mgn_ctx* ctx, const mgn_buf* a_f16, const mgn_weight* w,
                             const mgn_buf* d, mgn_buf* c, uint32_t m);

/* mgn_matmul_q for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Shapes whose K is cut into parts for different workgroups keep their partial sums in a
 * workspace (with arrival counters, or as hand-over words that read "empty" until a part has
 * stored its sum); mgn_matmul_q uses workspaces the context allocated, this entry uses an
 * array inside the library's own device image (MGN_STATIC_WORKSPACE_BYTES = 4 MiB of partial
 * sums, plus 4096 counters, plus as many bytes of hand-over words again, held on every device the
 * library runs on until the process ends) and calls no hipMalloc / hipFree or any other
 * allocating routine.  Same plan, same kernels and bit-identical results as mgn_matmul_q;
 * MGN_EUNSUPPORTED, with the byte counts in mgn_last_error, when the shape's partial sums or
 * hand-over words do not fit the static array.  All contexts of a device share the array: calls
 * that overlap on one device (two contexts, two threads) race; calls on one context are ordered by
 * its stream.  The array keeps the last call's contents: the counters are cleared and the
 * hand-over words a launch will use are set to the empty pattern by a small fill kernel in front
 * of every launch that uses them. */
#define MGN_STATIC_WORKSPACE_BYTES ((size_t)4 << 20)
mgn_status mgn_matmul_q_static(mgn_ctx* ctx, const mgn_buf* a, const mgn_weight* w, const mgn_buf* d,
                               mgn_buf* c, uint32_t m);

/* The same followed by unary operations on every output element, first to last:
 * C = f_n(... f_1(A x W + D)).  Stands in for a matmul dispatch that carries an epilogue
 * (compile.rs:915-1035 fuse_epilogues folds a Relu / Sigmoid / Neg / Silu that is the only
 * reader of a matmul's output into the matmul; formulas codegen.rs:62-100).  The reference
 * builds that pipeline with the f32 weight format even when the weight is quantized
 * (codegen.rs:617-642); here the epilogue rides on the quantized kernels.  n_ops <= 8. */
typedef enum mgn_unary {
  MGN_UNARY_NONE = 0,
  MGN_UNARY_RELU = 1,    /* max(v, 0) */
  MGN_UNARY_SIGMOID = 2, /* 1 / (1 + exp(-v)) */
  MGN_UNARY_NEG = 3,     /* -v */
  MGN_UNARY_SILU = 4     /* v / (1 + exp(-v)) */
} mgn_unary;
mgn_status mgn_matmul_q_epilogue(mgn_ctx* ctx, const mgn_buf* a, const mgn_weight* w, const mgn_buf* d,
                                 mgn_buf* c, uint32_t m, const mgn_unary* ops, size_t n_ops);
/* C[M,N] = A^T x W (+ D): the MatMulAT / FusedMatMulATAdd dispatches with a quantized B
 * (src/compile.rs:1423-1445, 1526-1549; codegen.rs gen_matmul_at).  a_t holds A as [K, M]
 * row-major, M = m.  The activations are transposed into a staging area of the context
 * (allocated or grown on the first call that needs it, kept afterwards) and the call then
 * is mgn_matmul_q_epilogue's: ops / n_ops as there, NULL / 0 for none.  c must not alias a_t. */
mgn_status mgn_matmul_q_at(mgn_ctx* ctx, const mgn_buf* a_t, const mgn_weight* w, const mgn_buf* d, mgn_buf* c,
                           uint32_t m, const mgn_unary* ops, size_t n_ops);

/* What mgn_matmul_q would launch for a shape, without a device: the kernel family the
 * automatic choice takes (the analogue of reading compile.rs:1390 and runtime.rs:1634 for the
 * reference) and the launch geometry.  For logs, and for checking the planner on the host.
 * `num_cus` is the device's compute-unit count (256 on MI355X); the workspace is assumed to be
 * the one every context owns.  a_is_f16: 0 = f32 activations of any magnitude (a context's
 * default), 1 = fp16 activations, 2 = f32 activations promised to lie in the fp16 range
 * (MGN_ACT_FP16_RANGE).  MGN_EINVAL for shapes no weight can have. */
typedef struct mgn_plan_info {
  int route;              /* mgn_route (never MGN_ROUTE_AUTO) */
  uint32_t grid[3];       /* workgroups: GEMV (column groups, K parts, 1); tiled routes (K parts, column groups, row
                           * groups) -- the LDS-resident MGN_ROUTE_TILE_MFMA form launches them as (column groups x
                           * row groups, rounded up to a multiple of 8 when K is in parts; K parts) */
  uint32_t threads;       /* per workgroup */
  uint32_t lds_bytes;     /* dynamic LDS per workgroup */
  uint32_t waves_n;       /* column quads (GEMV), 32-column tiles (MGN_ROUTE_GEMM_MFMA) or 16-column tiles
                           * (MGN_ROUTE_TILE_MFMA) per workgroup */
  uint32_t k_splits;      /* waves that share a quad / tile inside a workgroup */
  uint32_t k_parts;       /* workgroups that share a column group; > 1: partial sums through the workspace */
  uint32_t steps;         /* GEMV: 16-block steps per wave; tiled: 8-block chunks (slices of 256 elements) per wave and part */
  uint32_t quads_per_wave; /* GEMV: column quads per wave; MGN_ROUTE_TILE_MFMA: 0 for the form that keeps the
                            * activation images in LDS, else the launches the rows are spread over
                            * (more than one when their activation images exceed the workspace) */
  uint32_t full_steps;    /* GEMV: 1 when no step needs masking; MGN_ROUTE_TILE_MFMA: row tiles of 16 rows per workgroup */
  uint32_t tail_blocks;   /* GEMV only: 0, or the K blocks per column beyond `steps` full steps that the wave's
                           * quads share one more step for (K = 32 * (16 * steps + tail_blocks)) */
  uint64_t workspace_bytes; /* partial sums held in the context's workspace */
} mgn_plan_info;
mgn_status mgn_matmul_q_plan(mgn_fmt fmt, uint32_t m, uint64_t k, uint64_t n, int a_is_f16, int num_cus,
                             mgn_plan_info* out);

/* Two neighbours of the decode-time matmul folded into its activation staging, each
 * standing in for a dispatch pair of the reference's plan (M <= 4, f32 activations):
 *   RmsNorm then MatMul[Gemv][Add]   (src/shaders/rms_norm.wgsl:1-57; models/smollm2.rs:340-341,396):
 *     C = (x * rsqrt(mean(x^2) + eps) * norm_weight) x W (+ D), x[M,K], norm_weight[K];
 *   SwiGLUConcat then MatMul[Gemv][Add]   (src/shaders/swiglu_concat.wgsl:20-32; compile.rs:1814-1830):
 *     C = (gate * sigmoid(gate) * up) x W (+ D), gate_up[M,2K] = gate | up.
 * MGN_EUNSUPPORTED when the shape is not served by the kernel that can fuse (run the two
 * dispatches separately then); mgn_matmul_q_can_fuse tells beforehand (1 = yes). */
mgn_status mgn_matmul_q_rms_norm(mgn_ctx* ctx, const mgn_buf* x, const mgn_buf* norm_weight, float eps,
                                 const mgn_weight* w, const mgn_buf* d, mgn_buf* c, uint32_t m);
mgn_status mgn_matmul_q_swiglu(mgn_ctx* ctx, const mgn_buf* gate_up, const mgn_weight* w,
                               const mgn_buf* d, mgn_buf* c, uint32_t m);
int mgn_matmul_q_can_fuse(mgn_ctx* ctx, const mgn_weight* w, uint32_t m);

/* One launch for up to three decode matmuls that read the same activations (the q, k and v
 * projections: three MatMulGemv dispatches on one normed x, models/smollm2.rs:340-348), with the
 * same optional prologue.  Weights must share K and the format; each item has its own output
 * and optional residual.  C_j = prologue(A) x W_j (+ D_j).  Same availability rule and error
 * as the fused entries above. */
typedef enum mgn_prologue {
  MGN_PROLOGUE_NONE = 0,
  MGN_PROLOGUE_RMS_NORM = 1, /* A = x[M,K], with norm_weight[K] and eps */
  MGN_PROLOGUE_SWIGLU = 2    /* A = gate_up[M,2K] */
} mgn_prologue;
typedef struct mgn_matmul_item {
  const mgn_weight* w;
  const mgn_buf* d; /* may be null */
  mgn_buf* c;
} mgn_matmul_item;
mgn_status mgn_matmul_q_batch(mgn_ctx* ctx, const mgn_buf* a, mgn_prologue prologue, const mgn_buf* norm_weight,
                              float eps, const mgn_matmul_item* items, size_t count, uint32_t m);

/* ---- a whole chain of dependent decode matmuls in ONE launch.
 * The reference encodes every dispatch of a step into one command buffer and submits it once
 * (Session::step, src/runtime.rs:2843-2959); a decode step is a chain of small dependent matmuls
 * (src/models/smollm2.rs:392-405).  A chain object stands in for a run of such dispatches with
 * M = 1: stage j computes C_j = f_j(prologue_j(A_j) x W_j + D_j), where A_j and D_j may be outputs
 * of earlier stages of the same chain (recognised by the buffer handle) or buffers written before
 * the launch.  One resident launch walks the stages; outputs that later stages read travel through
 * a workspace of the chain, and a reader polls the data itself (bounded: MGN_ETIMEOUT at the next
 * synchronising call if it ever gives up).  Every C_j is also written to the caller's buffer.
 * mgn_chain_create: MGN_EUNSUPPORTED when a stage is not served (m != 1, a Q8 weight, K beyond
 * 16384, two stages writing one buffer, a stage writing a buffer that the chain also reads as
 * written before the launch), or when the context shares its device (mgn_ctx_set_shared_device:
 * a chain's workgroups wait for each other): run the dispatches one by one then.  It allocates (tables and
 * workspace) and synchronises; mgn_chain_run allocates nothing and is asynchronous on the
 * context's stream.  The weights and buffers must outlive the chain; free it before them.
 * A chain must not be recorded into a HIP graph that is replayed: consecutive runs alternate
 * between two sets of workspace slots. */
typedef struct mgn_chain mgn_chain;
typedef struct mgn_chain_stage {
  const mgn_weight* w;
  const mgn_buf* a;           /* [1, K] activations ([1, 2K] = gate | up with MGN_PROLOGUE_SWIGLU) */
  mgn_prologue prologue;      /* what the activations go through first (mgn_matmul_q_rms_norm / _swiglu) */
  const mgn_buf* norm_weight; /* [K], MGN_PROLOGUE_RMS_NORM only */
  float eps;
  const mgn_buf* d;           /* residual [1, N], may be null */
  mgn_buf* c;                 /* [1, N] */
  const mgn_unary* ops;       /* unary operations on the output, first to last (mgn_matmul_q_epilogue), may be null */
  size_t n_ops;               /* at most 8 */
} mgn_chain_stage;
mgn_status mgn_chain_create(mgn_ctx* ctx, const mgn_chain_stage* stages, size_t count, uint32_t m, mgn_chain** out);
mgn_status mgn_chain_run(mgn_ctx* ctx, mgn_chain* chain);
void mgn_chain_free(mgn_ctx* ctx, mgn_chain* chain);

/* ---- GPU timing on the context's stream: Session::set_profiling +
 *      dump_gpu_timings (src/runtime.rs:1965, 2798-2832) reduced to one
 *      start/stop pair of HIP events. */
mgn_status mgn_timer_start(mgn_ctx* ctx);
mgn_status mgn_timer_stop(mgn_ctx* ctx, float* elapsed_ms); /* waits for the stop event */

/* Library version, and the gfx target the kernels were built for ("gfx950"). */
const char* mgn_version(void);
const char* mgn_built_for(void);

#ifdef __cplusplus
}
#endif
#endif /* MGN_HIP_H */
