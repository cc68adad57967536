/*
 * mgn_session.h — C ABI over the host-side mirror of meganeura's operator
 * surface for the quantized matmul path: Graph -> build_inference_session ->
 * Session::{set_parameter, set_input, step, wait, read_output}.
 *
 * Only what reaches a quantized `matmul` is mirrored: leaf nodes, matmul, add
 * (so that MatMul+Add fuses as in the reference), swiglu (so that gate/up
 * projections fuse into one wide matmul) and rms_norm.  A matmul whose weight
 * is plain f32 compiles into the plan (routing can be inspected) but is not
 * executed by this backend: build returns MGN_EINVAL for it.
 *
 * Paths cited are relative to the reference checkout.
 */
#ifndef MGN_SESSION_H
#define MGN_SESSION_H

#include "mgn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mgn_graph mgn_graph;
typedef struct mgn_session mgn_session;

/* compile::ShaderEntry values that can appear in a plan here
 * (src/compile.rs ShaderEntry; lowering at 1381-1421, 1486-1524, 1814-1830). */
typedef enum mgn_shader {
  MGN_SHADER_MATMUL = 0,
  MGN_SHADER_MATMUL_GEMV = 1,
  MGN_SHADER_FUSED_MATMUL_ADD = 2,
  MGN_SHADER_MATMUL_GEMV_ADD = 3,
  MGN_SHADER_ADD = 4,
  MGN_SHADER_SWIGLU = 5,
  MGN_SHADER_SWIGLU_CONCAT = 6,
  MGN_SHADER_RMS_NORM = 7,
  MGN_SHADER_MATMUL_BT = 8,      /* ShaderEntry::MatMulBT:     C = A x B^T, B stored [N, K] */
  MGN_SHADER_MATMUL_GEMV_BT = 9, /* ShaderEntry::MatMulGemvBT: its M = 1 form */
  MGN_SHADER_RELU = 10,          /* the unary entries fuse_epilogues can fold into a matmul */
  MGN_SHADER_SIGMOID = 11,
  MGN_SHADER_NEG = 12,
  MGN_SHADER_SILU = 13,
  MGN_SHADER_MATMUL_AT = 14,           /* ShaderEntry::MatMulAT: C = A^T x B, A stored [K, M] (src/compile.rs:1423-1445) */
  MGN_SHADER_FUSED_MATMUL_AT_ADD = 15, /* ShaderEntry::FusedMatMulATAdd: A^T x B + D (src/compile.rs:1526-1549) */
  MGN_SHADER_FUSED_MATMUL_BT_ADD = 16  /* ShaderEntry::FusedMatMulBTAdd: A x B^T + D (src/compile.rs:1551-1574) */
} mgn_shader;

/* compile::Dispatch (src/compile.rs:435-488), the fields this path uses.
 * weight_format: 0 = F32, 1 = Q4, 2 = Q8 (compile::WeightFormat). */
typedef struct mgn_dispatch_info {
  int32_t shader;          /* mgn_shader */
  uint32_t workgroups[3];  /* the grid the reference would launch */
  uint32_t params[4];      /* [m, k, n, 0] for matmuls, [m, n, k, 0] for the AT and BT forms, [len, 0, 0, 0] for unary entries */
  int32_t weight_format;
  uint32_t epilogue;       /* Dispatch::epilogue of a matmul: mgn_unary codes, four bits each, first in the low bits */
} mgn_dispatch_info;

/* Graph::new and the builders (src/graph.rs:714-795, 996-999).  Each builder
 * returns the new node id (>= 0) or a negative mgn_status; the message is in
 * mgn_graph_last_error.  Shapes are 2-D [rows, cols] (rms_norm weight: [cols]). */
mgn_graph* mgn_graph_new(void);
void mgn_graph_free(mgn_graph* g);
const char* mgn_graph_last_error(const mgn_graph* g);
int32_t mgn_graph_input(mgn_graph* g, const char* name, size_t rows, size_t cols);
int32_t mgn_graph_parameter(mgn_graph* g, const char* name, size_t rows, size_t cols);
int32_t mgn_graph_parameter_q4(mgn_graph* g, const char* name, size_t rows, size_t cols);
int32_t mgn_graph_parameter_q8(mgn_graph* g, const char* name, size_t rows, size_t cols);
int32_t mgn_graph_matmul(mgn_graph* g, int32_t a, int32_t b);
/* Graph::matmul_bt (src/graph.rs:809-817): a[M,K], b[N,K] -> [M,N].  With a quantized b the
 * parameter is blocked along K (see mgn_weight_create_nk). */
int32_t mgn_graph_matmul_bt(mgn_graph* g, int32_t a, int32_t b);
/* Graph::matmul_at (src/graph.rs:798-806): a[K,M], b[K,N] -> [M,N] = a^T x b; what the ONNX / NNEF
 * loaders emit for a Gemm with a transposed first operand (src/load/onnx.rs:607). */
int32_t mgn_graph_matmul_at(mgn_graph* g, int32_t a, int32_t b);
int32_t mgn_graph_add(mgn_graph* g, int32_t a, int32_t b);
int32_t mgn_graph_swiglu(mgn_graph* g, int32_t gate, int32_t up);
int32_t mgn_graph_rms_norm(mgn_graph* g, int32_t x, int32_t weight, float eps);
/* Graph::relu / sigmoid / neg / silu (src/graph.rs): kind is a mgn_unary.  A unary node that is
 * the only reader of a tiled matmul's output becomes that matmul's epilogue when the graph is
 * compiled (compile.rs:915-1035); otherwise it is a dispatch of its own. */
int32_t mgn_graph_unary(mgn_graph* g, int32_t kind, int32_t x);
mgn_status mgn_graph_set_outputs(mgn_graph* g, const int32_t* ids, size_t count);

/* compile only (optimize + compile_with, src/train.rs:272-340 without the GPU
 * step): works without a device, for routing checks such as
 * tests/gemv_parity.rs:32-52. */
mgn_status mgn_graph_compile(const mgn_graph* g, mgn_dispatch_info* out, size_t cap, size_t* count);

/* build_inference_session (src/train.rs:380-389). */
mgn_status mgn_build_inference_session(const mgn_graph* g, int device_id, mgn_session** out);
void mgn_session_free(mgn_session* s);
const char* mgn_session_last_error(const mgn_session* s);
/* Session::plan().dispatches (src/compile.rs:494-528). */
size_t mgn_session_num_dispatches(const mgn_session* s);
mgn_status mgn_session_dispatch_info(const mgn_session* s, size_t index, mgn_dispatch_info* out);
/* Session::set_parameter (src/runtime.rs:2327-2493): f32 data of rows*cols
 * elements; quantized on upload for Q4/Q8 parameters; feeds derived
 * (concatenated) parameters.  Unknown name: MGN_ENOTFOUND (the reference panics). */
mgn_status mgn_session_set_parameter(mgn_session* s, const char* name, const float* data, size_t len);
/* Session::set_input (src/runtime.rs:2496-2504). */
mgn_status mgn_session_set_input(mgn_session* s, const char* name, const float* data, size_t len);
/* Session::step / wait (src/runtime.rs:2843-2959, 2835-2841). */
mgn_status mgn_session_step(mgn_session* s);
mgn_status mgn_session_wait(mgn_session* s);
/* The reference records a step's dispatches into one command buffer and submits it once
 * (src/runtime.rs:2843-2959).  Here a step is captured into one HIP graph the second time it
 * runs after the weights were set and replayed from then on; `enable = 0` keeps every step as
 * individual launches.  Off by default: on MI355X a replayed chain of small kernels measured
 * ~15 % slower than the same launches issued one by one (29 vs 25 us for a 9-dispatch decode
 * layer), so it only pays when the host thread is the bottleneck.
 * mgn_session_graph_active reports whether the next step will be a graph replay (1) or
 * individual launches (0). */
mgn_status mgn_session_set_graph_replay(mgn_session* s, int enable);
/* Launch-level fusion (on by default): an RmsNorm or SwiGLUConcat dispatch whose output is
 * read only by batch-1/2 quantized matmuls is not launched; those matmuls apply it while
 * staging their activations (mgn_matmul_q_rms_norm / mgn_matmul_q_swiglu).  The plan and
 * mgn_session_dispatch_info keep the reference's dispatch list (src/compile.rs:494-528);
 * mgn_session_num_launches reports how many kernels a step really launches.  The folded
 * dispatch's own output buffer is then never written. */
mgn_status mgn_session_set_fusion(mgn_session* s, int enable);
/* Chains (on by default; with launch fusion on and graph replay off): every run of at least three
 * consecutive launches that are one-row Q4 matmuls on weights of at most 4 MiB goes out as ONE launch (mgn_chain_create /
 * mgn_chain_run in mgn_hip.h), which is how the whole step of a decode plan becomes one submission
 * as in Session::step (src/runtime.rs:2843-2959).  Results are those of the separate launches. */
mgn_status mgn_session_set_chains(mgn_session* s, int enable);
size_t mgn_session_num_launches(mgn_session* s);
int mgn_session_graph_active(const mgn_session* s);
/* Session::read_output / read_output_by_index (src/runtime.rs:2612-2638). */
mgn_status mgn_session_read_output(mgn_session* s, float* out, size_t len);
mgn_status mgn_session_read_output_by_index(mgn_session* s, size_t index, float* out, size_t len);
/* The session's context, for timing with mgn_timer_start/stop. */
mgn_ctx* mgn_session_ctx(mgn_session* s);

#ifdef __cplusplus
}
#endif
#endif /* MGN_SESSION_H */
