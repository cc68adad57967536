// Host-side mirror of meganeura's Graph / compile / Session for the quantized
// matmul path.  Paths cited are relative to the reference checkout.
#pragma once
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "mgn_internal.h"

struct ihipGraph;
struct hipGraphExec;
#include "../../include/mgn_session.h"

namespace mgn {

using NodeId = uint32_t;

// graph::DType (src/graph.rs:5-16); F16/U32 do not occur on this path.
enum class DType { F32, Q4_0, Q8_0 };

// compile::WeightFormat (src/compile.rs:8-29)
enum class WeightFormat { F32 = 0, Q4 = 1, Q8 = 2 };
inline WeightFormat weight_format_from(DType d) {
  return d == DType::Q4_0 ? WeightFormat::Q4 : d == DType::Q8_0 ? WeightFormat::Q8 : WeightFormat::F32;
}

// TensorType (src/graph.rs:29-68)
struct TensorType {
  std::vector<size_t> shape;
  DType dtype = DType::F32;
  size_t num_elements() const {
    size_t n = 1;
    for (size_t s : shape) n *= s;
    return n;
  }
  // block-level sizing for quantized types (src/graph.rs:52-68)
  size_t size_bytes() const {
    const size_t blocks = (num_elements() + 31) / 32;
    if (dtype == DType::Q4_0) return blocks * 20;
    if (dtype == DType::Q8_0) return blocks * 36;
    return num_elements() * 4;
  }
};

enum class Op {
  Input, Parameter, MatMul, Add, SwiGLU, RmsNorm, FusedMatMulAdd, SwiGLUConcat, Nop, MatMulBT, Relu, Sigmoid, Neg, Silu,
  MatMulAT, FusedMatMulATAdd, FusedMatMulBTAdd
};

struct Node {
  NodeId id;
  Op op;
  std::string name;  // Input / Parameter
  std::vector<NodeId> inputs;
  TensorType ty;
  float eps = 0.0f;  // RmsNorm
};

// graph::DerivedParam with ParamTransform::HorizontalConcat (src/graph.rs:521-545)
struct DerivedParam {
  std::string name;
  std::vector<std::pair<std::string, size_t>> sources;  // (name, cols)
  size_t rows;
};

struct GraphError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

class Graph {
 public:
  NodeId input(const std::string& name, std::vector<size_t> shape);
  NodeId parameter(const std::string& name, std::vector<size_t> shape);
  NodeId parameter_q4(const std::string& name, std::vector<size_t> shape);
  NodeId parameter_q8(const std::string& name, std::vector<size_t> shape);
  NodeId matmul(NodeId a, NodeId b);
  NodeId matmul_bt(NodeId a, NodeId b);
  NodeId matmul_at(NodeId a, NodeId b);
  NodeId add(NodeId a, NodeId b);
  NodeId swiglu(NodeId gate, NodeId up);
  NodeId rms_norm(NodeId x, NodeId weight, float eps);
  NodeId unary(mgn_unary kind, NodeId x);  // relu / sigmoid / neg / silu
  void set_outputs(std::vector<NodeId> ids);

  const Node& node(NodeId id) const;
  const std::vector<Node>& nodes() const { return nodes_; }
  std::vector<Node>& nodes_mut() { return nodes_; }
  const std::vector<NodeId>& outputs() const { return outputs_; }
  bool is_output(NodeId id) const;
  NodeId add_raw_node(Op op, std::vector<NodeId> inputs, TensorType ty, std::string name = {}, float eps = 0.0f);
  std::vector<DerivedParam> derived_params;

 private:
  std::vector<Node> nodes_;
  std::vector<NodeId> outputs_;
};

// optimize::apply_matmul_add_fusions + apply_swiglu_concat_fusions
// (src/optimize.rs:724-767, 776-879), run to a fixpoint as the reference's loop
// does (src/optimize.rs:645-665).
Graph optimize(const Graph& g);

struct Dispatch {
  mgn_shader shader;
  uint32_t workgroups[3];
  std::vector<int> input_buffers;
  int output_buffer;
  uint32_t params[4];
  WeightFormat weight_format = WeightFormat::F32;
  float eps = 0.0f;
  std::vector<mgn_unary> epilogue;  // compile::Dispatch::epilogue (src/compile.rs:466), matmuls only
};

// compile::ExecutionPlan (src/compile.rs:494-528), the fields this path uses.
struct WeightBufferInfo {
  WeightFormat fmt;
  size_t rows, cols;  // shape[0], shape[1] as declared
  bool nk = false;    // read by matmul_bt: stored [N, K], blocked along K
};
struct ExecutionPlan {
  std::vector<size_t> buffers;  // byte sizes
  std::vector<Dispatch> dispatches;
  std::vector<std::pair<std::string, int>> param_buffers;
  std::vector<std::pair<std::string, int>> input_buffers;
  std::vector<int> output_buffers;
  std::map<int, WeightBufferInfo> weight_buffers;
  struct Derived {
    int buffer;
    std::vector<std::pair<std::string, size_t>> sources;
    size_t rows;
  };
  std::vector<Derived> derived_params;
};

// compile::compile_with for the ops above (src/compile.rs:1199-1272, 1381-1421, 1486-1524).
ExecutionPlan compile(const Graph& g);

class Session {
 public:
  Session(ExecutionPlan plan, int device_id);
  ~Session();
  Session(const Session&) = delete;
  Session& operator=(const Session&) = delete;

  const ExecutionPlan& plan() const { return plan_; }
  void set_parameter(const std::string& name, const float* data, size_t len);
  void set_input(const std::string& name, const float* data, size_t len);
  void step();
  // Replay steps as one captured HIP graph (off by default): the first step after the set
  // of weight handles changed runs launch by launch, the next one is captured, later ones
  // are a single graph launch.  Results are identical; only launch overhead changes --
  // less host work per step, but measured slower on the GPU side for chains of tiny kernels.
  void set_graph_replay(bool on);
  // Fold RmsNorm / SwiGLUConcat dispatches into the decode matmuls that consume them, serve
  // sibling decode matmuls (same activations, e.g. q/k/v) with one launch and let a matmul's
  // launch apply the unary dispatches that follow it (the compiler folds those into tiled
  // matmul entries only, not into the M = 1 ones) (default on).  The plan keeps the reference's dispatch list; only the launches differ.
  void set_fusion(bool on);
  // Runs of consecutive launches that are all one-row Q4 matmuls (with whatever was folded into
  // them) go out as ONE launch each (mgn_chain_*), the dependencies between them carried by the
  // data (default on; needs launch fusion, and is left out while graph replay is wanted).
  void set_chains(bool on);
  size_t num_launches();  // kernel launches one step makes with the current settings
  bool graph_active() const { return exec_ != nullptr; }
  void wait();
  void read_output(float* out, size_t len) { read_output_by_index(0, out, len); }
  void read_output_by_index(size_t index, float* out, size_t len);
  mgn_ctx* ctx() { return ctx_; }

 private:
  void upload_weight(int buf, const WeightBufferInfo& info, const float* data);
  void check(mgn_status st, const char* what);
  void release();
  void run_dispatches();
  void drop_graph();
  void plan_launches();
  struct Fused {
    int kind = 0;          // kProNone / kProRmsNorm / kProSwiglu
    int producer = -1;     // the folded-in dispatch
    int more[2] = {-1, -1};  // sibling matmuls (same activations) served by this dispatch's launch
    std::vector<mgn_unary> post;  // unary dispatches behind an M = 1 matmul, applied by its launch
    int out_buffer = -1;          // ... whose last output buffer the launch then writes
  };
  struct ChainRun {
    size_t first, last;  // dispatch indices the chain stands in for (the skipped ones between them included)
    mgn_chain* chain;
  };
  std::vector<ChainRun> chains_;
  std::vector<int> chain_of_;    // per dispatch: index into chains_ or -1
  bool chains_wanted_ = true;
  void plan_chains();
  void drop_chains();
  std::vector<Fused> fused_;     // per dispatch (matmuls only)
  std::vector<char> skipped_;    // per dispatch: folded into its consumers
  bool launches_planned_ = false;
  bool fusion_wanted_ = true;
  ExecutionPlan plan_;
  mgn_ctx* ctx_ = nullptr;
  std::vector<mgn_buf*> buffers_;        // f32 buffers (null for quantized params)
  std::vector<mgn_weight*> weights_;     // quantized params (null otherwise)
  std::map<int, std::vector<float>> weight_staging_;  // src/runtime.rs:2373-2376
  bool graph_wanted_ = false;
  int eager_steps_ = 0;  // launch-by-launch steps since the weight handles last changed
  ihipGraph* graph_ = nullptr;    // hipGraph_t
  hipGraphExec* exec_ = nullptr;  // hipGraphExec_t
};

// build_inference_session (src/train.rs:380-389): optimize -> compile -> Session.
std::unique_ptr<Session> build_inference_session(const Graph& g, int device_id = 0);

// pointwise kernels of the session layer (kernels_util.hip)
int launch_add(ihipStream_t* s, const float* a, const float* b, float* out, size_t len);
int launch_swiglu(ihipStream_t* s, const float* gate, const float* up, float* out, size_t len);
int launch_swiglu_concat(ihipStream_t* s, const float* in, float* out, size_t len, uint32_t half_n);
int launch_rms_norm(ihipStream_t* s, const float* x, const float* weight, float* out, uint32_t rows, uint32_t cols,
                    float eps);
int launch_unary(ihipStream_t* s, int kind, const float* in, float* out, size_t len);

}  // namespace mgn
