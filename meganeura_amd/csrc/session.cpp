// Graph building, the two matmul fusions, plan compilation and the Session
// verbs for the quantized matmul path.  See session.h for what is mirrored.
#include "session.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

namespace mgn {

// ---------------------------------------------------------------- Graph ----

NodeId Graph::add_raw_node(Op op, std::vector<NodeId> inputs, TensorType ty, std::string name, float eps) {
  const NodeId id = (NodeId)nodes_.size();
  nodes_.push_back(Node{id, op, std::move(name), std::move(inputs), std::move(ty), eps});
  return id;
}

const Node& Graph::node(NodeId id) const {
  if (id >= nodes_.size()) throw GraphError("node id out of range");
  return nodes_[id];
}

bool Graph::is_output(NodeId id) const { return std::find(outputs_.begin(), outputs_.end(), id) != outputs_.end(); }

static NodeId leaf(Graph& g, Op op, const std::string& name, std::vector<size_t> shape, DType dt) {
  if (shape.empty()) throw GraphError("leaf node needs a shape");
  for (size_t s : shape)
    if (s == 0) throw GraphError("zero-sized dimension");
  return g.add_raw_node(op, {}, TensorType{std::move(shape), dt}, name);
}

NodeId Graph::input(const std::string& name, std::vector<size_t> shape) {
  return leaf(*this, Op::Input, name, std::move(shape), DType::F32);
}
NodeId Graph::parameter(const std::string& name, std::vector<size_t> shape) {
  return leaf(*this, Op::Parameter, name, std::move(shape), DType::F32);
}
// src/graph.rs:752-773: only the dtype tag differs; the shape stays logical [K, N].
NodeId Graph::parameter_q4(const std::string& name, std::vector<size_t> shape) {
  return leaf(*this, Op::Parameter, name, std::move(shape), DType::Q4_0);
}
NodeId Graph::parameter_q8(const std::string& name, std::vector<size_t> shape) {
  return leaf(*this, Op::Parameter, name, std::move(shape), DType::Q8_0);
}

// src/graph.rs:787-795
NodeId Graph::matmul(NodeId a, NodeId b) {
  const auto& as = node(a).ty.shape;
  const auto& bs = node(b).ty.shape;
  if (as.size() != 2 || bs.size() != 2) throw GraphError("matmul requires 2D tensors");
  if (as[1] != bs[0]) throw GraphError("matmul inner dimensions must match");
  return add_raw_node(Op::MatMul, {a, b}, TensorType{{as[0], bs[1]}, DType::F32});
}

// src/graph.rs:809-817
NodeId Graph::matmul_bt(NodeId a, NodeId b) {
  const auto& as = node(a).ty.shape;
  const auto& bs = node(b).ty.shape;
  if (as.size() != 2 || bs.size() != 2) throw GraphError("matmul_bt requires 2D tensors");
  if (as[1] != bs[1]) throw GraphError("MatMulBT: K dimensions must match");
  return add_raw_node(Op::MatMulBT, {a, b}, TensorType{{as[0], bs[0]}, DType::F32});
}

// src/graph.rs:798-806
NodeId Graph::matmul_at(NodeId a, NodeId b) {
  const auto& as = node(a).ty.shape;
  const auto& bs = node(b).ty.shape;
  if (as.size() != 2 || bs.size() != 2) throw GraphError("matmul_at requires 2D tensors");
  if (as[0] != bs[0]) throw GraphError("MatMulAT: K dimensions must match");
  return add_raw_node(Op::MatMulAT, {a, b}, TensorType{{as[1], bs[1]}, DType::F32});
}

// src/graph.rs:821-827
NodeId Graph::add(NodeId a, NodeId b) {
  if (node(a).ty.shape != node(b).ty.shape) throw GraphError("add requires matching shapes");
  return add_raw_node(Op::Add, {a, b}, TensorType{node(a).ty.shape, DType::F32});
}

// src/graph.rs:996-999
NodeId Graph::swiglu(NodeId gate, NodeId up) {
  if (node(gate).ty.shape != node(up).ty.shape) throw GraphError("swiglu requires matching shapes");
  return add_raw_node(Op::SwiGLU, {gate, up}, TensorType{node(gate).ty.shape, DType::F32});
}

// src/graph.rs:1029-1040
NodeId Graph::rms_norm(NodeId x, NodeId weight, float eps) {
  const auto& xs = node(x).ty.shape;
  const auto& ws = node(weight).ty.shape;
  if (xs.size() != 2) throw GraphError("rms_norm requires 2D input");
  if (ws.size() != 1) throw GraphError("rms_norm weight must be 1D");
  if (xs[1] != ws[0]) throw GraphError("rms_norm weight size must match last dim");
  return add_raw_node(Op::RmsNorm, {x, weight}, TensorType{xs, DType::F32}, {}, eps);
}

NodeId Graph::unary(mgn_unary kind, NodeId x) {
  const Op op = kind == MGN_UNARY_RELU ? Op::Relu : kind == MGN_UNARY_SIGMOID ? Op::Sigmoid : kind == MGN_UNARY_NEG ? Op::Neg
              : kind == MGN_UNARY_SILU ? Op::Silu : Op::Nop;
  if (op == Op::Nop) throw GraphError("unknown unary operation");
  if (node(x).ty.dtype != DType::F32) throw GraphError("unary operations take f32 tensors");
  return add_raw_node(op, {x}, TensorType{node(x).ty.shape, DType::F32});
}

void Graph::set_outputs(std::vector<NodeId> ids) {
  for (NodeId id : ids) (void)node(id);
  outputs_ = std::move(ids);
}

// ------------------------------------------------------------- optimize ----

static size_t use_count(const Graph& g, NodeId id) {
  size_t n = 0;
  for (const Node& nd : g.nodes())
    if (nd.op != Op::Nop && std::find(nd.inputs.begin(), nd.inputs.end(), id) != nd.inputs.end()) n++;
  return n;
}

// src/optimize.rs:724-767: Add(MatMul(a,b), d) -> FusedMatMulAdd(a,b,d) when the
// matmul feeds only this Add and is not itself a graph output; the same for the AT and BT forms.
static bool apply_matmul_add_fusions(Graph& g) {
  bool changed = false;
  const size_t count = g.nodes().size();
  auto plain_matmul = [](Op op) { return op == Op::MatMul || op == Op::MatMulAT || op == Op::MatMulBT; };
  for (size_t id = 0; id < count; id++) {
    const Node& nd = g.nodes()[id];
    if (nd.op != Op::Add) continue;
    const NodeId lhs = nd.inputs[0], rhs = nd.inputs[1];
    NodeId mm, addend;
    if (plain_matmul(g.node(lhs).op)) {
      mm = lhs;
      addend = rhs;
    } else if (plain_matmul(g.node(rhs).op)) {
      mm = rhs;
      addend = lhs;
    } else {
      continue;
    }
    if (use_count(g, mm) != 1 || g.is_output(mm)) continue;
    const NodeId a = g.node(mm).inputs[0], b = g.node(mm).inputs[1];
    const Op mm_op = g.node(mm).op;
    g.nodes_mut()[id].op = mm_op == Op::MatMul ? Op::FusedMatMulAdd : mm_op == Op::MatMulAT ? Op::FusedMatMulATAdd : Op::FusedMatMulBTAdd;
    g.nodes_mut()[id].inputs = {a, b, addend};
    g.nodes_mut()[mm].op = Op::Nop;
    changed = true;
  }
  return changed;
}

// src/optimize.rs:776-879: SwiGLU(MatMul(h,Wg), MatMul(h,Wu)) -> SwiGLUConcat(MatMul(h, [Wg|Wu])).
// The concatenated parameter is named "<gate>+<up>", keeps the sources' dtype
// (848-854) and is recorded as a derived parameter so that set_parameter on
// either source refills it (842-847).
static bool apply_swiglu_concat_fusions(Graph& g) {
  bool changed = false;
  const size_t count = g.nodes().size();
  for (size_t id = 0; id < count; id++) {
    if (g.nodes()[id].op != Op::SwiGLU) continue;
    const NodeId gate_id = g.nodes()[id].inputs[0], up_id = g.nodes()[id].inputs[1];
    const Node gate = g.node(gate_id), up = g.node(up_id);
    if (gate.op != Op::MatMul || up.op != Op::MatMul) continue;
    if (gate.inputs[0] != up.inputs[0]) continue;
    if (use_count(g, gate_id) != 1 || use_count(g, up_id) != 1) continue;
    if (g.is_output(gate_id) || g.is_output(up_id)) continue;
    const NodeId h = gate.inputs[0], w_gate = gate.inputs[1], w_up = up.inputs[1];
    const Node wg = g.node(w_gate), wu = g.node(w_up);
    if (wg.ty.shape.size() != 2 || wu.ty.shape.size() != 2) continue;
    if (wg.ty.shape != wu.ty.shape) continue;
    if (wg.op != Op::Parameter || wu.op != Op::Parameter) continue;
    // The reference keeps the gate's dtype even if the up projection's differs;
    // a mixed pair would then be quantized in a format its owner did not ask
    // for, so here a mixed pair is simply left unfused.
    if (wg.ty.dtype != wu.ty.dtype) continue;
    const size_t in_f = wg.ty.shape[0], out_f = wg.ty.shape[1];
    const std::string name = wg.name + "+" + wu.name;
    g.derived_params.push_back(DerivedParam{name, {{wg.name, out_f}, {wu.name, out_f}}, in_f});
    const NodeId concat_w =
        g.add_raw_node(Op::Parameter, {}, TensorType{{in_f, 2 * out_f}, wg.ty.dtype}, name);
    const size_t m = g.node(h).ty.shape[0];
    const NodeId wide = g.add_raw_node(Op::MatMul, {h, concat_w}, TensorType{{m, 2 * out_f}, DType::F32});
    Node& sw = g.nodes_mut()[id];
    sw.op = Op::SwiGLUConcat;
    sw.inputs = {wide};
    sw.ty = TensorType{{m, out_f}, DType::F32};
    g.nodes_mut()[gate_id].op = Op::Nop;
    g.nodes_mut()[up_id].op = Op::Nop;
    changed = true;
  }
  return changed;
}

Graph optimize(const Graph& src) {
  Graph g = src;
  for (int iter = 0; iter < 8; iter++) {
    bool changed = apply_matmul_add_fusions(g);
    changed |= apply_swiglu_concat_fusions(g);
    if (!changed) break;
  }
  return g;
}

// -------------------------------------------------------------- compile ----

static std::vector<NodeId> toposort(const Graph& g) {
  // fusion appends nodes (the wide matmul) after their consumer, so order by dependencies
  const size_t n = g.nodes().size();
  std::vector<int> state(n, 0);
  std::vector<NodeId> order;
  order.reserve(n);
  std::vector<std::pair<NodeId, size_t>> stack;
  for (NodeId root = 0; root < n; root++) {
    if (state[root]) continue;
    stack.push_back({root, 0});
    state[root] = 1;
    while (!stack.empty()) {
      auto& [id, next] = stack.back();
      const Node& nd = g.nodes()[id];
      if (next < nd.inputs.size()) {
        const NodeId in = nd.inputs[next++];
        if (state[in] == 0) {
          state[in] = 1;
          stack.push_back({in, 0});
        } else if (state[in] == 1) {
          throw GraphError("cycle in graph");
        }
      } else {
        state[id] = 2;
        order.push_back(id);
        stack.pop_back();
      }
    }
  }
  return order;
}

static mgn_unary unary_of(mgn_shader s) {
  return s == MGN_SHADER_RELU ? MGN_UNARY_RELU : s == MGN_SHADER_SIGMOID ? MGN_UNARY_SIGMOID
         : s == MGN_SHADER_NEG ? MGN_UNARY_NEG : s == MGN_SHADER_SILU ? MGN_UNARY_SILU : MGN_UNARY_NONE;
}

// fuse_epilogues (src/compile.rs:915-1035): a Relu / Sigmoid / Neg / Silu dispatch whose input
// is written by a tiled matmul entry and read by nothing else is removed; the matmul takes its
// output buffer and applies the operation to every element it stores.  Chains fold one by one.
// The M = 1 entries (MatMulGemv*) are not candidates in the reference and are none here.
// Differences: the reference builds the resulting pipeline with the f32 weight format whatever
// the weight is (src/codegen.rs:617-642) -- here the quantized kernels apply the epilogue; and
// it does not look at graph outputs, so a matmul result that is itself an output would never
// be written -- here such a matmul keeps its buffer and the unary stays a dispatch.
static void fuse_epilogues(ExecutionPlan& plan) {
  auto& ds = plan.dispatches;
  std::map<int, size_t> producer;
  for (size_t i = 0; i < ds.size(); i++) producer[ds[i].output_buffer] = i;
  std::map<int, size_t> read_count;
  for (const Dispatch& d : ds)
    for (int b : d.input_buffers) read_count[b]++;
  std::vector<size_t> to_remove;
  for (size_t i = 0; i < ds.size(); i++) {
    const mgn_unary op = unary_of(ds[i].shader);
    if (op == MGN_UNARY_NONE || ds[i].input_buffers.size() != 1) continue;
    const int primary = ds[i].input_buffers[0];
    auto pit = producer.find(primary);
    if (pit == producer.end()) continue;
    Dispatch& prod = ds[pit->second];
    const bool tiled = prod.shader == MGN_SHADER_MATMUL || prod.shader == MGN_SHADER_FUSED_MATMUL_ADD ||
                       prod.shader == MGN_SHADER_MATMUL_BT || prod.shader == MGN_SHADER_MATMUL_AT ||
                       prod.shader == MGN_SHADER_FUSED_MATMUL_AT_ADD || prod.shader == MGN_SHADER_FUSED_MATMUL_BT_ADD;
    if (!tiled || read_count[primary] != 1 || prod.epilogue.size() >= 8) continue;
    if (std::find(plan.output_buffers.begin(), plan.output_buffers.end(), primary) != plan.output_buffers.end()) continue;
    prod.epilogue.push_back(op);
    prod.output_buffer = ds[i].output_buffer;
    producer[ds[i].output_buffer] = pit->second;
    to_remove.push_back(i);
  }
  for (auto it = to_remove.rbegin(); it != to_remove.rend(); ++it) ds.erase(ds.begin() + (std::ptrdiff_t)*it);
}

ExecutionPlan compile(const Graph& g) {
  ExecutionPlan plan;
  std::map<NodeId, int> node_buf;
  // pass 1 (src/compile.rs:1201-1262): a buffer per live node; quantized parameters are
  // registered with (format, rows = shape[0], cols = shape[1]) (1229-1241)
  for (const Node& nd : g.nodes()) {
    if (nd.op == Op::Nop) continue;
    const int buf = (int)plan.buffers.size();
    plan.buffers.push_back(std::max<size_t>(nd.ty.size_bytes(), 4));
    node_buf[nd.id] = buf;
    if (nd.op == Op::Parameter) {
      plan.param_buffers.push_back({nd.name, buf});
      const WeightFormat wf = weight_format_from(nd.ty.dtype);
      if (wf != WeightFormat::F32) {
        const auto& sh = nd.ty.shape;
        plan.weight_buffers[buf] = WeightBufferInfo{wf, sh[0], sh.size() >= 2 ? sh[1] : 1};
      }
    } else if (nd.op == Op::Input) {
      plan.input_buffers.push_back({nd.name, buf});
    }
  }
  // a quantized parameter read by matmul_bt is blocked along its second dimension
  for (const Node& nd : g.nodes()) {
    if (nd.op != Op::MatMulBT && nd.op != Op::FusedMatMulBTAdd) continue;
    auto it = node_buf.find(nd.inputs[1]);
    if (it == node_buf.end()) continue;
    auto wb = plan.weight_buffers.find(it->second);
    if (wb == plan.weight_buffers.end()) continue;
    wb->second.nk = true;
  }
  for (const Node& nd : g.nodes()) {
    if (nd.op != Op::MatMul && nd.op != Op::FusedMatMulAdd && nd.op != Op::MatMulAT && nd.op != Op::FusedMatMulATAdd) continue;
    auto it = node_buf.find(nd.inputs[1]);
    if (it == node_buf.end()) continue;
    auto wb = plan.weight_buffers.find(it->second);
    if (wb != plan.weight_buffers.end() && wb->second.nk)
      throw GraphError("a quantized parameter cannot feed both matmul and matmul_bt: its blocks run along one dimension only");
  }
  for (const DerivedParam& dp : g.derived_params) {
    for (const auto& pb : plan.param_buffers)
      if (pb.first == dp.name) plan.derived_params.push_back({pb.second, dp.sources, dp.rows});
  }
  auto buf_of = [&](NodeId id) {
    auto it = node_buf.find(id);
    if (it == node_buf.end()) throw GraphError("node consumed after being fused away");
    return it->second;
  };
  // pass 2: one dispatch per compute node
  for (NodeId id : toposort(g)) {
    const Node& nd = g.nodes()[id];
    Dispatch d{};
    d.output_buffer = nd.op == Op::Nop ? -1 : buf_of(id);
    switch (nd.op) {
      case Op::Input:
      case Op::Parameter:
      case Op::Nop:
        continue;
      case Op::MatMul:
      case Op::FusedMatMulAdd: {
        // src/compile.rs:1381-1421, 1486-1524: M == 1 and N % 4 == 0 take the GEMV entry
        // with grid [N/4,1,1]; everything else the 64x64 tiled entry
        const auto& as = g.node(nd.inputs[0]).ty.shape;
        const Node& bn = g.node(nd.inputs[1]);
        const uint32_t m = (uint32_t)as[0], k = (uint32_t)as[1], n = (uint32_t)bn.ty.shape[1];
        const bool fused = nd.op == Op::FusedMatMulAdd;
        if (m == 1 && n % 4 == 0) {
          d.shader = fused ? MGN_SHADER_MATMUL_GEMV_ADD : MGN_SHADER_MATMUL_GEMV;
          d.workgroups[0] = n / 4, d.workgroups[1] = 1, d.workgroups[2] = 1;
        } else {
          d.shader = fused ? MGN_SHADER_FUSED_MATMUL_ADD : MGN_SHADER_MATMUL;
          d.workgroups[0] = (n + 63) / 64, d.workgroups[1] = (m + 63) / 64, d.workgroups[2] = 1;
        }
        d.input_buffers = {buf_of(nd.inputs[0]), buf_of(nd.inputs[1])};
        if (fused) d.input_buffers.push_back(buf_of(nd.inputs[2]));
        d.params[0] = m, d.params[1] = k, d.params[2] = n, d.params[3] = 0;
        d.weight_format = weight_format_from(bn.ty.dtype);
        break;
      }
      case Op::MatMulAT:
      case Op::FusedMatMulATAdd: {
        // src/compile.rs:1423-1445, 1526-1549: A is [K, M]; always the 64x64 tiled entry;
        // parameter order [m, n, k, 0]
        const auto& as = g.node(nd.inputs[0]).ty.shape;
        const Node& bn = g.node(nd.inputs[1]);
        const uint32_t k = (uint32_t)as[0], m = (uint32_t)as[1], n = (uint32_t)bn.ty.shape[1];
        const bool fused = nd.op == Op::FusedMatMulATAdd;
        d.shader = fused ? MGN_SHADER_FUSED_MATMUL_AT_ADD : MGN_SHADER_MATMUL_AT;
        d.workgroups[0] = (n + 63) / 64, d.workgroups[1] = (m + 63) / 64, d.workgroups[2] = 1;
        d.input_buffers = {buf_of(nd.inputs[0]), buf_of(nd.inputs[1])};
        if (fused) d.input_buffers.push_back(buf_of(nd.inputs[2]));
        d.params[0] = m, d.params[1] = n, d.params[2] = k, d.params[3] = 0;
        d.weight_format = weight_format_from(bn.ty.dtype);
        break;
      }
      case Op::FusedMatMulBTAdd: {
        // src/compile.rs:1551-1574: always the tiled entry, [m, n, k, 0]
        const auto& as = g.node(nd.inputs[0]).ty.shape;
        const Node& bn = g.node(nd.inputs[1]);
        const uint32_t m = (uint32_t)as[0], k = (uint32_t)as[1], n = (uint32_t)bn.ty.shape[0];
        d.shader = MGN_SHADER_FUSED_MATMUL_BT_ADD;
        d.workgroups[0] = (n + 63) / 64, d.workgroups[1] = (m + 63) / 64, d.workgroups[2] = 1;
        d.input_buffers = {buf_of(nd.inputs[0]), buf_of(nd.inputs[1]), buf_of(nd.inputs[2])};
        d.params[0] = m, d.params[1] = n, d.params[2] = k, d.params[3] = 0;
        d.weight_format = weight_format_from(bn.ty.dtype);
        break;
      }
      case Op::MatMulBT: {
        // src/compile.rs:1447-1485: M == 1 and K % 4 == 0 take the GEMV-BT entry with grid
        // [N,1,1]; everything else the 64x64 tiled one.  Parameter order [m, n, k, 0].
        const auto& as = g.node(nd.inputs[0]).ty.shape;
        const Node& bn = g.node(nd.inputs[1]);
        const uint32_t m = (uint32_t)as[0], k = (uint32_t)as[1], n = (uint32_t)bn.ty.shape[0];
        if (m == 1 && k % 4 == 0) {
          d.shader = MGN_SHADER_MATMUL_GEMV_BT;
          d.workgroups[0] = n, d.workgroups[1] = 1, d.workgroups[2] = 1;
        } else {
          d.shader = MGN_SHADER_MATMUL_BT;
          d.workgroups[0] = (n + 63) / 64, d.workgroups[1] = (m + 63) / 64, d.workgroups[2] = 1;
        }
        d.input_buffers = {buf_of(nd.inputs[0]), buf_of(nd.inputs[1])};
        d.params[0] = m, d.params[1] = n, d.params[2] = k, d.params[3] = 0;
        d.weight_format = weight_format_from(bn.ty.dtype);
        break;
      }
      case Op::Add:
      case Op::SwiGLU: {
        const uint32_t len = (uint32_t)nd.ty.num_elements();
        d.shader = nd.op == Op::Add ? MGN_SHADER_ADD : MGN_SHADER_SWIGLU;
        d.workgroups[0] = (len + 255) / 256, d.workgroups[1] = 1, d.workgroups[2] = 1;
        d.input_buffers = {buf_of(nd.inputs[0]), buf_of(nd.inputs[1])};
        d.params[0] = len;
        break;
      }
      case Op::SwiGLUConcat: {
        // src/compile.rs:1814-1830
        const uint32_t len = (uint32_t)nd.ty.num_elements();
        d.shader = MGN_SHADER_SWIGLU_CONCAT;
        d.workgroups[0] = (len + 255) / 256, d.workgroups[1] = 1, d.workgroups[2] = 1;
        d.input_buffers = {buf_of(nd.inputs[0])};
        d.params[0] = len, d.params[1] = (uint32_t)nd.ty.shape[1];
        break;
      }
      case Op::Relu:
      case Op::Sigmoid:
      case Op::Neg:
      case Op::Silu: {
        // emit_unary (src/compile.rs:3433-3453): grid [ceil(len / 256), 1, 1], params [len, 0, 0, 0]
        const uint32_t len = (uint32_t)nd.ty.num_elements();
        d.shader = nd.op == Op::Relu ? MGN_SHADER_RELU : nd.op == Op::Sigmoid ? MGN_SHADER_SIGMOID
                   : nd.op == Op::Neg ? MGN_SHADER_NEG : MGN_SHADER_SILU;
        d.workgroups[0] = (len + 255) / 256, d.workgroups[1] = 1, d.workgroups[2] = 1;
        d.input_buffers = {buf_of(nd.inputs[0])};
        d.params[0] = len;
        break;
      }
      case Op::RmsNorm: {
        // src/compile.rs:1851-1872 (the hand-written entry: one workgroup per row)
        const auto& xs = g.node(nd.inputs[0]).ty.shape;
        d.shader = MGN_SHADER_RMS_NORM;
        d.workgroups[0] = (uint32_t)xs[0], d.workgroups[1] = 1, d.workgroups[2] = 1;
        d.input_buffers = {buf_of(nd.inputs[0]), buf_of(nd.inputs[1])};
        d.params[0] = (uint32_t)xs[0], d.params[1] = (uint32_t)xs[1];
        std::memcpy(&d.params[2], &nd.eps, 4);
        d.eps = nd.eps;
        break;
      }
    }
    plan.dispatches.push_back(std::move(d));
  }
  for (NodeId out : g.outputs()) plan.output_buffers.push_back(buf_of(out));
  fuse_epilogues(plan);
  return plan;
}

// -------------------------------------------------------------- Session ----

void Session::check(mgn_status st, const char* what) {
  if (st != MGN_OK) throw std::runtime_error(std::string(what) + ": " + mgn_last_error(ctx_));
}

static bool is_bt(mgn_shader s) {
  return s == MGN_SHADER_MATMUL_BT || s == MGN_SHADER_MATMUL_GEMV_BT || s == MGN_SHADER_FUSED_MATMUL_BT_ADD;
}
// the forms whose activations arrive transposed ([K, M])
static bool is_at(mgn_shader s) { return s == MGN_SHADER_MATMUL_AT || s == MGN_SHADER_FUSED_MATMUL_AT_ADD; }
static bool is_matmul(mgn_shader s) { return s <= MGN_SHADER_MATMUL_GEMV_ADD || is_bt(s) || is_at(s); }
// K of a matmul dispatch: params are [m, k, n, 0], or [m, n, k, 0] for the AT and BT forms
static uint32_t matmul_k(const Dispatch& d) { return is_bt(d.shader) || is_at(d.shader) ? d.params[2] : d.params[1]; }

Session::Session(ExecutionPlan plan, int device_id) : plan_(std::move(plan)) {
  // This backend serves matmuls whose weight is quantized; a plain f32 weight
  // stays with the host runtime's own dispatch.
  for (const Dispatch& d : plan_.dispatches)
    if (is_matmul(d.shader) && d.weight_format == WeightFormat::F32)
      throw std::runtime_error("matmul with an f32 weight is not on the quantized path of this backend");
  mgn_status st = mgn_ctx_create(device_id, &ctx_);
  if (st != MGN_OK) throw std::runtime_error(std::string("mgn_ctx_create: ") + mgn_last_error(nullptr));
  buffers_.assign(plan_.buffers.size(), nullptr);
  weights_.assign(plan_.buffers.size(), nullptr);
  try {
    // every plan buffer exists and is zero-filled up front (src/runtime.rs:1737-1755);
    // a quantized parameter gets its device storage when it is first set
    for (size_t i = 0; i < plan_.buffers.size(); i++)
      if (!plan_.weight_buffers.count((int)i)) check(mgn_buf_alloc(ctx_, plan_.buffers[i], &buffers_[i]), "mgn_buf_alloc");
    // the A^T matmul forms transpose their activations into a staging area of the context: sized
    // here for the whole plan, so that no step allocates (a step may run under stream capture)
    size_t at_bytes = 0;
    for (const Dispatch& d : plan_.dispatches)
      if (is_at(d.shader)) at_bytes = std::max(at_bytes, (size_t)d.params[0] * matmul_k(d) * sizeof(float));
    if (at_bytes) check(mgn::reserve_at_stage(ctx_, at_bytes), "A^T staging area");
  } catch (...) {
    release();
    throw;
  }
}

Session::~Session() { release(); }

void Session::release() {
  if (!ctx_) return;
  (void)mgn_sync(ctx_);  // Drop waits for the GPU first (src/runtime.rs:4339-4345)
  drop_graph();
  drop_chains();
  for (mgn_buf* b : buffers_) mgn_buf_free(ctx_, b);
  for (mgn_weight* w : weights_) mgn_weight_free(ctx_, w);
  buffers_.clear();
  weights_.clear();
  mgn_ctx_destroy(ctx_);
  ctx_ = nullptr;
}

void Session::upload_weight(int buf, const WeightBufferInfo& info, const float* data) {
  mgn_weight* fresh = nullptr;
  const mgn_fmt fmt = info.fmt == WeightFormat::Q4 ? MGN_FMT_Q4 : MGN_FMT_Q8;
  if (info.nk) check(mgn_weight_create_nk(ctx_, fmt, data, info.rows, info.cols, &fresh), "mgn_weight_create_nk");
  else check(mgn_weight_create(ctx_, fmt, data, info.rows, info.cols, &fresh), "mgn_weight_create");
  drop_graph();  // a captured step holds the old handle's addresses
  drop_chains();  // ... and so does a chain
  launches_planned_ = false;
  mgn_weight_free(ctx_, weights_[buf]);  // waits for in-flight work that may still read it
  weights_[buf] = fresh;
}

// src/runtime.rs:2327-2493
void Session::set_parameter(const std::string& name, const float* data, size_t len) {
  for (const auto& pb : plan_.param_buffers) {
    if (pb.first != name) continue;
    const int buf = pb.second;
    auto wb = plan_.weight_buffers.find(buf);
    if (wb != plan_.weight_buffers.end()) {
      if (len != wb->second.rows * wb->second.cols) throw std::invalid_argument("parameter '" + name + "': length is not rows*cols");
      upload_weight(buf, wb->second, data);
    } else {
      if (len * 4 > plan_.buffers[buf]) throw std::invalid_argument("parameter '" + name + "': data exceeds buffer");
      check(mgn_buf_upload(ctx_, buffers_[buf], 0, data, len * 4), "mgn_buf_upload");
    }
    // derived (horizontally concatenated) parameters fed by this source (2349-2432)
    for (const auto& dp : plan_.derived_params) {
      bool feeds = false;
      size_t total_cols = 0;
      for (const auto& s : dp.sources) {
        feeds |= s.first == name;
        total_cols += s.second;
      }
      if (!feeds) continue;
      auto dwb = plan_.weight_buffers.find(dp.buffer);
      const size_t rows = dp.rows;
      // f32 staging copy of the whole concatenated matrix, kept across calls (2373-2391)
      std::vector<float>& staging = weight_staging_[dp.buffer];
      if (staging.empty()) staging.assign(rows * total_cols, 0.0f);
      size_t col_off = 0;
      for (const auto& s : dp.sources) {
        if (s.first == name) {
          if (len != rows * s.second) throw std::invalid_argument("parameter '" + name + "': length does not match derived source");
          for (size_t r = 0; r < rows; r++)
            std::memcpy(&staging[r * total_cols + col_off], data + r * s.second, s.second * sizeof(float));
        }
        col_off += s.second;
      }
      if (dwb != plan_.weight_buffers.end())
        upload_weight(dp.buffer, dwb->second, staging.data());  // re-quantize the whole matrix (2392-2406)
      else
        check(mgn_buf_upload(ctx_, buffers_[dp.buffer], 0, staging.data(), staging.size() * 4), "mgn_buf_upload");
    }
    return;
  }
  throw std::out_of_range("unknown parameter: " + name);
}

// src/runtime.rs:2496-2504
void Session::set_input(const std::string& name, const float* data, size_t len) {
  for (const auto& ib : plan_.input_buffers) {
    if (ib.first != name) continue;
    if (len * 4 > plan_.buffers[ib.second]) throw std::invalid_argument("input '" + name + "': data exceeds buffer");
    check(mgn_buf_upload(ctx_, buffers_[ib.second], 0, data, len * 4), "mgn_buf_upload");
    return;
  }
  throw std::out_of_range("unknown input: " + name);
}

// src/runtime.rs:2843-2959: replay the dispatch list on the stream; returns after
// submission.  Stream order stands in for the barriers between dependency groups.
// src/runtime.rs:2843-2959 submits the whole plan as one command buffer; the equivalent here
// is one captured graph.  Kernel nodes only: nothing on this path records a memset.
void Session::step() {
  plan_launches();  // (may free chains and synchronise: never inside a stream capture)
  if (exec_) {
    hipError_t e = hipGraphLaunch(exec_, ctx_->stream);
    if (e != hipSuccess) throw std::runtime_error(std::string("hipGraphLaunch: ") + hipGetErrorString(e));
    return;
  }
  if (!graph_wanted_ || eager_steps_ == 0) {
    // the first step also lets every kernel variant do its one-time attribute setup
    run_dispatches();
    eager_steps_++;
    return;
  }
  hipError_t e = hipStreamBeginCapture(ctx_->stream, hipStreamCaptureModeThreadLocal);
  if (e != hipSuccess) {
    graph_wanted_ = false;
    run_dispatches();
    return;
  }
  std::exception_ptr failure;
  try {
    run_dispatches();
  } catch (...) {
    failure = std::current_exception();
  }
  e = hipStreamEndCapture(ctx_->stream, &graph_);
  if (failure) {
    drop_graph();
    graph_wanted_ = false;
    std::rethrow_exception(failure);
  }
  if (e == hipSuccess) e = hipGraphInstantiate(&exec_, graph_, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    // capture is an optimisation: fall back to plain launches for good
    (void)hipGetLastError();
    drop_graph();
    graph_wanted_ = false;
    run_dispatches();
    return;
  }
  e = hipGraphLaunch(exec_, ctx_->stream);
  if (e != hipSuccess) throw std::runtime_error(std::string("hipGraphLaunch: ") + hipGetErrorString(e));
}

void Session::set_graph_replay(bool on) {
  if (on != graph_wanted_) launches_planned_ = false;  // chains are left out of a replayed graph
  graph_wanted_ = on;
  if (!on) drop_graph();
}

void Session::drop_graph() {
  if (exec_ || graph_) (void)mgn_sync(ctx_);
  if (exec_) (void)hipGraphExecDestroy(exec_);
  if (graph_) (void)hipGraphDestroy(graph_);
  exec_ = nullptr;
  graph_ = nullptr;
  eager_steps_ = 0;
}

void Session::set_fusion(bool on) {
  if (on == fusion_wanted_) return;
  fusion_wanted_ = on;
  launches_planned_ = false;
  drop_graph();
}

void Session::set_chains(bool on) {
  if (on == chains_wanted_) return;
  chains_wanted_ = on;
  launches_planned_ = false;
  drop_graph();
}

void Session::drop_chains() {
  for (ChainRun& c : chains_) mgn_chain_free(ctx_, c.chain);
  chains_.clear();
  chain_of_.clear();
}

size_t Session::num_launches() {
  plan_launches();
  size_t n = 0;
  for (size_t i = 0; i < skipped_.size(); i++) {
    if (skipped_[i]) continue;
    const int c = chain_of_.empty() ? -1 : chain_of_[i];
    n += c < 0 || chains_[c].first == i ? 1 : 0;  // a chain is one launch
  }
  return n;
}

// One launch for every run of at least three consecutive launches that the chain kernel serves (M = 1,
// Q4, no transposed activations) and that are launch-bound: every weight at most 4 MiB packed
// (src/runtime.rs:2843-2959 encodes the whole step once; here the runs between other kinds of
// dispatches are what can go out together).  Where it pays was measured: a hand-over inside a chain
// costs about 3.3 us against 3.7-4 us for a dependent launch, so two stages in a chain take what
// two launches take (576 -> 3072 -> 576: 7.3 us either way; 1024 -> 6144 -> 1024: 8.4 against 7.6),
// the gain comes from stages that run side by side and from the one launch they all share (eight
// SmolLM2 decode layers: 9.8 against 15.8 us per layer), and a chain's looped stage streams a large
// weight more slowly than the kernels written out for it (4096 -> 28672 -> 4096: 28.7 against 25.5 us).
void Session::plan_chains() {
  drop_chains();
  const size_t nd = plan_.dispatches.size();
  chain_of_.assign(nd, -1);
  if (!chains_wanted_ || !fusion_wanted_ || graph_wanted_) return;
  auto chainable = [&](size_t i) {
    const Dispatch& d = plan_.dispatches[i];
    if (!is_matmul(d.shader) || is_at(d.shader) || d.params[0] != 1) return false;
    mgn_weight* w = weights_[d.input_buffers[1]];
    return w && w->fmt == MGN_FMT_Q4 && w->meta_bytes + w->quant_bytes <= ((size_t)4 << 20);
  };
  for (size_t i = 0; i < nd;) {
    if (skipped_[i] || !chainable(i)) {
      i++;
      continue;
    }
    // the run: launches i .. j-1 (skipped dispatches between them belong to some launch of the run or to none that matters)
    size_t j = i, launches = 0, last = i;
    while (j < nd && (skipped_[j] || chainable(j))) {
      if (!skipped_[j]) launches++, last = j;
      j++;
    }
    if (launches >= 3) {
      std::vector<mgn_chain_stage> stages;
      std::vector<std::vector<mgn_unary>> ops;  // kept alive until the chain is made
      ops.reserve(2 * (last - i + 1));
      for (size_t di = i; di <= last; di++) {
        if (skipped_[di]) continue;
        const Dispatch& d = plan_.dispatches[di];
        const Fused& f = fused_[di];
        const Dispatch* p = f.kind != kProNone ? &plan_.dispatches[f.producer] : nullptr;
        auto add = [&](const Dispatch& md, const Fused* mf) {
          mgn_chain_stage st{};
          st.w = weights_[md.input_buffers[1]];
          st.a = p ? buffers_[p->input_buffers[0]] : buffers_[md.input_buffers[0]];
          st.prologue = (mgn_prologue)f.kind;
          st.norm_weight = f.kind == kProRmsNorm ? buffers_[p->input_buffers[1]] : nullptr;
          st.eps = p ? p->eps : 0.0f;
          st.d = md.input_buffers.size() > 2 ? buffers_[md.input_buffers[2]] : nullptr;
          ops.emplace_back(md.epilogue);
          if (mf) ops.back().insert(ops.back().end(), mf->post.begin(), mf->post.end());
          st.ops = ops.back().empty() ? nullptr : ops.back().data();
          st.n_ops = ops.back().size();
          st.c = buffers_[mf && mf->out_buffer >= 0 ? mf->out_buffer : md.output_buffer];
          stages.push_back(st);
        };
        add(d, &f);
        for (int sib : f.more)
          if (sib >= 0) add(plan_.dispatches[sib], nullptr);
      }
      mgn_chain* ch = nullptr;
      const mgn_status st = mgn_chain_create(ctx_, stages.data(), stages.size(), 1, &ch);
      if (st == MGN_OK) {
        for (size_t di = i; di <= last; di++) chain_of_[di] = (int)chains_.size();
        chains_.push_back(ChainRun{i, last, ch});
      } else if (st != MGN_EUNSUPPORTED) {
        check(st, "mgn_chain_create");
      }
    }
    i = j;
  }
}

// Which RmsNorm / SwiGLUConcat dispatches disappear into the matmuls that read them
// (models/smollm2.rs:340-341,396: norm -> q/k/v and norm -> gate/up; compile.rs:1814-1830:
// swiglu_concat -> down).  A producer is folded only if every reader of its output is a
// decode matmul taking it as the activation operand and served by the fusing kernel.
void Session::plan_launches() {
  if (launches_planned_) return;
  const size_t nd = plan_.dispatches.size();
  fused_.assign(nd, Fused{});
  skipped_.assign(nd, 0);
  launches_planned_ = true;
  drop_chains();
  chain_of_.assign(nd, -1);
  if (!fusion_wanted_) return;
  std::vector<std::vector<int>> readers(plan_.buffers.size());
  for (size_t i = 0; i < nd; i++)
    for (int b : plan_.dispatches[i].input_buffers) readers[b].push_back((int)i);
  std::vector<char> is_output(plan_.buffers.size(), 0);
  for (int b : plan_.output_buffers) is_output[b] = 1;
  for (size_t pi = 0; pi < nd; pi++) {
    const Dispatch& p = plan_.dispatches[pi];
    const bool norm = p.shader == MGN_SHADER_RMS_NORM, swi = p.shader == MGN_SHADER_SWIGLU_CONCAT;
    if (!norm && !swi) continue;
    const int out = p.output_buffer;
    if (is_output[out] || readers[out].empty()) continue;
    const uint32_t width = p.params[1];  // columns of the produced activation
    bool ok = true;
    for (int ci : readers[out]) {
      const Dispatch& c = plan_.dispatches[ci];
      mgn_weight* w = is_matmul(c.shader) ? weights_[c.input_buffers[1]] : nullptr;
      ok = ok && (size_t)ci > pi && w && c.input_buffers[0] == out && is_matmul(c.shader) && !is_at(c.shader) && matmul_k(c) == width &&
           (c.input_buffers.size() < 3 || c.input_buffers[2] != out) && fused_[ci].kind == 0 && c.epilogue.empty() &&
           mgn_matmul_q_can_fuse(ctx_, w, c.params[0]) == 1;
    }
    if (!ok) continue;
    skipped_[pi] = 1;
    for (int ci : readers[out]) {
      fused_[ci].kind = norm ? kProRmsNorm : kProSwiglu;
      fused_[ci].producer = (int)pi;
    }
  }
  // Sibling decode matmuls: same activations (and prologue), same K and format.  The later
  // ones move up to the first one's launch, which is legal when whatever else they read (the
  // residual) already exists at that point.
  std::vector<int> producer_of(plan_.buffers.size(), -1);
  for (size_t i = 0; i < nd; i++) producer_of[plan_.dispatches[i].output_buffer] = (int)i;
  auto batchable = [&](size_t i) {
    const Dispatch& d = plan_.dispatches[i];
    if (skipped_[i] || !is_matmul(d.shader) || is_at(d.shader) || !d.epilogue.empty()) return false;
    mgn_weight* w = weights_[d.input_buffers[1]];
    return w && mgn_matmul_q_can_fuse(ctx_, w, d.params[0]) == 1;
  };
  for (size_t i = 0; i < nd; i++) {
    if (!batchable(i)) continue;
    const Dispatch& di = plan_.dispatches[i];
    int found = 0;
    for (size_t j = i + 1; j < nd && found < 2; j++) {
      if (!batchable(j)) continue;
      const Dispatch& dj = plan_.dispatches[j];
      const bool same_src = dj.input_buffers[0] == di.input_buffers[0] && fused_[j].kind == fused_[i].kind &&
                            fused_[j].producer == fused_[i].producer;
      const bool same_shape = dj.params[0] == di.params[0] && matmul_k(dj) == matmul_k(di) &&
                              dj.weight_format == di.weight_format;
      const bool addend_ready = dj.input_buffers.size() < 3 || producer_of[dj.input_buffers[2]] < (int)i;
      if (!same_src || !same_shape || !addend_ready) continue;
      // the launch is planned for the columns of the whole batch: a sibling joins only if the
      // batch with it still has a plan (each weight planning alone does not settle that)
      const mgn_weight* group[3] = {weights_[di.input_buffers[1]], nullptr, nullptr};
      for (int f = 0; f < found; f++) group[1 + f] = weights_[plan_.dispatches[fused_[i].more[f]].input_buffers[1]];
      group[1 + found] = weights_[dj.input_buffers[1]];
      if (!batch_plans(ctx_, group, (size_t)found + 2, di.params[0], fused_[i].kind)) continue;
      fused_[i].more[found++] = (int)j;
      skipped_[j] = 1;
    }
  }
  // Unary dispatches behind a matmul that the compiler left alone (M = 1 entries): the matmul's
  // launch applies them when nothing else reads the intermediate result.
  for (size_t ui = 0; ui < nd; ui++) {
    const Dispatch& u = plan_.dispatches[ui];
    const mgn_unary op = unary_of(u.shader);
    if (op == MGN_UNARY_NONE || skipped_[ui]) continue;
    const int in = u.input_buffers[0];
    const int pi = producer_of[in];
    if (pi < 0 || (size_t)pi >= ui || skipped_[pi] || !is_matmul(plan_.dispatches[pi].shader)) continue;
    Fused& f = fused_[pi];
    if (f.kind != kProNone || f.more[0] >= 0 || is_output[in] || readers[in].size() != 1) continue;
    if (!weights_[plan_.dispatches[pi].input_buffers[1]]) continue;
    if (plan_.dispatches[pi].epilogue.size() + f.post.size() >= 8) continue;
    // every dispatch between the two must leave the unary's output buffer alone (it is a buffer
    // of its own in a compiled plan, so this always holds; checked because it is cheap)
    f.post.push_back(op);
    f.out_buffer = u.output_buffer;
    producer_of[u.output_buffer] = pi;
    skipped_[ui] = 1;
  }
  plan_chains();
}

void Session::run_dispatches() {
  plan_launches();
  // A norm or SwiGLU dispatch that was folded into the matmuls behind it, run on its own after all
  // (into the buffer the plan gave it); returns that buffer.
  auto run_producer = [&](const Dispatch& p) -> const mgn_buf* {
    const float* in0 = (const float*)buffers_[p.input_buffers[0]]->ptr;
    float* dst = (float*)buffers_[p.output_buffer]->ptr;
    const int e = p.shader == MGN_SHADER_RMS_NORM
                      ? launch_rms_norm(ctx_->stream, in0, (const float*)buffers_[p.input_buffers[1]]->ptr, dst, p.params[0], p.params[1], p.eps)
                      : launch_swiglu_concat(ctx_->stream, in0, dst, p.params[0], p.params[1]);
    if (e != 0) throw std::runtime_error(std::string("kernel launch: ") + hipGetErrorString((hipError_t)e));
    return buffers_[p.output_buffer];
  };
  for (size_t di = 0; di < plan_.dispatches.size(); di++) {
    if (skipped_[di]) continue;
    if (chain_of_[di] >= 0) {  // the whole run goes out with its first launch
      const ChainRun& run = chains_[chain_of_[di]];
      if (run.first == di) check(mgn_chain_run(ctx_, run.chain), "mgn_chain_run");
      continue;
    }
    const Dispatch& d = plan_.dispatches[di];
    float* out = (float*)buffers_[d.output_buffer]->ptr;
    auto fin = [&](size_t i) { return (const float*)buffers_[d.input_buffers[i]]->ptr; };
    int rc = 0;
    switch (d.shader) {
      case MGN_SHADER_MATMUL:
      case MGN_SHADER_MATMUL_GEMV:
      case MGN_SHADER_FUSED_MATMUL_ADD:
      case MGN_SHADER_MATMUL_GEMV_ADD:
      case MGN_SHADER_MATMUL_BT:
      case MGN_SHADER_MATMUL_GEMV_BT:
      case MGN_SHADER_FUSED_MATMUL_BT_ADD:
      case MGN_SHADER_MATMUL_AT:
      case MGN_SHADER_FUSED_MATMUL_AT_ADD: {
        mgn_weight* w = weights_[d.input_buffers[1]];
        if (!w) throw std::runtime_error("quantized parameter was never set");
        const mgn_buf* addend = d.input_buffers.size() > 2 ? buffers_[d.input_buffers[2]] : nullptr;
        const Fused& f = fused_[di];
        if (is_at(d.shader)) {
          std::vector<mgn_unary> ops = d.epilogue;
          ops.insert(ops.end(), f.post.begin(), f.post.end());
          mgn_buf* dst = buffers_[f.out_buffer >= 0 ? f.out_buffer : d.output_buffer];
          check(mgn_matmul_q_at(ctx_, buffers_[d.input_buffers[0]], w, addend, dst, d.params[0], ops.data(), ops.size()),
                "mgn_matmul_q_at");
        } else if (f.more[0] >= 0) {
          mgn_matmul_item items[3] = {{w, addend, buffers_[d.output_buffer]}, {}, {}};
          size_t count = 1;
          for (int sib : f.more) {
            if (sib < 0) continue;
            const Dispatch& sd = plan_.dispatches[sib];
            items[count++] = {weights_[sd.input_buffers[1]],
                              sd.input_buffers.size() > 2 ? buffers_[sd.input_buffers[2]] : nullptr,
                              buffers_[sd.output_buffer]};
          }
          const Dispatch* p = f.kind != kProNone ? &plan_.dispatches[f.producer] : nullptr;
          const mgn_buf* act = p ? buffers_[p->input_buffers[0]] : buffers_[d.input_buffers[0]];
          const mgn_buf* nw = f.kind == kProRmsNorm ? buffers_[p->input_buffers[1]] : nullptr;
          mgn_status st = mgn_matmul_q_batch(ctx_, act, (mgn_prologue)f.kind, nw, p ? p->eps : 0.0f, items, count, d.params[0]);
          if (st == MGN_EUNSUPPORTED) {
            // planned as one launch, refused now (the route was changed since): the producer's own
            // dispatch into its own buffer, then one plain matmul per weight
            const mgn_buf* plain = p ? run_producer(*p) : act;
            st = MGN_OK;
            for (size_t j = 0; j < count && st == MGN_OK; j++) st = mgn_matmul_q(ctx_, plain, items[j].w, items[j].d, items[j].c, d.params[0]);
          }
          check(st, "mgn_matmul_q_batch");
        } else if (f.kind == kProRmsNorm || f.kind == kProSwiglu) {
          const Dispatch& p = plan_.dispatches[f.producer];
          mgn_status st = f.kind == kProRmsNorm
                              ? mgn_matmul_q_rms_norm(ctx_, buffers_[p.input_buffers[0]], buffers_[p.input_buffers[1]], p.eps, w, addend,
                                                      buffers_[d.output_buffer], d.params[0])
                              : mgn_matmul_q_swiglu(ctx_, buffers_[p.input_buffers[0]], w, addend, buffers_[d.output_buffer], d.params[0]);
          if (st == MGN_EUNSUPPORTED)  // as above: the fused kernel no longer takes the call
            st = mgn_matmul_q(ctx_, run_producer(p), w, addend, buffers_[d.output_buffer], d.params[0]);
          check(st, f.kind == kProRmsNorm ? "mgn_matmul_q_rms_norm" : "mgn_matmul_q_swiglu");
        } else if (!d.epilogue.empty() || !f.post.empty()) {
          std::vector<mgn_unary> ops = d.epilogue;
          ops.insert(ops.end(), f.post.begin(), f.post.end());
          mgn_buf* dst = buffers_[f.out_buffer >= 0 ? f.out_buffer : d.output_buffer];
          check(mgn_matmul_q_epilogue(ctx_, buffers_[d.input_buffers[0]], w, addend, dst, d.params[0], ops.data(), ops.size()),
                "mgn_matmul_q_epilogue");
        } else {
          check(mgn_matmul_q(ctx_, buffers_[d.input_buffers[0]], w, addend, buffers_[d.output_buffer], d.params[0]),
                "mgn_matmul_q");
        }
        break;
      }
      case MGN_SHADER_RELU:
      case MGN_SHADER_SIGMOID:
      case MGN_SHADER_NEG:
      case MGN_SHADER_SILU:
        rc = launch_unary(ctx_->stream, (int)unary_of(d.shader), fin(0), out, d.params[0]);
        break;
      case MGN_SHADER_ADD:
        rc = launch_add(ctx_->stream, fin(0), fin(1), out, d.params[0]);
        break;
      case MGN_SHADER_SWIGLU:
        rc = launch_swiglu(ctx_->stream, fin(0), fin(1), out, d.params[0]);
        break;
      case MGN_SHADER_SWIGLU_CONCAT:
        rc = launch_swiglu_concat(ctx_->stream, fin(0), out, d.params[0], d.params[1]);
        break;
      case MGN_SHADER_RMS_NORM:
        rc = launch_rms_norm(ctx_->stream, fin(0), fin(1), out, d.params[0], d.params[1], d.eps);
        break;
    }
    if (rc != 0) throw std::runtime_error(std::string("kernel launch: ") + hipGetErrorString((hipError_t)rc));
  }
}

void Session::wait() { check(mgn_sync(ctx_), "mgn_sync"); }

void Session::read_output_by_index(size_t index, float* out, size_t len) {
  if (index >= plan_.output_buffers.size()) throw std::out_of_range("output index out of range");
  const int buf = plan_.output_buffers[index];
  if (!buffers_[buf]) throw std::runtime_error("output is a quantized parameter");
  if (len * 4 > plan_.buffers[buf]) throw std::invalid_argument("read_output: length exceeds buffer");
  check(mgn_buf_download(ctx_, buffers_[buf], 0, out, len * 4), "mgn_buf_download");
}

std::unique_ptr<Session> build_inference_session(const Graph& g, int device_id) {
  return std::make_unique<Session>(compile(optimize(g)), device_id);
}

}  // namespace mgn

// ------------------------------------------------------------ C wrappers ----

struct mgn_graph {
  mgn::Graph g;
  std::string err;
};

struct mgn_session {
  std::unique_ptr<mgn::Session> s;
  std::string err;
};

namespace {

thread_local std::string g_build_error;

template <class F>
int32_t graph_node(mgn_graph* g, F&& f) {
  if (!g) return -(int32_t)MGN_EINVAL;
  try {
    return (int32_t)f();
  } catch (const std::exception& e) {
    g->err = e.what();
    return -(int32_t)MGN_EINVAL;
  }
}

std::vector<size_t> shape2(size_t rows, size_t cols) { return cols == 0 ? std::vector<size_t>{rows} : std::vector<size_t>{rows, cols}; }

void fill_info(const mgn::Dispatch& d, mgn_dispatch_info* out) {
  out->shader = d.shader;
  for (int i = 0; i < 3; i++) out->workgroups[i] = d.workgroups[i];
  for (int i = 0; i < 4; i++) out->params[i] = d.params[i];
  out->weight_format = (int32_t)d.weight_format;
  out->epilogue = 0;
  for (size_t i = 0; i < d.epilogue.size() && i < 8; i++) out->epilogue |= (uint32_t)d.epilogue[i] << (4 * i);
}

template <class F>
mgn_status session_call(mgn_session* s, F&& f) {
  if (!s || !s->s) return MGN_EINVAL;
  try {
    f();
    return MGN_OK;
  } catch (const std::out_of_range& e) {
    s->err = e.what();
    return MGN_ENOTFOUND;
  } catch (const std::invalid_argument& e) {
    s->err = e.what();
    return MGN_EINVAL;
  } catch (const std::bad_alloc&) {
    s->err = "out of host memory";
    return MGN_ENOMEM;
  } catch (const std::exception& e) {
    s->err = e.what();
    return MGN_EHIP;
  }
}

}  // namespace

extern "C" {

mgn_graph* mgn_graph_new(void) { return new (std::nothrow) mgn_graph(); }
void mgn_graph_free(mgn_graph* g) { delete g; }
const char* mgn_graph_last_error(const mgn_graph* g) { return g ? g->err.c_str() : g_build_error.c_str(); }

// a 1-D shape is passed as cols == 0
int32_t mgn_graph_input(mgn_graph* g, const char* name, size_t rows, size_t cols) {
  return graph_node(g, [&] { return g->g.input(name ? name : "", shape2(rows, cols)); });
}
int32_t mgn_graph_parameter(mgn_graph* g, const char* name, size_t rows, size_t cols) {
  return graph_node(g, [&] { return g->g.parameter(name ? name : "", shape2(rows, cols)); });
}
int32_t mgn_graph_parameter_q4(mgn_graph* g, const char* name, size_t rows, size_t cols) {
  return graph_node(g, [&] { return g->g.parameter_q4(name ? name : "", shape2(rows, cols)); });
}
int32_t mgn_graph_parameter_q8(mgn_graph* g, const char* name, size_t rows, size_t cols) {
  return graph_node(g, [&] { return g->g.parameter_q8(name ? name : "", shape2(rows, cols)); });
}
int32_t mgn_graph_matmul(mgn_graph* g, int32_t a, int32_t b) {
  return graph_node(g, [&] { return g->g.matmul((mgn::NodeId)a, (mgn::NodeId)b); });
}
int32_t mgn_graph_matmul_bt(mgn_graph* g, int32_t a, int32_t b) {
  return graph_node(g, [&] { return g->g.matmul_bt((mgn::NodeId)a, (mgn::NodeId)b); });
}
int32_t mgn_graph_matmul_at(mgn_graph* g, int32_t a, int32_t b) {
  return graph_node(g, [&] { return g->g.matmul_at((mgn::NodeId)a, (mgn::NodeId)b); });
}
int32_t mgn_graph_add(mgn_graph* g, int32_t a, int32_t b) {
  return graph_node(g, [&] { return g->g.add((mgn::NodeId)a, (mgn::NodeId)b); });
}
int32_t mgn_graph_swiglu(mgn_graph* g, int32_t gate, int32_t up) {
  return graph_node(g, [&] { return g->g.swiglu((mgn::NodeId)gate, (mgn::NodeId)up); });
}
int32_t mgn_graph_rms_norm(mgn_graph* g, int32_t x, int32_t weight, float eps) {
  return graph_node(g, [&] { return g->g.rms_norm((mgn::NodeId)x, (mgn::NodeId)weight, eps); });
}

int32_t mgn_graph_unary(mgn_graph* g, int32_t kind, int32_t x) {
  return graph_node(g, [&] { return g->g.unary((mgn_unary)kind, (mgn::NodeId)x); });
}
mgn_status mgn_graph_set_outputs(mgn_graph* g, const int32_t* ids, size_t count) {
  if (!g || (!ids && count)) return MGN_EINVAL;
  try {
    std::vector<mgn::NodeId> v(ids, ids + count);
    g->g.set_outputs(std::move(v));
    return MGN_OK;
  } catch (const std::exception& e) {
    g->err = e.what();
    return MGN_EINVAL;
  }
}

mgn_status mgn_graph_compile(const mgn_graph* g, mgn_dispatch_info* out, size_t cap, size_t* count) {
  if (!g || !count) return MGN_EINVAL;
  try {
    const mgn::ExecutionPlan plan = mgn::compile(mgn::optimize(g->g));
    *count = plan.dispatches.size();
    for (size_t i = 0; i < plan.dispatches.size() && i < cap && out; i++) fill_info(plan.dispatches[i], &out[i]);
    return MGN_OK;
  } catch (const std::exception& e) {
    g_build_error = e.what();
    return MGN_EINVAL;
  }
}

mgn_status mgn_build_inference_session(const mgn_graph* g, int device_id, mgn_session** out) {
  if (!g || !out) return MGN_EINVAL;
  *out = nullptr;
  auto* s = new (std::nothrow) mgn_session();
  if (!s) return MGN_ENOMEM;
  try {
    s->s = mgn::build_inference_session(g->g, device_id);
  } catch (const mgn::GraphError& e) {
    g_build_error = e.what();
    delete s;
    return MGN_EINVAL;
  } catch (const std::exception& e) {
    g_build_error = e.what();
    delete s;
    return std::strstr(e.what(), "mgn_ctx_create") ? MGN_ENODEVICE : MGN_EINVAL;
  }
  *out = s;
  return MGN_OK;
}

void mgn_session_free(mgn_session* s) { delete s; }
const char* mgn_session_last_error(const mgn_session* s) { return s ? s->err.c_str() : g_build_error.c_str(); }

size_t mgn_session_num_dispatches(const mgn_session* s) { return s && s->s ? s->s->plan().dispatches.size() : 0; }

mgn_status mgn_session_dispatch_info(const mgn_session* s, size_t index, mgn_dispatch_info* out) {
  if (!s || !s->s || !out || index >= s->s->plan().dispatches.size()) return MGN_EINVAL;
  fill_info(s->s->plan().dispatches[index], out);
  return MGN_OK;
}

mgn_status mgn_session_set_parameter(mgn_session* s, const char* name, const float* data, size_t len) {
  if (!name || !data) return MGN_EINVAL;
  return session_call(s, [&] { s->s->set_parameter(name, data, len); });
}
mgn_status mgn_session_set_input(mgn_session* s, const char* name, const float* data, size_t len) {
  if (!name || !data) return MGN_EINVAL;
  return session_call(s, [&] { s->s->set_input(name, data, len); });
}
mgn_status mgn_session_step(mgn_session* s) { return session_call(s, [&] { s->s->step(); }); }
mgn_status mgn_session_wait(mgn_session* s) { return session_call(s, [&] { s->s->wait(); }); }
mgn_status mgn_session_set_graph_replay(mgn_session* s, int enable) {
  return session_call(s, [&] { s->s->set_graph_replay(enable != 0); });
}
mgn_status mgn_session_set_fusion(mgn_session* s, int enable) {
  return session_call(s, [&] { s->s->set_fusion(enable != 0); });
}
mgn_status mgn_session_set_chains(mgn_session* s, int enable) {
  return session_call(s, [&] { s->s->set_chains(enable != 0); });
}
size_t mgn_session_num_launches(mgn_session* s) {
  size_t n = 0;
  if (s && s->s) (void)session_call(s, [&] { n = s->s->num_launches(); });
  return n;
}
int mgn_session_graph_active(const mgn_session* s) { return s && s->s && s->s->graph_active() ? 1 : 0; }
mgn_status mgn_session_read_output(mgn_session* s, float* out, size_t len) {
  if (!out) return MGN_EINVAL;
  return session_call(s, [&] { s->s->read_output(out, len); });
}
mgn_status mgn_session_read_output_by_index(mgn_session* s, size_t index, float* out, size_t len) {
  if (!out) return MGN_EINVAL;
  return session_call(s, [&] { s->s->read_output_by_index(index, out, len); });
}
mgn_ctx* mgn_session_ctx(mgn_session* s) { return s && s->s ? s->s->ctx() : nullptr; }

}  // extern "C"
