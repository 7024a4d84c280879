// Build-time fusion of node sequences the ROCm backend can run as one kernel.  The reference ships
// fused graphs as a second, offline-generated model (model.cpu.pb, tfcc_runtime/framework/model.cpp:
// 74-76,311-322, operations/fusion/); here the plain graph is pattern-matched when it is built:
//
//   MatmulWithBias -> Gelu                 one GEMM with the activation in its tile store
//   MatmulWithBias -> Add(other tensor)    one GEMM that also adds the other tensor (residual)
//   Div(tensor, value) -> Softmax          one softmax pass that divides first
//   Transpose -> Matmul -> Transpose       a batched product that walks the permuted tensors in place
//   2-4 x MatmulWithBias on one input with constant weights of one shape (query / key / value): one launch
//   Identity of a variable nobody else reads: the buffer is handed over instead of copied
//
// A producer is absorbed only when its output is a float VARIABLE symbol with exactly one consumer
// that is not an output of the graph, and when every symbol of the graph has one producer.  Each
// fused kernel rounds to fp32 after every original step, so results are bit-identical to the
// unfused graph; when a run-time shape does not fit the fused form the steps run unfused.
#include <unordered_map>

#include "runtime.h"
#include "tfcc_rocm_device.h"

namespace tfcc {
namespace runtime {

namespace {

bool is_op(const proto::Node& n, const char* message, size_t inputs) {
  return n.version == 1 && n.typeUrl == type_url(message) && n.inputs.size() == inputs && n.outputs.size() == 1;
}

bool float_tensor(SymbolManager& sm, const std::string& name) {
  if (!sm.has(name)) return false;
  const SymbolInfo& info = sm.getSymbolInfo(name);
  return info.dtype == FLOAT && is_tensor(info.stype);
}

bool float_variable(SymbolManager& sm, const std::string& name) {
  if (!sm.has(name)) return false;
  const SymbolInfo& info = sm.getSymbolInfo(name);
  return info.dtype == FLOAT && info.stype == SymbolType::VARIABLE;
}

}  // namespace

std::vector<FusionPlan> plan_fusions(const proto::Graph& g, SymbolManager& sm) {
  std::vector<FusionPlan> plan(g.nodes.size());
  std::unordered_map<std::string, size_t> producer;
  std::unordered_map<std::string, std::vector<size_t>> consumers;
  for (size_t i = 0; i < g.nodes.size(); ++i) {
    for (const std::string& o : g.nodes[i].outputs) {
      if (producer.count(o)) return plan;  // a symbol written twice: leave the graph as it is
      producer[o] = i;
    }
    for (const std::string& in : g.nodes[i].inputs) consumers[in].push_back(i);
  }
  std::set<std::string> kept(g.outputs.begin(), g.outputs.end());
  for (const std::string& in : g.inputs)
    if (producer.count(in)) return plan;

  // the node that alone produces `name` for node j, if absorbing it is allowed
  auto sole_producer = [&](const std::string& name, size_t j, size_t& i) {
    auto p = producer.find(name);
    if (p == producer.end() || p->second >= j || kept.count(name)) return false;
    if (consumers[name].size() != 1 || plan[p->second].kind != FusionPlan::NONE) return false;
    if (!float_variable(sm, name)) return false;
    i = p->second;
    return true;
  };
  auto all_float_tensors = [&](const proto::Node& n) {
    for (const std::string& s : n.inputs)
      if (!float_tensor(sm, s)) return false;
    return true;
  };

  for (size_t j = 0; j < g.nodes.size(); ++j) {
    const proto::Node& n = g.nodes[j];
    if (plan[j].kind != FusionPlan::NONE) continue;
    if (!sm.has(n.outputs.empty() ? std::string() : n.outputs[0])) continue;
    size_t i = 0;
    if (is_op(n, "math.Gelu", 1) && float_variable(sm, n.outputs[0]) && sole_producer(n.inputs[0], j, i) &&
        is_op(g.nodes[i], "math.MatmulWithBias", 3) && all_float_tensors(g.nodes[i])) {
      plan[j] = {FusionPlan::MATMUL_GELU, i, 0};
      plan[i] = {FusionPlan::ABSORBED, j, 0};
    } else if (is_op(n, "math.Add", 2) && float_variable(sm, n.outputs[0]) && all_float_tensors(n)) {
      for (unsigned side = 0; side < 2; ++side) {
        if (sole_producer(n.inputs[side], j, i) && is_op(g.nodes[i], "math.MatmulWithBias", 3) &&
            all_float_tensors(g.nodes[i]) && n.inputs[0] != n.inputs[1]) {
          plan[j] = {FusionPlan::MATMUL_ADD, i, side};
          plan[i] = {FusionPlan::ABSORBED, j, 0};
          break;
        }
      }
    } else if (is_op(n, "math.Softmax", 1) && float_variable(sm, n.outputs[0]) && sole_producer(n.inputs[0], j, i) &&
               is_op(g.nodes[i], "math.Div", 2) && float_tensor(sm, g.nodes[i].inputs[0]) &&
               sm.has(g.nodes[i].inputs[1]) && sm.getSymbolInfo(g.nodes[i].inputs[1]).dtype == FLOAT &&
               is_value(sm.getSymbolInfo(g.nodes[i].inputs[1]).stype)) {
      plan[j] = {FusionPlan::DIV_SOFTMAX, i, 0};
      plan[i] = {FusionPlan::ABSORBED, j, 0};
    } else if (is_op(n, "math.Matmul", 2) && float_variable(sm, n.outputs[0]) && all_float_tensors(n)) {
      FusionPlan f;
      f.kind = FusionPlan::MATMUL_PERMUTED;
      size_t t = 0;
      if (sole_producer(n.inputs[0], j, t) && is_op(g.nodes[t], "base.Transpose", 1) && float_tensor(sm, g.nodes[t].inputs[0]))
        f.transposeA = t;
      if (n.inputs[1] != n.inputs[0] && sole_producer(n.inputs[1], j, t) && is_op(g.nodes[t], "base.Transpose", 1) &&
          float_tensor(sm, g.nodes[t].inputs[0]))
        f.transposeB = t;
      const std::string& out = n.outputs[0];
      if (!kept.count(out) && consumers[out].size() == 1 && consumers[out][0] > j) {
        const size_t c = consumers[out][0];
        if (plan[c].kind == FusionPlan::NONE && is_op(g.nodes[c], "base.Transpose", 1) &&
            float_variable(sm, g.nodes[c].outputs[0]))
          f.transposeC = c;
      }
      if (f.transposeA != FusionPlan::kNoNode || f.transposeB != FusionPlan::kNoNode || f.transposeC != FusionPlan::kNoNode) {
        plan[j] = f;
        for (size_t t2 : {f.transposeA, f.transposeB, f.transposeC})
          if (t2 != FusionPlan::kNoNode) plan[t2] = {FusionPlan::ABSORBED, j, 0};
      }
    } else if (is_op(n, "base.Identity", 1) && float_variable(sm, n.outputs[0]) && float_variable(sm, n.inputs[0]) &&
               producer.count(n.inputs[0]) && producer[n.inputs[0]] < j && consumers[n.inputs[0]].size() == 1 &&
               !kept.count(n.inputs[0])) {
      plan[j] = {FusionPlan::MOVE_IDENTITY, j, 0};
    }
  }
  // MatmulWithBias nodes left as they are that share their input and have constant weights: groups of up to 4
  std::unordered_map<std::string, std::vector<size_t>> byInput;
  std::vector<std::string> order;
  for (size_t j = 0; j < g.nodes.size(); ++j) {
    const proto::Node& n = g.nodes[j];
    if (plan[j].kind != FusionPlan::NONE || !is_op(n, "math.MatmulWithBias", 3) || !all_float_tensors(n) ||
        !float_variable(sm, n.outputs[0]))
      continue;
    if (sm.getSymbolInfo(n.inputs[1]).stype != SymbolType::CONSTANT_TENSOR ||
        sm.getSymbolInfo(n.inputs[2]).stype != SymbolType::CONSTANT_TENSOR)
      continue;
    // the shared input must exist before the first member runs: a graph input or produced earlier
    auto p = producer.find(n.inputs[0]);
    if (p != producer.end() && p->second >= j) continue;
    if (!byInput.count(n.inputs[0])) order.push_back(n.inputs[0]);
    byInput[n.inputs[0]].push_back(j);
  }
  for (const std::string& name : order) {
    std::vector<size_t>& members = byInput[name];
    // the input's producer must precede the first member (members are in node order)
    auto p = producer.find(name);
    if (p != producer.end() && p->second > members.front()) continue;
    for (size_t at = 0; at + 1 < members.size(); at += 4) {
      const size_t count = std::min<size_t>(4, members.size() - at);
      if (count < 2) break;
      FusionPlan f;
      f.kind = FusionPlan::MATMUL_GROUPED;
      f.group.assign(members.begin() + at, members.begin() + at + count);
      for (size_t q = 1; q < count; ++q) plan[f.group[q]] = {FusionPlan::ABSORBED, f.group[0], 0};
      plan[f.group[0]] = f;
    }
  }
  return plan;
}

namespace {
std::vector<size_t> transpose_perm(const proto::Node& n) {
  std::vector<size_t> perm;
  wire::Reader r(n.operation);
  uint32_t field, type;
  while (r.next(field, type)) {
    if (field == 1) r.repeatedVarint(type, perm);
    else r.skip(type);
  }
  return perm;
}
}  // namespace

void emit_fused(const proto::Graph& g, const FusionPlan& f, size_t j, Graph& graph) {
  SymbolManager& sm = graph.getSymbolManager();
  const proto::Node& n = g.nodes[j];
  if (f.kind == FusionPlan::MATMUL_GROUPED) {
    const Tensor<float>* a = sm.getTensor(n.inputs[0], float());
    std::vector<const Tensor<float>*> bs, biases;
    std::vector<Variable<float>*> outs;
    for (size_t member : f.group) {
      bs.push_back(sm.getTensor(g.nodes[member].inputs[1], float()));
      biases.push_back(sm.getTensor(g.nodes[member].inputs[2], float()));
      outs.push_back(sm.getVariable(g.nodes[member].outputs[0], float()));
    }
    graph.addStep([a, bs, biases, outs] {
      try {
        std::vector<Variable<float>> results = rocm::blas::matmul_grouped(*a, bs, biases);
        for (size_t q = 0; q < outs.size(); ++q) *outs[q] = std::move(results[q]);
        return;
      } catch (NotImplementedError&) {
        // weights of different shapes, or a layout the grouped launch does not take: one launch each
      }
      for (size_t q = 0; q < outs.size(); ++q) *outs[q] = blas::matmul(*a, *bs[q], *biases[q]);
    });
    return;
  }
  if (f.kind == FusionPlan::MATMUL_PERMUTED) {
    const bool ta = f.transposeA != FusionPlan::kNoNode, tb = f.transposeB != FusionPlan::kNoNode,
               tc = f.transposeC != FusionPlan::kNoNode;
    const Tensor<float>* a = sm.getTensor(ta ? g.nodes[f.transposeA].inputs[0] : n.inputs[0], float());
    const Tensor<float>* b = sm.getTensor(tb ? g.nodes[f.transposeB].inputs[0] : n.inputs[1], float());
    Variable<float>* result = sm.getVariable(tc ? g.nodes[f.transposeC].outputs[0] : n.outputs[0], float());
    const std::vector<size_t> pa = ta ? transpose_perm(g.nodes[f.transposeA]) : std::vector<size_t>();
    const std::vector<size_t> pb = tb ? transpose_perm(g.nodes[f.transposeB]) : std::vector<size_t>();
    const std::vector<size_t> pc = tc ? transpose_perm(g.nodes[f.transposeC]) : std::vector<size_t>();
    graph.addStep([a, b, result, pa, pb, pc, ta, tb, tc] {
      try {
        *result = rocm::blas::matmul_permuted(*a, pa, *b, pb, pc);
        return;
      } catch (NotImplementedError&) {
        // a layout the strided kernel does not take: run the nodes as written
      }
      Variable<float> xa, xb;
      if (ta) xa = base::transpose(*a, pa);
      if (tb) xb = base::transpose(*b, pb);
      Variable<float> c = blas::matmul(ta ? static_cast<const Tensor<float>&>(xa) : *a,
                                       tb ? static_cast<const Tensor<float>&>(xb) : *b);
      if (tc) *result = base::transpose(c, pc);
      else *result = std::move(c);
    });
    return;
  }
  Variable<float>* out = sm.getVariable(n.outputs[0], float());
  if (f.kind == FusionPlan::MOVE_IDENTITY) {
    Variable<float>* in = sm.getVariable(n.inputs[0], float());
    graph.addStep([in, out] { *out = std::move(*in); });
    return;
  }
  const proto::Node& p = g.nodes[f.partner];
  if (f.kind == FusionPlan::DIV_SOFTMAX) {
    const Tensor<float>* a = sm.getTensor(p.inputs[0], float());
    const float* divisor = sm.getValue(p.inputs[1], float());
    size_t axis = 0;
    wire::Reader r(n.operation);
    uint32_t field, type;
    while (r.next(field, type)) {
      if (field == 1 && type == 0) axis = static_cast<size_t>(r.varint());
      else r.skip(type);
    }
    graph.addStep([a, divisor, axis, out] {
      if (axis + 1 == a->shape().size()) {
        *out = rocm::math::softmax_div(*a, axis, *divisor);
      } else {
        Variable<float> t = *a / *divisor;
        *out = math::softmax(t, axis);
      }
    });
    return;
  }
  const Tensor<float>* a = sm.getTensor(p.inputs[0], float());
  const Tensor<float>* b = sm.getTensor(p.inputs[1], float());
  const Tensor<float>* bias = sm.getTensor(p.inputs[2], float());
  if (f.kind == FusionPlan::MATMUL_GELU) {
    graph.addStep([a, b, bias, out] {
      *out = rocm::blas::matmul_fused(*a, *b, bias, nullptr, rocm::blas::Activation::GELU);
    });
    return;
  }
  // MATMUL_ADD: the Add's other operand is the residual when it has the product's shape
  const Tensor<float>* other = sm.getTensor(n.inputs[1 - f.side], float());
  const bool productFirst = f.side == 0;
  graph.addStep([a, b, bias, other, productFirst, out] {
    const size_t ra = a->shape().size(), rb = b->shape().size();
    bool fits = ra >= 2 && rb >= 2 && a->size() > 0 && b->size() > 0;
    if (fits) {
      std::vector<unsigned> s = ra >= rb ? a->shape().toVector() : b->shape().toVector();
      s[s.size() - 2] = a->shape(ra - 2);
      s[s.size() - 1] = b->shape(rb - 1);
      fits = other->shape() == Shape(std::move(s));
    }
    if (fits) {
      *out = rocm::blas::matmul_fused(*a, *b, bias, other, rocm::blas::Activation::NONE);
    } else {
      Variable<float> t = blas::matmul(*a, *b, *bias);
      *out = productFirst ? t + *other : *other + t;
    }
  });
}

}  // namespace runtime
}  // namespace tfcc
