// Build-time fusion of node sequences the ROCm backend can run as one kernel.  The reference ships
// fused graphs as a second, offline-generated model (model.cpu.pb, tfcc_runtime/framework/model.cpp:
// 74-76,311-322, operations/fusion/); here the plain graph is pattern-matched when it is built:
//
//   MatmulWithBias -> Gelu                 one GEMM with the activation in its tile store
//   MatmulWithBias -> Add(other tensor)    one GEMM that also adds the other tensor (residual)
//   Div(tensor, value) -> Softmax          one softmax pass that divides first
//   Transpose -> Matmul -> Transpose       a batched product that walks the permuted tensors in place
//   Matmul -> [Div] -> Softmax -> Matmul   (each Matmul with its Transposes) the attention core in one launch
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

FusionPlan simple_plan(FusionPlan::Kind kind, size_t partner, unsigned side = 0) {
  FusionPlan f;
  f.kind = kind;
  f.partner = partner;
  f.side = side;
  return f;
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
      plan[j] = simple_plan(FusionPlan::MATMUL_GELU, i, 0);
      plan[i] = simple_plan(FusionPlan::ABSORBED, j);
    } else if (is_op(n, "math.Add", 2) && float_variable(sm, n.outputs[0]) && all_float_tensors(n)) {
      for (unsigned side = 0; side < 2; ++side) {
        if (sole_producer(n.inputs[side], j, i) && is_op(g.nodes[i], "math.MatmulWithBias", 3) &&
            all_float_tensors(g.nodes[i]) && n.inputs[0] != n.inputs[1]) {
          plan[j] = simple_plan(FusionPlan::MATMUL_ADD, i, side);
          plan[i] = simple_plan(FusionPlan::ABSORBED, j);
          break;
        }
      }
    } else if (is_op(n, "math.Softmax", 1) && float_variable(sm, n.outputs[0]) && sole_producer(n.inputs[0], j, i) &&
               is_op(g.nodes[i], "math.Div", 2) && float_tensor(sm, g.nodes[i].inputs[0]) &&
               sm.has(g.nodes[i].inputs[1]) && sm.getSymbolInfo(g.nodes[i].inputs[1]).dtype == FLOAT &&
               is_value(sm.getSymbolInfo(g.nodes[i].inputs[1]).stype)) {
      plan[j] = simple_plan(FusionPlan::DIV_SOFTMAX, i, 0);
      plan[i] = simple_plan(FusionPlan::ABSORBED, j);
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
          if (t2 != FusionPlan::kNoNode) plan[t2] = simple_plan(FusionPlan::ABSORBED, j);
      }
    } else if (is_op(n, "math.MatmulWithBias", 3) && float_variable(sm, n.outputs[0]) && all_float_tensors(n)) {
      // what the converter makes of an ONNX Gemm with transA / transB (tfcc_code_generator/frontend/onnx/converter/
      // math/gemm.py:37-68): Transpose nodes in front of the product's operands
      FusionPlan f;
      f.kind = FusionPlan::MATMUL_PERMUTED;
      size_t t = 0;
      if (sole_producer(n.inputs[0], j, t) && is_op(g.nodes[t], "base.Transpose", 1) && float_tensor(sm, g.nodes[t].inputs[0]))
        f.transposeA = t;
      if (n.inputs[1] != n.inputs[0] && sole_producer(n.inputs[1], j, t) && is_op(g.nodes[t], "base.Transpose", 1) &&
          float_tensor(sm, g.nodes[t].inputs[0]))
        f.transposeB = t;
      if (f.transposeA != FusionPlan::kNoNode || f.transposeB != FusionPlan::kNoNode) {
        plan[j] = f;
        for (size_t t2 : {f.transposeA, f.transposeB})
          if (t2 != FusionPlan::kNoNode) plan[t2] = simple_plan(FusionPlan::ABSORBED, j);
      }
    } else if (is_op(n, "base.Identity", 1) && float_variable(sm, n.outputs[0]) && float_variable(sm, n.inputs[0]) &&
               producer.count(n.inputs[0]) && producer[n.inputs[0]] < j && consumers[n.inputs[0]].size() == 1 &&
               !kept.count(n.inputs[0])) {
      plan[j] = simple_plan(FusionPlan::MOVE_IDENTITY, j, 0);
    }
  }
  // softmax(Q K^T [/ value]) V: two products (with whatever Transposes they folded) around a Softmax
  for (size_t j = 0; j < g.nodes.size(); ++j) {
    const proto::Node& n = g.nodes[j];
    if (!is_op(n, "math.Matmul", 2) || !sm.has(n.outputs[0]) || !float_variable(sm, n.outputs[0]) || !all_float_tensors(n))
      continue;
    if (plan[j].kind != FusionPlan::NONE && plan[j].kind != FusionPlan::MATMUL_PERMUTED) continue;
    if (plan[j].kind == FusionPlan::MATMUL_PERMUTED && plan[j].transposeA != FusionPlan::kNoNode) continue;
    // a value produced by node `from` for one reader, droppable from the graph
    auto private_value = [&](const std::string& name, size_t reader, size_t& from) {
      auto p = producer.find(name);
      if (p == producer.end() || p->second >= reader || kept.count(name)) return false;
      if (consumers[name].size() != 1 || !float_variable(sm, name)) return false;
      from = p->second;
      return true;
    };
    size_t soft = 0, first = 0;
    if (!private_value(n.inputs[0], j, soft) || n.inputs[0] == n.inputs[1]) continue;
    const proto::Node& softNode = g.nodes[soft];
    if (!is_op(softNode, "math.Softmax", 1)) continue;
    if (plan[soft].kind != FusionPlan::NONE && plan[soft].kind != FusionPlan::DIV_SOFTMAX) continue;
    size_t div = plan[soft].kind == FusionPlan::DIV_SOFTMAX ? plan[soft].partner : FusionPlan::kNoNode;
    // Softmax(Add(scores [/ value], mask)): the Add of an attention mask, either operand order
    size_t maskNode = FusionPlan::kNoNode, reader = div != FusionPlan::kNoNode ? div : soft;
    unsigned maskSide = 0;
    std::string scoresName = div != FusionPlan::kNoNode ? g.nodes[div].inputs[0] : softNode.inputs[0];
    size_t add = 0;
    if (div == FusionPlan::kNoNode && private_value(scoresName, soft, add) && is_op(g.nodes[add], "math.Add", 2) &&
        plan[add].kind == FusionPlan::NONE && all_float_tensors(g.nodes[add]) &&
        g.nodes[add].inputs[0] != g.nodes[add].inputs[1]) {
      for (unsigned side = 0; side < 2 && maskNode == FusionPlan::kNoNode; ++side) {
        const std::string& chain = g.nodes[add].inputs[side];
        size_t from = 0;
        if (!private_value(chain, add, from) || plan[from].kind == FusionPlan::ABSORBED) continue;
        const proto::Node& fromNode = g.nodes[from];
        const bool valueDiv = is_op(fromNode, "math.Div", 2) && plan[from].kind == FusionPlan::NONE &&
                              float_tensor(sm, fromNode.inputs[0]) && sm.has(fromNode.inputs[1]) &&
                              sm.getSymbolInfo(fromNode.inputs[1]).dtype == FLOAT &&
                              is_value(sm.getSymbolInfo(fromNode.inputs[1]).stype);
        if (valueDiv) {
          maskNode = add;
          maskSide = 1 - side;
          div = from;
          scoresName = fromNode.inputs[0];
          reader = from;
        } else if (is_op(fromNode, "math.Matmul", 2)) {
          maskNode = add;
          maskSide = 1 - side;
          scoresName = chain;
          reader = add;
        }
      }
      if (maskNode == FusionPlan::kNoNode) continue;
    }
    if (!private_value(scoresName, reader, first)) continue;
    const proto::Node& firstNode = g.nodes[first];
    if (!is_op(firstNode, "math.Matmul", 2) || !all_float_tensors(firstNode)) continue;
    if (plan[first].kind != FusionPlan::NONE && plan[first].kind != FusionPlan::MATMUL_PERMUTED) continue;
    if (plan[first].kind == FusionPlan::MATMUL_PERMUTED && plan[first].transposeC != FusionPlan::kNoNode) continue;
    FusionPlan f;
    f.kind = FusionPlan::ATTENTION;
    f.scoresNode = first;
    f.softmaxNode = soft;
    f.divNode = div;
    f.maskNode = maskNode;
    f.maskSide = maskSide;
    if (plan[first].kind == FusionPlan::MATMUL_PERMUTED) {
      f.transposeA = plan[first].transposeA;
      f.transposeB = plan[first].transposeB;
    }
    if (plan[j].kind == FusionPlan::MATMUL_PERMUTED) {
      f.transposeV = plan[j].transposeB;
      f.transposeC = plan[j].transposeC;
    }
    // every input of the fused step must exist before the first absorbed node ran in the plain order; it runs
    // at the position of the second product (or of its folded Transpose), which is later
    plan[j] = f;
    plan[first] = simple_plan(FusionPlan::ABSORBED, j);
    plan[soft] = simple_plan(FusionPlan::ABSORBED, j);
    if (div != FusionPlan::kNoNode) plan[div] = simple_plan(FusionPlan::ABSORBED, j);
    if (maskNode != FusionPlan::kNoNode) plan[maskNode] = simple_plan(FusionPlan::ABSORBED, j);
    for (size_t t2 : {f.transposeA, f.transposeB, f.transposeV, f.transposeC})
      if (t2 != FusionPlan::kNoNode) plan[t2] = simple_plan(FusionPlan::ABSORBED, j);
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
      for (size_t q = 1; q < count; ++q) plan[f.group[q]] = simple_plan(FusionPlan::ABSORBED, f.group[0]);
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
size_t softmax_axis(const proto::Node& n) {
  size_t axis = 0;
  wire::Reader r(n.operation);
  uint32_t field, type;
  while (r.next(field, type)) {
    if (field == 1 && type == 0) axis = static_cast<size_t>(r.varint());
    else r.skip(type);
  }
  return axis;
}

// transpose(matmul(transpose(a, pa), transpose(b, pb)), pc); an empty perm stands for no Transpose node
Variable<float> permuted_product(const Tensor<float>& a, const std::vector<size_t>& pa, const Tensor<float>& b,
                                 const std::vector<size_t>& pb, const std::vector<size_t>& pc,
                                 const Tensor<float>* bias = nullptr) {
  if (!pa.empty() || !pb.empty() || !pc.empty()) {
    try {
      return rocm::blas::matmul_permuted(a, pa, b, pb, pc, bias);
    } catch (NotImplementedError&) {
      // a layout the strided kernel does not take: run the nodes as written
    }
  }
  Variable<float> xa, xb;
  if (!pa.empty()) xa = base::transpose(a, pa);
  if (!pb.empty()) xb = base::transpose(b, pb);
  const Tensor<float>& ra = pa.empty() ? a : static_cast<const Tensor<float>&>(xa);
  const Tensor<float>& rb = pb.empty() ? b : static_cast<const Tensor<float>&>(xb);
  Variable<float> c = bias ? blas::matmul(ra, rb, *bias) : blas::matmul(ra, rb);
  if (!pc.empty()) return base::transpose(c, pc);
  return c;
}

// softmax(a [/ *divisor], axis)
Variable<float> divided_softmax(const Tensor<float>& a, const float* divisor, size_t axis) {
  if (divisor == nullptr) return math::softmax(a, axis);
  if (axis + 1 == a.shape().size()) return rocm::math::softmax_div(a, axis, *divisor);
  Variable<float> t = a / *divisor;
  return math::softmax(t, axis);
}
}  // namespace

void emit_fused(const proto::Graph& g, const FusionPlan& f, size_t j, Graph& graph) {
  SymbolManager& sm = graph.getSymbolManager();
  const proto::Node& n = g.nodes[j];
  if (f.kind == FusionPlan::ATTENTION) {
    const proto::Node& first = g.nodes[f.scoresNode];
    auto perm_of = [&](size_t node) { return node != FusionPlan::kNoNode ? transpose_perm(g.nodes[node]) : std::vector<size_t>(); };
    auto source = [&](size_t transposeNode, const std::string& name) {
      return sm.getTensor(transposeNode != FusionPlan::kNoNode ? g.nodes[transposeNode].inputs[0] : name, float());
    };
    const Tensor<float>* q = source(f.transposeA, first.inputs[0]);
    const Tensor<float>* k = source(f.transposeB, first.inputs[1]);
    const Tensor<float>* v = source(f.transposeV, n.inputs[1]);
    const std::vector<size_t> pq = perm_of(f.transposeA), pk = perm_of(f.transposeB), pv = perm_of(f.transposeV),
                              po = perm_of(f.transposeC);
    const float* divisor = f.divNode != FusionPlan::kNoNode ? sm.getValue(g.nodes[f.divNode].inputs[1], float()) : nullptr;
    const size_t axis = softmax_axis(g.nodes[f.softmaxNode]);
    const Tensor<float>* mask =
        f.maskNode != FusionPlan::kNoNode ? sm.getTensor(g.nodes[f.maskNode].inputs[f.maskSide], float()) : nullptr;
    const bool maskFirst = f.maskSide == 0;
    Variable<float>* result =
        sm.getVariable(f.transposeC != FusionPlan::kNoNode ? g.nodes[f.transposeC].outputs[0] : n.outputs[0], float());
    graph.addStep([q, k, v, pq, pk, pv, po, divisor, axis, mask, maskFirst, result] {
      if (axis == 3 && q->shape().size() == 4 && k->shape().size() == 4 && v->shape().size() == 4) {
        try {
          *result = rocm::blas::attention_permuted(*q, pq, *k, pk, *v, pv, po, divisor, mask);
          return;
        } catch (NotImplementedError&) {
          // longer sequences, wider heads, another layout or mask shape: the steps one after the other
        }
      }
      Variable<float> scores = permuted_product(*q, pq, *k, pk, {});
      Variable<float> probabilities;
      if (mask == nullptr) {
        probabilities = divided_softmax(scores, divisor, axis);
      } else {
        if (divisor != nullptr) scores = scores / *divisor;
        Variable<float> masked = maskFirst ? *mask + scores : scores + *mask;
        probabilities = math::softmax(masked, axis);
      }
      *result = permuted_product(probabilities, {}, *v, pv, po);
    });
    return;
  }
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
    const Tensor<float>* bias = n.inputs.size() == 3 ? sm.getTensor(n.inputs[2], float()) : nullptr;
    // A constant weight given transposed (a Linear layer exported as Gemm with transB): transposed once, at the
    // first run, and multiplied as stored from then on - the plain graph transposes it in every run.
    if (tb && sm.getSymbolInfo(g.nodes[f.transposeB].inputs[0]).stype == SymbolType::CONSTANT_TENSOR) {
      auto cached = std::make_shared<Variable<float>>();
      auto filled = std::make_shared<bool>(false);
      graph.addStep([a, b, result, pa, pb, pc, bias, cached, filled] {
        if (!*filled) {
          *cached = base::transpose(*b, pb);
          *filled = true;
        }
        *result = permuted_product(*a, pa, *cached, {}, pc, bias);
      });
      return;
    }
    graph.addStep([a, b, result, pa, pb, pc, bias] { *result = permuted_product(*a, pa, *b, pb, pc, bias); });
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
    const size_t axis = softmax_axis(n);
    graph.addStep([a, divisor, axis, out] { *out = divided_softmax(*a, divisor, axis); });
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
