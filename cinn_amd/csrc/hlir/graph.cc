#include "hlir/graph.h"

#include <algorithm>
#include <sstream>

namespace cinn {
namespace hlir {
namespace framework {

NodeData* Graph::GetOrCreateVar(const frontend::Variable& v) {
  auto it = vars_.find(v->id);
  if (it != vars_.end()) return it->second.get();
  auto data   = std::make_unique<NodeData>();
  data->id    = v->id;
  data->shape = v->shape;
  data->dtype = v->type;
  data->is_const = v->is_const;
  auto* p     = data.get();
  vars_[v->id] = std::move(data);
  return p;
}

Graph::Graph(const frontend::Program& program, const std::set<std::string>& fetch_ids, const common::Target& target)
    : target_(target) {
  for (char c : program.name()) name_.push_back((isalnum(static_cast<unsigned char>(c)) || c == '_') ? c : '_');
  for (auto& in : program.GetInputs()) inputs_.push_back(GetOrCreateVar(in));

  // Common sub-expression elimination while the graph is built: an instruction with the same op,
  // inputs and attributes as an earlier one reuses the earlier outputs.  The softmax decomposition,
  // for example, evaluates exp(x) twice; this keeps one.
  std::map<std::string, Node*> seen;
  std::map<std::string, NodeData*> alias;  // id of an eliminated output -> surviving value
  auto resolve = [&](const frontend::Variable& v) -> NodeData* {
    auto it = alias.find(v->id);
    if (it != alias.end()) return it->second;
    return GetOrCreateVar(v);
  };

  for (auto& ins : program.instructions()) {
    const Operator& op = OpRegistry::Global().Get(ins->op_type);
    std::vector<NodeData*> ins_inputs;
    for (auto& v : ins->inputs) ins_inputs.push_back(resolve(v));
    for (auto* in : ins_inputs) {
      CINN_CHECK(in->producer || std::find(inputs_.begin(), inputs_.end(), in) != inputs_.end())
          << "variable " << in->id << " is used by " << ins->op_type << " before it is defined";
    }

    std::ostringstream key;
    key << ins->op_type << "(";
    for (auto* in : ins_inputs) key << in->id << ",";
    key << ")";
    for (auto& kv : ins->attrs) key << kv.first << "=" << utils::AttributeToString(kv.second) << ";";
    bool any_fetch = false;
    for (auto& o : ins->outputs) any_fetch |= fetch_ids.count(o->id) != 0;
    auto sit = seen.find(key.str());
    if (sit != seen.end() && !any_fetch && ins->op_type != "fill_constant") {
      for (size_t i = 0; i < ins->outputs.size(); ++i) alias[ins->outputs[i]->id] = sit->second->outputs[i];
      continue;
    }

    auto node   = std::make_unique<Node>();
    node->index = static_cast<int>(nodes_.size());
    node->op    = &op;
    node->attrs = ins->attrs;
    node->inputs = ins_inputs;
    for (auto* in : ins_inputs) in->consumers.push_back(node.get());
    for (auto& o : ins->outputs) {
      auto* out = GetOrCreateVar(o);
      CINN_CHECK(!out->producer) << "variable " << out->id << " is written twice";
      out->producer = node.get();
      out->is_fetch = fetch_ids.count(out->id) != 0;
      node->outputs.push_back(out);
    }
    seen[key.str()] = node.get();
    nodes_.push_back(std::move(node));
  }
  for (auto& id : fetch_ids) {
    auto* v = FindVar(id);
    CINN_CHECK(v) << "fetch variable " << id << " does not exist in the program";
    v->is_fetch = true;
  }
  ConstPropagate();
}

// ConstPropagatePass (cinn/hlir/pass/const_propagate.cc:33-58): a node whose inputs are all const is a pre-run node
// and its outputs are const.  Only fed inputs start const-ness here; a fill_constant joins the pre-run set when
// a pre-run node consumes it, otherwise it stays with (and is folded into) its consumers.
void Graph::ConstPropagate() {
  auto known = [](const NodeData* in) {
    return in->is_const || (in->producer && in->producer->op_type() == "fill_constant");
  };
  // Nodes are in program order, so one sweep settles everything but replications, which look at their consumers'
  // other inputs: sweep until nothing changes.
  for (bool changed = true; changed;) {
    changed = false;
    for (auto& np : nodes_) {
      Node* n = np.get();
      if (n->pre_run || n->op_type() == "fill_constant") continue;
      bool all_const = !n->inputs.empty();
      for (auto* in : n->inputs) all_const = all_const && known(in);
      // something fed must take part: a chain of literals alone is folded, not pre-run
      bool any_fed = false;
      for (auto* in : n->inputs) any_fed = any_fed || in->is_const;
      if (!all_const || !any_fed) continue;
      if (n->op->pattern == OpPatternKind::kBroadcast) {
        // Replicating a const value is left to the consumer, which reads the small tensor in place: materialising the
        // replicated tensor once would turn a per-channel vector into a full activation-sized read in every execution.
        // Unless every consumer is computed from const values alone (a scale multiplied into a filter): then the
        // replication runs once with them.
        bool only_const_consumers = !n->outputs.empty();
        for (auto* o : n->outputs) {
          only_const_consumers = only_const_consumers && !o->consumers.empty() && !o->is_fetch;
          for (Node* c : o->consumers)
            for (auto* in : c->inputs) only_const_consumers = only_const_consumers && (in == o || known(in));
        }
        if (!only_const_consumers) continue;
      }
      n->pre_run = true;
      for (auto* o : n->outputs) o->is_const = true;
      changed = true;
    }
  }
  for (auto& np : nodes_) {
    Node* n = np.get();
    if (n->op_type() != "fill_constant" || n->outputs[0]->consumers.empty()) continue;
    // with consumers on both sides it is computed once up front and read from memory by the others
    // a library call cannot fold a literal into its kernel: what it reads is filled once as well
    bool any_pre_run = false;
    for (Node* c : n->outputs[0]->consumers)
      any_pre_run = any_pre_run || c->pre_run || c->op->pattern == OpPatternKind::kNonFusible;
    n->pre_run = any_pre_run;
  }
}

NodeData* Graph::FindVar(const std::string& id) const {
  auto it = vars_.find(id);
  return it == vars_.end() ? nullptr : it->second.get();
}

std::vector<NodeData*> Graph::AllVars() const {
  std::vector<NodeData*> out;
  for (auto& kv : vars_) out.push_back(kv.second.get());
  return out;
}

std::string Graph::DebugGroupString() const {
  std::ostringstream os;
  for (auto& g : groups) {
    os << "group " << g->id << " ";
    switch (g->kind) {
      case GroupKind::kElementwise: os << "elementwise"; break;
      case GroupKind::kRowReduce: os << "row_reduce[" << g->rows << "x" << g->cols << "]"; break;
      case GroupKind::kGeneralReduce: os << "general_reduce"; break;
      case GroupKind::kLibraryCall: os << "library_call"; break;
    }
    if (g->pre_run) os << " pre_run";
    os << " {";
    for (auto* n : g->nodes) os << " " << n->op_type();
    os << " } in:";
    for (auto* v : g->inputs) os << " " << v->id;
    os << " out:";
    for (auto* v : g->outputs) os << " " << v->id;
    os << "\n";
  }
  return os.str();
}

bool IsReduceRun(const Node& node) { return node.op_type().rfind("reduce_run_", 0) == 0; }

std::vector<int> ReduceDimsOf(const Node& node) {
  int rank = static_cast<int>(node.inputs[0]->shape.size());
  std::vector<int> dims;
  if (node.op->reduce_kind == "argmax" || node.op->reduce_kind == "argmin") {
    int axis = GetAttr<int>(node.attrs, "axis", 0);
    if (axis < 0) axis += rank;
    dims.push_back(axis);
  } else {
    dims = GetAttr<std::vector<int>>(node.attrs, "dim", {});
    if (dims.empty()) {
      for (int i = 0; i < rank; ++i) dims.push_back(i);
    }
    for (auto& d : dims)
      if (d < 0) d += rank;
    std::sort(dims.begin(), dims.end());
    dims.erase(std::unique(dims.begin(), dims.end()), dims.end());
  }
  return dims;
}

bool TrailingReduceSpace(const ShapeType& shape, const std::vector<int>& dims, int64_t* rows, int64_t* cols) {
  int rank = static_cast<int>(shape.size());
  std::vector<bool> reduced(rank, false);
  for (int d : dims) reduced[d] = true;
  // once a reduced axis of size > 1 is seen, every later axis of size > 1 must be reduced as well
  bool in_tail = false;
  int64_t r = 1, c = 1;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 1) continue;
    if (reduced[i]) {
      in_tail = true;
      c *= shape[i];
    } else {
      if (in_tail) return false;
      r *= shape[i];
    }
  }
  *rows = r;
  *cols = c;
  return true;
}

RowKind ClassifyBroadcastInput(const ShapeType& in_shape, const ShapeType& out_shape, const std::vector<int>& axes,
                               int64_t rows, int64_t cols) {
  int64_t in_numel = ShapeNumel(in_shape);
  if (ShapeNumel(out_shape) != rows * cols) return RowKind::kInvalid;
  if (in_numel == 1) return RowKind::kScalar;
  if (in_numel == rows * cols) return RowKind::kElem;
  // position in out_shape where the leading product reaches `rows`
  int split = -1;
  int64_t prod = 1;
  if (rows == 1) split = 0;
  for (size_t i = 0; i < out_shape.size() && split < 0; ++i) {
    prod *= out_shape[i];
    if (prod == rows) split = static_cast<int>(i) + 1;
    if (prod > rows) break;
  }
  if (split < 0) return RowKind::kInvalid;
  bool all_lead = true, all_tail = true;
  int out_rank  = static_cast<int>(out_shape.size());
  int prev_axis = -1;
  for (size_t i = 0; i < in_shape.size(); ++i) {
    if (in_shape[i] == 1) continue;
    int ax = axes[i] < 0 ? axes[i] + out_rank : axes[i];
    if (ax <= prev_axis) return RowKind::kInvalid;  // a permuting broadcast is not a plain row / column vector
    prev_axis = ax;
    // size-1 output axes right at the split can belong to either side
    if (ax >= split) all_lead = false;
    if (ax < split) all_tail = false;
  }
  if (all_lead && in_numel == rows) return RowKind::kRow;
  if (all_tail && in_numel == cols) return RowKind::kCol;
  return RowKind::kInvalid;
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
