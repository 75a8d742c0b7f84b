// Partition of the graph into fusion groups.  It plays the role of OpFusionPass + FusionMergePass
// (cinn/hlir/pass/op_fusion_pass.cc, fusion_merge_pass.cc) for the gfx950 backend with a rule set
// that is driven by what one kernel template can hold:
//   - every node starts as its own group;
//   - a producer group and a consumer group merge when the union is still expressible by one
//     template (element-wise over one flat space, or row-resident reduce over one rows x cols space)
//     and the merge closes no cycle in the group graph, i.e. there is no other path from the producer
//     to the consumer; merging repeats until nothing changes.  A value with consumers outside the
//     merged group simply stays an output of it, so no computation is ever duplicated;
//   - then sibling groups merge (horizontal fusion, fusion_merge_pass.cc:85-120 and 176-260): two groups that read
//     the same value, live in the same iteration space (equal flat size, or equal rows x cols) and do not depend
//     on each other become one kernel that reads the shared value once - `reduce_sum(x)` and `argmax(x)` of one
//     tensor are one pass over x;
//   - kNonFusible ops and reductions over non-trailing axes stay alone.
#include <algorithm>
#include <cstdlib>
#include <map>
#include <set>

#include "hlir/graph.h"

namespace cinn {
namespace hlir {
namespace framework {

namespace {

bool IsRowGroupOp(const Node& n) {
  if (n.op->pattern == OpPatternKind::kElementWise) return true;
  if (n.op->pattern == OpPatternKind::kReduction) return true;
  return n.op_type() == "broadcast_to" || n.op_type() == "reshape";
}

bool IsFusibleOp(const Node& n) {
  switch (n.op->pattern) {
    case OpPatternKind::kElementWise:
    case OpPatternKind::kBroadcast:
    case OpPatternKind::kInjective: return true;
    default: return false;
  }
}

struct WorkGroup {
  GroupKind kind;
  std::vector<Node*> nodes;  // kept sorted by node index
  bool pre_run{false};
  int64_t numel{0};          // kElementwise: size of the flat space
  int64_t rows{0}, cols{0};  // kRowReduce
};

std::vector<Node*> WithNode(const std::vector<Node*>& nodes, Node* n) {
  std::vector<Node*> out = nodes;
  out.push_back(n);
  std::sort(out.begin(), out.end(), [](Node* a, Node* b) { return a->index < b->index; });
  return out;
}

}  // namespace

bool ClassifyRowReduceGroup(const std::vector<Node*>& nodes, int64_t rows, int64_t cols,
                            std::map<const NodeData*, RowKind>* kinds) {
  std::map<const NodeData*, RowKind> k;
  auto by_numel = [&](const NodeData* v) {
    int64_t n = v->numel();
    if (n == rows * cols) return RowKind::kElem;
    if (n == rows) return RowKind::kRow;
    if (n == 1) return RowKind::kScalar;
    return RowKind::kInvalid;
  };
  auto set_kind = [&](const NodeData* v, RowKind kind) -> bool {
    if (kind == RowKind::kInvalid) return false;
    auto it = k.find(v);
    if (it != k.end() && it->second != kind) {
      // a scalar may be used where a row value is expected and vice versa when rows == 1
      bool compatible = (it->second == RowKind::kScalar && kind == RowKind::kRow && rows == 1) ||
                        (it->second == RowKind::kRow && kind == RowKind::kScalar && rows == 1);
      if (!compatible) return false;
      return true;
    }
    k[v] = kind;
    return true;
  };
  if (cols <= 1) return false;
  for (Node* n : nodes) {
    if (!IsRowGroupOp(*n)) return false;
    if (n->op->pattern == OpPatternKind::kReduction) {
      int64_t r, c;
      if (!TrailingReduceSpace(n->inputs[0]->shape, ReduceDimsOf(*n), &r, &c)) return false;
      if (r != rows || c != cols) return false;
      if (!set_kind(n->inputs[0], RowKind::kElem)) return false;
      if (!set_kind(n->outputs[0], RowKind::kRow)) return false;
      continue;
    }
    if (n->op_type() == "broadcast_to") {
      auto axes = GetAttr<std::vector<int>>(n->attrs, "broadcast_axes", {});
      int64_t out_numel = n->outputs[0]->numel();
      if (out_numel == rows * cols) {
        RowKind in_kind = ClassifyBroadcastInput(n->inputs[0]->shape, n->outputs[0]->shape, axes, rows, cols);
        if (!set_kind(n->inputs[0], in_kind)) return false;
        if (!set_kind(n->outputs[0], RowKind::kElem)) return false;
      } else if (out_numel == rows && n->inputs[0]->numel() == 1) {
        if (!set_kind(n->inputs[0], RowKind::kScalar)) return false;
        if (!set_kind(n->outputs[0], RowKind::kRow)) return false;
      } else if (out_numel == rows && n->inputs[0]->numel() == rows) {
        if (!set_kind(n->inputs[0], RowKind::kRow)) return false;
        if (!set_kind(n->outputs[0], RowKind::kRow)) return false;
      } else {
        return false;
      }
      continue;
    }
    if (n->op_type() == "fill_constant") {
      // a constant is a scalar whatever its nominal shape, but it must be usable where it is consumed
      k[n->outputs[0]] = by_numel(n->outputs[0]);
      if (k[n->outputs[0]] == RowKind::kInvalid) return false;
      continue;
    }
    // element-wise ops and reshape: every operand and the result live in the same space
    RowKind out_kind = by_numel(n->outputs[0]);
    if (out_kind == RowKind::kInvalid) return false;
    for (auto* in : n->inputs) {
      if (by_numel(in) != out_kind) return false;
      if (!set_kind(in, out_kind)) return false;
    }
    for (auto* out : n->outputs)
      if (!set_kind(out, out_kind)) return false;
  }
  // a column vector may only enter through broadcast_to from outside the group
  std::map<const NodeData*, bool> produced;
  for (Node* n : nodes)
    for (auto* o : n->outputs) produced[o] = true;
  for (auto& kv : k)
    if (kv.second == RowKind::kCol && produced.count(kv.first)) return false;
  if (kinds) *kinds = std::move(k);
  return true;
}

void Graph::BuildFusionGroups() {
  groups.clear();
  std::vector<std::unique_ptr<WorkGroup>> work;
  std::map<Node*, WorkGroup*> group_of;

  // every node starts alone
  for (auto& np : nodes_) {
    Node* n = np.get();
    auto g  = std::make_unique<WorkGroup>();
    g->nodes.push_back(n);
    g->pre_run = n->pre_run;
    if (n->op->pattern == OpPatternKind::kReduction && IsReduceRun(*n)) {
      g->kind = GroupKind::kGeneralReduce;
    } else if (n->op->pattern == OpPatternKind::kReduction) {
      int64_t r, c;
      if (TrailingReduceSpace(n->inputs[0]->shape, ReduceDimsOf(*n), &r, &c) && c > 1 &&
          ClassifyRowReduceGroup(g->nodes, r, c, nullptr)) {
        g->kind = GroupKind::kRowReduce;
        g->rows = r;
        g->cols = c;
      } else {
        g->kind = GroupKind::kGeneralReduce;
      }
    } else if (IsFusibleOp(*n)) {
      g->kind  = GroupKind::kElementwise;
      g->numel = n->outputs[0]->numel();
    } else {
      g->kind = GroupKind::kLibraryCall;
    }
    group_of[n] = g.get();
    work.push_back(std::move(g));
  }

  auto successors = [&](WorkGroup* g) {
    std::set<WorkGroup*> out;
    for (Node* n : g->nodes)
      for (auto* o : n->outputs)
        for (Node* c : o->consumers)
          if (group_of.at(c) != g) out.insert(group_of.at(c));
    return out;
  };
  // is `to` reachable from `from` through at least one other group?
  auto has_indirect_path = [&](WorkGroup* from, WorkGroup* to) {
    std::set<WorkGroup*> visited;
    std::vector<WorkGroup*> stack;
    for (WorkGroup* s : successors(from))
      if (s != to) stack.push_back(s);
    int last_to = to->nodes.back()->index;
    while (!stack.empty()) {
      WorkGroup* g = stack.back();
      stack.pop_back();
      if (g == to) return true;
      if (!visited.insert(g).second) continue;
      // a group whose nodes all come after the last node of `to` cannot lead back to it
      if (g->nodes.front()->index > last_to) continue;
      for (WorkGroup* s : successors(g)) stack.push_back(s);
    }
    return false;
  };

  // one template must be able to hold the union
  auto merged_shape = [&](WorkGroup* p, WorkGroup* c, WorkGroup* out) -> bool {
    auto fusible_kind = [](GroupKind k) { return k == GroupKind::kElementwise || k == GroupKind::kRowReduce; };
    if (!fusible_kind(p->kind) || !fusible_kind(c->kind)) return false;
    // pre-run nodes execute once, ahead of everything else: they only fuse among themselves
    if (p->pre_run != c->pre_run) return false;
    std::vector<Node*> nodes = p->nodes;
    nodes.insert(nodes.end(), c->nodes.begin(), c->nodes.end());
    std::sort(nodes.begin(), nodes.end(), [](Node* a, Node* b) { return a->index < b->index; });
    out->nodes = nodes;
    if (p->kind == GroupKind::kElementwise && c->kind == GroupKind::kElementwise) {
      if (p->numel != c->numel) return false;
      out->kind  = GroupKind::kElementwise;
      out->numel = p->numel;
      return true;
    }
    int64_t rows = p->kind == GroupKind::kRowReduce ? p->rows : c->rows;
    int64_t cols = p->kind == GroupKind::kRowReduce ? p->cols : c->cols;
    if (p->kind == GroupKind::kRowReduce && c->kind == GroupKind::kRowReduce && (p->rows != c->rows || p->cols != c->cols))
      return false;
    if (!ClassifyRowReduceGroup(nodes, rows, cols, nullptr)) return false;
    out->kind = GroupKind::kRowReduce;
    out->rows = rows;
    out->cols = cols;
    return true;
  };

  // merge producer groups into consumer groups until nothing changes
  bool changed = true;
  while (changed) {
    changed = false;
    for (auto& np : nodes_) {
      Node* n = np.get();
      for (auto* in : n->inputs) {
        if (!in->producer) continue;
        WorkGroup* p = group_of.at(in->producer);
        WorkGroup* c = group_of.at(n);
        if (p == c) continue;
        WorkGroup merged;
        if (!merged_shape(p, c, &merged)) continue;
        if (has_indirect_path(p, c)) continue;
        // p absorbs c
        p->kind  = merged.kind;
        p->nodes = merged.nodes;
        p->numel = merged.numel;
        p->rows  = merged.rows;
        p->cols  = merged.cols;
        for (Node* m : c->nodes) group_of[m] = p;
        c->nodes.clear();
        changed = true;
      }
    }
  }

  // horizontal fusion: sibling groups over a shared input.  `reaches(a, b)`: b depends on a, directly or not.
  auto reaches = [&](WorkGroup* from, WorkGroup* to) {
    std::set<WorkGroup*> visited;
    std::vector<WorkGroup*> stack;
    for (WorkGroup* s : successors(from)) stack.push_back(s);
    while (!stack.empty()) {
      WorkGroup* g = stack.back();
      stack.pop_back();
      if (g == to) return true;
      if (!visited.insert(g).second) continue;
      for (WorkGroup* s : successors(g)) stack.push_back(s);
    }
    return false;
  };
  auto group_inputs = [&](WorkGroup* g) {
    std::set<const NodeData*> produced, ins;
    for (Node* n : g->nodes)
      for (auto* o : n->outputs) produced.insert(o);
    for (Node* n : g->nodes)
      for (auto* in : n->inputs)
        if (!produced.count(in)) ins.insert(in);
    return ins;
  };
  // FLAGS_cinn_hip_horizontal_fusion=0 keeps sibling groups apart (one kernel each, the shared value read by each)
  const char* horizontal_flag = getenv("FLAGS_cinn_hip_horizontal_fusion");
  changed                     = !(horizontal_flag && horizontal_flag[0] == '0');
  while (changed) {
    changed = false;
    std::vector<WorkGroup*> live;
    for (auto& g : work)
      if (!g->nodes.empty() && (g->kind == GroupKind::kElementwise || g->kind == GroupKind::kRowReduce)) live.push_back(g.get());
    for (size_t i = 0; i < live.size() && !changed; ++i) {
      const auto ins_a = group_inputs(live[i]);
      for (size_t j = i + 1; j < live.size() && !changed; ++j) {
        WorkGroup *a = live[i], *b = live[j];
        if (a->kind != b->kind) continue;  // an element-wise group next to a row group gains nothing from the row's phases
        bool shared = false;
        for (const NodeData* in : group_inputs(b))
          // the shared value must be one both kernels stream (the whole space), not a per-row or scalar operand
          if (ins_a.count(in) && in->numel() == (a->kind == GroupKind::kRowReduce ? a->rows * a->cols : a->numel)) shared = true;
        if (!shared) continue;
        WorkGroup merged;
        if (!merged_shape(a, b, &merged)) continue;
        if (reaches(a, b) || reaches(b, a)) continue;
        a->kind  = merged.kind;
        a->nodes = merged.nodes;
        a->numel = merged.numel;
        a->rows  = merged.rows;
        a->cols  = merged.cols;
        for (Node* m : b->nodes) group_of[m] = a;
        b->nodes.clear();
        changed = true;
      }
    }
  }

  // execution order: topological order of the group graph (Kahn), ties by first node
  std::vector<WorkGroup*> alive;
  for (auto& g : work)
    if (!g->nodes.empty()) alive.push_back(g.get());
  std::map<WorkGroup*, int> pending;
  for (WorkGroup* g : alive) pending[g] = 0;
  for (WorkGroup* g : alive)
    for (WorkGroup* s : successors(g)) pending[s]++;
  auto by_first = [](WorkGroup* a, WorkGroup* b) { return a->nodes.front()->index < b->nodes.front()->index; };
  std::vector<WorkGroup*> ready, ordered;
  for (WorkGroup* g : alive)
    if (pending[g] == 0) ready.push_back(g);
  while (!ready.empty()) {
    std::sort(ready.begin(), ready.end(), by_first);
    WorkGroup* g = ready.front();
    ready.erase(ready.begin());
    ordered.push_back(g);
    for (WorkGroup* s : successors(g))
      if (--pending[s] == 0) ready.push_back(s);
  }
  CINN_CHECK_EQ(ordered.size(), alive.size()) << "fusion produced a cyclic group graph";

  int gid = 0;
  for (WorkGroup* w : ordered) {
    auto g   = std::make_unique<Group>();
    g->id    = gid++;
    g->kind  = w->kind;
    g->nodes = w->nodes;
    g->rows  = w->rows;
    g->cols  = w->cols;
    g->pre_run = w->pre_run;
    std::map<NodeData*, bool> produced;
    for (Node* n : g->nodes) {
      n->group_id = g->id;
      for (auto* o : n->outputs) produced[o] = true;
    }
    for (Node* n : g->nodes) {
      for (auto* in : n->inputs) {
        // a library call takes its operands by position: the same value may be passed twice (a residual that is
        // also the convolution's input); generated kernels take every value once
        bool by_position = g->kind == GroupKind::kLibraryCall;
        if (!produced.count(in) && (by_position || std::find(g->inputs.begin(), g->inputs.end(), in) == g->inputs.end()))
          g->inputs.push_back(in);
      }
      for (auto* o : n->outputs) {
        bool external = o->is_fetch;
        for (Node* c : o->consumers) external |= (group_of.at(c) != w);
        if (o->consumers.empty()) external = true;
        if (external) g->outputs.push_back(o);
      }
    }
    std::string base = g->nodes.back()->op_type();
    g->func_name     = "fn_" + (name_.empty() ? std::string() : name_ + "_") + base + "_" + std::to_string(g->id);
    groups.push_back(std::move(g));
  }
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
