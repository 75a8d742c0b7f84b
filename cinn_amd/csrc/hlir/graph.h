// Dataflow graph of a front-end Program plus its partition into fusion groups.  Mirrors the role of
// hlir::framework::Graph / Node / NodeData / Graph::Group (cinn/hlir/framework/graph.h) for the
// GPU path: one Group becomes one kernel (or one library call).
#pragma once
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "common/target.h"
#include "frontend/syntax.h"
#include "hlir/op.h"

namespace cinn {
namespace hlir {
namespace framework {

struct Node;

// a tensor value of the graph
struct NodeData {
  std::string id;
  ShapeType shape;
  common::Type dtype;
  Node* producer{nullptr};  // nullptr: fed input
  std::vector<Node*> consumers;
  bool is_fetch{false};
  // value that does not change between executions: a program input marked const (weights) or the result of an
  // operator whose inputs are all const (NodeData::is_const of cinn/hlir/framework/node.h)
  bool is_const{false};
  int64_t numel() const { return ShapeNumel(shape); }
};

struct Node {
  int index{0};  // position in topological order
  const Operator* op{nullptr};
  AttributeMap attrs;
  std::vector<NodeData*> inputs;
  std::vector<NodeData*> outputs;
  int group_id{-1};
  // all inputs are const: runs once in Program::PreRun instead of in every execution (the "pre_run" attribute of
  // cinn/hlir/pass/const_propagate.cc:33-58)
  bool pre_run{false};
  const std::string& op_type() const { return op->name; }
};

enum class GroupKind {
  kElementwise,  // injective chain over one flat iteration space
  kRowReduce,    // reductions over the trailing (contiguous) axes with fused producers and consumers
  kGeneralReduce,  // a single reduction over arbitrary axes, serial per output element
  kLibraryCall   // matmul / conv2d / pool2d and other kNonFusible ops
};

struct Group {
  int id{0};
  GroupKind kind{GroupKind::kElementwise};
  std::vector<Node*> nodes;           // topological order
  std::vector<NodeData*> inputs;      // values produced outside the group
  std::vector<NodeData*> outputs;     // values consumed outside the group or fetched
  // kRowReduce: rows x cols of the reduction space
  int64_t rows{0}, cols{0};
  bool pre_run{false};  // every node of the group is a pre-run node
  std::string func_name;
};

class Graph {
 public:
  Graph(const frontend::Program& program, const std::set<std::string>& fetch_ids, const common::Target& target);

  const common::Target& target() const { return target_; }
  const std::string& name() const { return name_; }
  const std::vector<std::unique_ptr<Node>>& nodes() const { return nodes_; }
  NodeData* FindVar(const std::string& id) const;
  const std::vector<NodeData*>& inputs() const { return inputs_; }
  std::vector<NodeData*> AllVars() const;

  // partition into fusion groups (hlir/fusion.cc); fills `groups`
  void BuildFusionGroups();
  std::vector<std::unique_ptr<Group>> groups;

  std::string DebugGroupString() const;

 private:
  NodeData* GetOrCreateVar(const frontend::Variable& v);
  void ConstPropagate();
  common::Target target_;
  std::string name_;
  std::vector<std::unique_ptr<Node>> nodes_;
  std::map<std::string, std::unique_ptr<NodeData>> vars_;
  std::vector<NodeData*> inputs_;
};

// ---- shape classification shared by the fusion pass and the reduce lowering ------------------------
// Splits a reduce over `dims` of `shape` into rows x cols when the reduced axes are the trailing
// ones (size-1 axes are ignored).  Returns false for any other axis set.
bool TrailingReduceSpace(const ShapeType& shape, const std::vector<int>& dims, int64_t* rows, int64_t* cols);
std::vector<int> ReduceDimsOf(const Node& node);
// a reduce_run_<kind> node (reduction of a [a, parts, r / parts, c] view, see the op registry)
bool IsReduceRun(const Node& node);

// how a value relates to the rows x cols space of a row-reduce group
enum class RowKind { kElem, kRow, kCol, kScalar, kInvalid };
// kind of broadcast_to's input given that its output is a kElem value of shape out_shape
RowKind ClassifyBroadcastInput(const ShapeType& in_shape, const ShapeType& out_shape, const std::vector<int>& axes,
                               int64_t rows, int64_t cols);

// Assigns a RowKind to every value the nodes (in topological order) touch, for a rows x cols
// row-reduce group.  Returns false when some node does not fit the pattern (then the nodes cannot
// share one row-resident kernel).
bool ClassifyRowReduceGroup(const std::vector<Node*>& nodes, int64_t rows, int64_t cols,
                            std::map<const NodeData*, RowKind>* kinds);

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
