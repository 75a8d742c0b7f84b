// Several generated kernels in one launch.
//
// A launch on this GPU costs about 3.3 us from kernel to kernel before the first byte moves, and a cold kernel needs
// another 1.5 - 2 us until its first loads return; a fused group that streams 33 MB (4 us of HBM time) spends more
// time starting and draining than streaming.  Groups that do not depend on each other need no ordering between them,
// so consecutive independent kernels of a program are emitted as ONE kernel whose blocks are handed out member by
// member: blocks [0, g0) run the first member's body, [g0, g0 + g1) the second's, and so on.  The chip never drains
// between members; the launch cost and the cold start are paid once.  This extends the horizontal fusion of the
// reference (cinn/hlir/pass/fusion_merge_pass.cc:176-260, sibling groups of one producer) to groups that share
// nothing: there the gain is one read of the shared value, here it is the launch.
#pragma once
#include <string>
#include <vector>

#include "hlir/graph.h"
#include "ir/ir.h"

namespace cinn {
namespace hlir {
namespace framework {

// one instruction of the compiled program: a group's function, or several groups' kernels merged into one
struct LaunchUnit {
  std::string func_name;
  std::vector<NodeData*> inputs, outputs;  // kernel parameter order: inputs, then outputs
  bool pre_run{false};
  std::vector<const Group*> members;
};

struct KernelMergeOptions {
  bool enabled{true};
  int max_members{8};
};

// `funcs[i]` is the lowered function of `groups[i]` (device functions already passed through OptimizeFuncGPU);
// `barrier[i]` marks groups that end a run whatever they are (e.g. groups that become views).  Returns the program's
// instructions in order; merged kernels are appended to `funcs_out`, members of a merged kernel are left out of it.
std::vector<LaunchUnit> MergeIndependentKernels(const std::vector<std::unique_ptr<Group>>& groups,
                                                const std::vector<ir::LoweredFuncRef>& funcs, const std::vector<bool>& barrier,
                                                const KernelMergeOptions& options, std::vector<ir::LoweredFuncRef>* funcs_out);

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
