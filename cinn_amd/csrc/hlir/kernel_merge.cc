#include "hlir/kernel_merge.h"

#include <algorithm>
#include <cstdlib>
#include <map>
#include <set>

#include "ir/ir_mutator.h"

namespace cinn {
namespace hlir {
namespace framework {

namespace {

using ir::Expr;

// a kernel whose body only knows its own blockIdx.x: one grid axis, every argument a buffer, no use of the grid size
bool Mergeable(const ir::LoweredFunc& f) {
  if (!f.is_device || !f.axis_info.valid) return false;
  if (f.axis_info.grid[1] != 1 || f.axis_info.grid[2] != 1) return false;
  for (auto& a : f.args)
    if (!a.is_buffer()) return false;
  for (const char* v : {"gridDim.x", "gridDim.y", "gridDim.z", "blockIdx.y", "blockIdx.z"})
    if (ir::UsesVar(f.body, v)) return false;
  return true;
}

bool SameBlock(const ir::LoweredFunc& a, const ir::LoweredFunc& b) {
  for (int d = 0; d < 3; ++d)
    if (a.axis_info.block[d] != b.axis_info.block[d]) return false;
  return true;
}

// A block of bx x by threads whose body can run in a flat block of bx * by threads, with threadIdx.x and threadIdx.y
// recovered from the flat index: bx a power of two, no third axis, no use of the block's extents (the device library's
// wave and block reductions work on the linear thread index; the column reduction walks blockDim.y and is excluded
// by the group kinds that get here).
bool Flattenable(const Group& g, const ir::LoweredFunc& f) {
  if (g.kind != GroupKind::kElementwise && g.kind != GroupKind::kRowReduce) return false;
  const int bx = f.axis_info.block[0];
  if (f.axis_info.block[2] != 1 || bx <= 0 || (bx & (bx - 1)) != 0) return false;
  for (const char* v : {"blockDim.x", "blockDim.y", "blockDim.z", "threadIdx.z"})
    if (ir::UsesVar(f.body, v)) return false;
  return true;
}

int Threads(const ir::LoweredFunc& f) { return f.axis_info.block[0] * f.axis_info.block[1] * f.axis_info.block[2]; }

LaunchUnit UnitOf(const Group& g) {
  LaunchUnit u;
  u.func_name = g.func_name;
  u.inputs    = g.inputs;
  u.outputs   = g.outputs;
  u.pre_run   = g.pre_run;
  u.members   = {&g};
  return u;
}

}  // namespace

std::vector<LaunchUnit> MergeIndependentKernels(const std::vector<std::unique_ptr<Group>>& groups,
                                                const std::vector<ir::LoweredFuncRef>& funcs, const std::vector<bool>& barrier,
                                                const KernelMergeOptions& options, std::vector<ir::LoweredFuncRef>* funcs_out) {
  CINN_CHECK_EQ(groups.size(), funcs.size());
  std::vector<LaunchUnit> units;
  size_t i = 0;
  while (i < groups.size()) {
    const Group& first = *groups[i];
    if (!options.enabled || barrier[i] || !Mergeable(*funcs[i])) {
      units.push_back(UnitOf(first));
      funcs_out->push_back(funcs[i]);
      ++i;
      continue;
    }
    // the longest run of consecutive kernels none of which reads what an earlier one of the run writes; the run is
    // consecutive in execution order, so a dependence through other groups would pass through a member as well
    std::set<const NodeData*> written(first.outputs.begin(), first.outputs.end());
    int64_t blocks = funcs[i]->axis_info.grid[0];
    size_t end     = i + 1;
    // A run keeps one block shape, or - once a member of another shape joins - every member must be able to run in a
    // flat block of the same number of threads (a member that cannot, e.g. a column reduction, shares launches only
    // with kernels of its own shape).
    bool run_flat        = false;
    bool all_flattenable = Flattenable(first, *funcs[i]);
    while (end < groups.size() && static_cast<int>(end - i) < options.max_members) {
      const Group& g = *groups[end];
      if (barrier[end] || !Mergeable(*funcs[end]) || g.pre_run != first.pre_run) break;
      const bool same   = SameBlock(*funcs[i], *funcs[end]);
      const bool g_flat = Flattenable(g, *funcs[end]);
      if (run_flat || !same) {
        if (!all_flattenable || !g_flat || Threads(*funcs[i]) != Threads(*funcs[end])) break;
      }
      bool depends = false;
      for (auto* in : g.inputs) depends |= written.count(in) > 0;
      if (depends) break;
      if (blocks + funcs[end]->axis_info.grid[0] > 0x7fffffff) break;
      blocks += funcs[end]->axis_info.grid[0];
      written.insert(g.outputs.begin(), g.outputs.end());
      run_flat        = run_flat || !same;
      all_flattenable = all_flattenable && g_flat;
      ++end;
    }
    if (end - i < 2) {
      units.push_back(UnitOf(first));
      funcs_out->push_back(funcs[i]);
      ++i;
      continue;
    }
    // one kernel: parameters are the members' inputs (each value once) followed by their outputs
    LaunchUnit unit;
    unit.pre_run = first.pre_run;
    auto merged  = std::make_shared<ir::LoweredFunc>();
    merged->is_device = true;
    merged->axis_info = funcs[i]->axis_info;
    merged->axis_info.grid[0] = static_cast<int>(blocks);
    // members of different block shapes: the launch is a flat block and every member recovers its own threadIdx.x / y
    bool flat = false;
    for (size_t k = i + 1; k < end; ++k) flat = flat || !SameBlock(*funcs[i], *funcs[k]);
    if (flat) {
      merged->axis_info.block[0] = funcs[i]->axis_info.block[0] * funcs[i]->axis_info.block[1];
      merged->axis_info.block[1] = 1;
    }
    merged->name = first.func_name + "_and_" + std::to_string(end - i - 1) + "_more";
    std::map<std::string, ir::Argument> arg_of;  // by buffer name: the first member's buffer object is declared
    for (size_t k = i; k < end; ++k) {
      unit.members.push_back(groups[k].get());
      for (auto& a : funcs[k]->args) arg_of.emplace(a.buffer->name, a);
    }
    std::set<const NodeData*> seen;
    std::vector<ir::Argument> ins, outs;
    for (size_t k = i; k < end; ++k) {
      const Group& g = *groups[k];
      CINN_CHECK_EQ(funcs[k]->args.size(), g.inputs.size() + g.outputs.size());
      for (size_t a = 0; a < g.inputs.size(); ++a) {
        if (!seen.insert(g.inputs[a]).second) continue;
        unit.inputs.push_back(g.inputs[a]);
        ins.push_back(arg_of.at(funcs[k]->args[a].buffer->name));
        ins.back().io = ir::Argument::IO::kInput;
      }
      for (size_t a = 0; a < g.outputs.size(); ++a) {
        unit.outputs.push_back(g.outputs[a]);
        outs.push_back(funcs[k]->args[g.inputs.size() + a]);
        outs.back().io = ir::Argument::IO::kOutput;
      }
    }
    merged->args = ins;
    merged->args.insert(merged->args.end(), outs.begin(), outs.end());
    // bodies: block b of the launch is block b - start of the member whose range holds it.  Blocks are dispatched in
    // index order: the member with the most blocks comes first, so that the launch ends on short members
    // (measured on six members of 2048 - 4096 blocks: within 0.5 % of program order and of the reverse;
    // FLAGS_cinn_hip_merge_order = 0: program order, 2: fewest blocks first).
    std::vector<size_t> order;
    for (size_t k = i; k < end; ++k) order.push_back(k);
    static const int order_flag = [] {
      const char* v = getenv("FLAGS_cinn_hip_merge_order");
      return v && *v ? atoi(v) : 1;
    }();
    if (order_flag == 1 || order_flag == 2)
      std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) {
        return order_flag == 1 ? funcs[a]->axis_info.grid[0] > funcs[b]->axis_info.grid[0]
                               : funcs[a]->axis_info.grid[0] < funcs[b]->axis_info.grid[0];
      });
    Expr block_x = ir::MakeVar("blockIdx.x", common::Int(32));
    Expr chain;
    int64_t start = blocks;
    for (size_t pos = order.size(); pos-- > 0;) {
      const size_t k = order[pos];
      start -= funcs[k]->axis_info.grid[0];
      // temporaries are declared once at the top of the kernel: keep the members' names apart
      for (auto& buf : funcs[k]->temp_bufs) {
        buf->name = "m" + std::to_string(k - i) + "_" + buf->name;
        merged->temp_bufs.push_back(buf);
      }
      Expr body = start == 0 ? funcs[k]->body : ir::Substitute(funcs[k]->body, "blockIdx.x", block_x - Expr(static_cast<int>(start)));
      if (flat && funcs[k]->axis_info.block[1] > 1) {
        const int bx = funcs[k]->axis_info.block[0];
        int shift    = 0;
        while ((1 << shift) < bx) ++shift;
        const std::string tag = "m" + std::to_string(k - i);
        Expr tx = ir::MakeVar(tag + "_tx", common::Int(32)), ty = ir::MakeVar(tag + "_ty", common::Int(32));
        Expr tid = ir::MakeVar("threadIdx.x", common::Int(32));
        body = ir::Substitute(ir::Substitute(body, "threadIdx.x", tx), "threadIdx.y", ty);
        body = ir::MakeBlock({ir::MakeLet(tx, tid % Expr(bx)), ir::MakeLet(ty, tid / Expr(bx)), body});
      }
      if (!chain.defined()) {
        chain = ir::MakeBlock({body});  // the last member takes every remaining block
      } else {
        chain = ir::MakeIf(block_x < Expr(static_cast<int>(start + funcs[k]->axis_info.grid[0])), ir::MakeBlock({body}), chain);
      }
    }
    merged->body   = chain;
    unit.func_name = merged->name;
    funcs_out->push_back(merged);
    units.push_back(unit);
    i = end;
  }
  return units;
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
