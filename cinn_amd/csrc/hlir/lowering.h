// Lowering of one fusion group to one LoweredFunc for gfx950.  This is the GPU-schedule side of the
// backend: it decides the launch shape and the loop structure the reference derives in
// OpLowerer::IRSchedule (cinn/hlir/framework/op_lowering.cc:516-658) with the schedules of
// cinn/hlir/pe/ir_schedule_pe.cc and the reduce loop assignment of
// cinn/hlir/framework/op_lowering_util.cc:485-1177 - re-designed for 64-lane wavefronts:
//   * element-wise groups: one flat space, 128-bit accesses, 256-thread blocks;
//   * row-reduce groups (reductions over the trailing axes plus everything fused around them):
//     one wavefront - or, for long rows, one block - owns a row, keeps it in registers across all
//     reductions and writes every output once, so the group reads and writes each tensor exactly
//     once whatever the number of reductions in it;
//   * other reductions: one thread per output element, serial over the reduced axes;
//   * kNonFusible ops: a host function holding one call to a runtime intrinsic, as
//     cinn/hlir/op/custom_call.cc:70-217 builds them.
#pragma once
#include <string>

#include "hlir/graph.h"
#include "ir/ir.h"

namespace cinn {
namespace hlir {
namespace framework {

struct LoweringOptions {
  // longest row (in elements per thread) that is kept in registers by the row-reduce template
  int max_cached_elems_per_thread{64};
  // elements per lane above which a row is given to a whole block instead of one wavefront
  int wave_row_elems_per_lane{64};
  // elements per thread a block-per-row team aims for (the team is the smallest power of two of at
  // least 128 threads that gets at or below this)
  int block_row_elems_per_thread{16};
  // outputs of at least this many bytes are written with non-temporal stores (0 disables): a large
  // streamed output would otherwise evict the input rows still to be read from the last-level cache
  int64_t nontemporal_store_bytes{8 << 20};
  // inputs of at least this many bytes are read with non-temporal loads (0 disables)
  int64_t nontemporal_load_bytes{0};
  // threads of an element-wise block
  int elementwise_block{256};
  // waves (rows) per block when one wavefront owns a row
  int rows_per_block{4};
  // rows one wavefront works through (unrolled, so their loads overlap).  Measured on MI355X this does
  // not pay for the BASELINE shapes (1 is the best setting for every one of them), so it stays a knob.
  int rows_per_wave{1};
  // the same for a row-reduce group that becomes a member of a merged launch (hlir/kernel_merge.h) and requests at
  // most 32 bytes per lane and row: there the heaviest member's registers set the occupancy of all, and such rows need
  // two per wavefront to keep as many bytes in flight as their own kernel has (configs[1] step: 64.5 -> 62.5 us;
  // four rows, or two rows of 64 bytes per lane, measured slower).  1 switches it off.
  int merged_rows_per_wave{2};
  // reductions over one non-trailing run of axes use the column-reduce kernel (off: one thread per output element)
  bool column_reduce{true};
  // element-wise groups around a transpose that moves the innermost axis stage the input through LDS tiles
  bool tiled_transpose{true};
  // rows of at most 32 vectors are given to teams of 1 .. 32 lanes, several rows per wavefront
  bool sub_wave_rows{true};
  static LoweringOptions FromEnv();
};

class OpLowerer {
 public:
  OpLowerer(const common::Target& target, const LoweringOptions& options = LoweringOptions::FromEnv());
  // One function per group.  Device functions come back scheduled, with loops still carrying their
  // GPU bindings (optim::OptimizeFuncGPU turns them into a kernel body and launch dimensions).
  // merged_member: the group's kernel will share a launch with others (see merged_rows_per_wave)
  ir::LoweredFuncRef Lower(const Group& group, bool merged_member = false) const;
  // argument order of the function generated for `group`: inputs, then outputs
  static std::vector<NodeData*> ArgumentsOf(const Group& group);

 private:
  ir::LoweredFuncRef LowerElementwise(const Group& group) const;
  ir::LoweredFuncRef LowerRowReduce(const Group& group, bool merged_member) const;
  ir::LoweredFuncRef LowerGeneralReduce(const Group& group) const;
  ir::LoweredFuncRef LowerLibraryCall(const Group& group) const;
  common::Target target_;
  LoweringOptions options_;
};

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
