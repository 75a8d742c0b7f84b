// SplitReductions: rewrites reductions over non-trailing axes into chains the GPU templates run at memory speed.
//
//   * A reduction whose reduced axes form several runs (e.g. N, H, W of an NCHW tensor) becomes one reduction per
//     run, the last run first: the trailing run goes to the row-reduce template, every other run is a
//     reduce_run_<kind> op (input viewed as [a][r][c], r reduced; see the op registry).
//   * A run whose a x c output gives the column-reduce kernel too few blocks to fill the chip is reduced in two
//     steps: `parts` slices of r first ([a][parts][r / parts][c] -> [a][parts][c]), then the parts.
//   * 16-bit floating sums and products keep their partial results in fp32 and round once, at the last step.
// Reductions over trailing axes only (softmax, layer_norm, ...) are left alone.  The reference does the same for
// its block-reduce schedules in cinn/hlir/pass/reduce_split_pass.cc.
#pragma once
#include "frontend/syntax.h"

namespace cinn {
namespace frontend {

Program SplitReductions(const Program& program, int num_compute_units);

}  // namespace frontend
}  // namespace cinn
