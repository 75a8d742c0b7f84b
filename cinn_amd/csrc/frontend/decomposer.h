// Program pass that rewrites composite operators into the primitives the backend fuses.  It covers
// the two decompositions the GPU configs need:
//   softmax     cinn/frontend/decomposer/activation.cc:70-118 (mode "fast": exp(x) / sum(exp(x));
//               any other mode subtracts the row maximum first)
//   batch_norm  inference form with the operation order of pe::BatchNorm_NCHW
//               (cinn/hlir/pe/nn.cc:700-721): (x - mean) * scale / sqrt(variance + eps) + bias
#pragma once
#include <map>

#include "frontend/syntax.h"

namespace cinn {
namespace frontend {

// Returns the rewritten program.  Output variables of rewritten instructions keep their ids.
Program ApplyDecomposer(const Program& program);

}  // namespace frontend
}  // namespace cinn
