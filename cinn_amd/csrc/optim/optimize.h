// IR passes that turn a scheduled loop nest into a kernel body.  They cover, for the gfx950 backend,
// what the reference does in cinn/optim/transform_gpu_forloop.cc (bound loops -> blockIdx/threadIdx,
// 53-171 and 628-661), ir::SetCudaAxisInfo (cinn/ir/ir_schedule_util.cc:74-108) and the CUDA part of
// cinn/optim/vectorize_loops.cc (60-307).
#pragma once
#include "ir/ir.h"

namespace cinn {
namespace optim {

// Loops marked ForType::Vectorized whose body is a single element copy `dst[a + v] = src[b + v]`
// become one vector copy of `extent` lanes (at most 16 bytes).  Loops that do not match stay as
// unrolled scalar loops.
ir::Expr VectorizeLoops(const ir::Expr& body);

// Loops bound to a GPU axis disappear: the loop variable is replaced by blockIdx.* / threadIdx.* and
// the extent is recorded as the launch dimension of that axis.  When two loops bound to the same
// axis have different extents the launch uses the larger one and the smaller loop body is guarded
// with `if (axis < extent)`.
ir::Expr TransformGpuForloops(const ir::Expr& body, ir::GpuAxisInfo* axis_info);

// The driver: vectorize, bind, and record launch dimensions into func->axis_info.
void OptimizeFuncGPU(ir::LoweredFunc* func);

}  // namespace optim
}  // namespace cinn
