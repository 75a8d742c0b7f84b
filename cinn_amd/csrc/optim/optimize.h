// IR passes that turn a scheduled loop nest into a kernel body.  They cover, for the gfx950 backend,
// what the reference does in cinn/optim/transform_gpu_forloop.cc (bound loops -> blockIdx/threadIdx,
// 53-171 and 628-661), ir::SetCudaAxisInfo (cinn/ir/ir_schedule_util.cc:74-108) and the CUDA part of
// cinn/optim/vectorize_loops.cc (60-307), and cinn/optim/map_extern_call.cc (45-115).
#pragma once
#include "common/target.h"
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

// Calls of the target-independent math names (cinn/optim/map_extern_call.cc:25-40: exp, erf, sigmoid, ..., pow, mod
// on floating-point operands; left_shift, bitwise_*, clz, popc, pow, mod on integers) become calls of the device
// library's function for the type of the first argument, cinn_hip_<name>_<type> on this backend (the reference
// spells them cinn_nvgpu_<name>_<type>; the library defines both).  pow(x, 0.5) and pow(x, -0.5) become sqrt(x) and
// rsqrt(x) first, as in the reference (map_extern_call.cc:95-110).  Calls without arguments (__syncthreads) and
// names outside the two tables are left alone; on other targets nothing changes.
ir::Expr MapExternCall(const ir::Expr& body, const common::Target& target);

// `if (x == 0) { __syncthreads(); }` becomes `__syncthreads();`: a barrier that only some threads of a block reach
// never completes (cinn/optim/transform_gpu_forloop.cc:628-661).
ir::Expr SyncThreadsDropIfThenElse(const ir::Expr& body);

// The driver: map extern calls, vectorize, bind, free barriers from their guards, and record launch dimensions into
// func->axis_info.
void OptimizeFuncGPU(ir::LoweredFunc* func);

}  // namespace optim
}  // namespace cinn
