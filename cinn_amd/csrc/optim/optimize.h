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

// Temporaries of a kernel (GPUShared / GPULocal buffers) written by a schedule as slices of a full-size tensor get the
// shape of what one block / one thread really touches (cinn/optim/transform_gpu_forloop.cc, OptimizeExprGPU: 257-342
// UpdateBufferAxisPass, 376-478 SharedAxisVisitor / LocalAxisVisitor, 562-608 ReplaceVarToZero).  Works on loops that
// still carry their GPU bindings, i.e. before TransformGpuForloops; indices are flat here, so "dropping an axis" is
// substituting 0 for its loop variable:
//   * a GPULocal buffer is private to a thread: the variables of every loop bound to a block or thread axis that
//     encloses an access, and of every loop that encloses ALL accesses of the buffer, become 0 in its indices;
//   * a GPUShared buffer is private to a block: the same for loops bound to a block axis and for the serial loops that
//     enclose all of its accesses; loops bound to a thread axis stay, they distinguish the block's threads;
//   * in every index, the variable of a loop with extent 1 becomes the loop's first value.
ir::Expr UpdateBufferAxes(const ir::Expr& body);

// Shrinks the temporaries of `func` to the largest index its accesses can reach plus one (the reference's
// ResizeBufferSizeVisitor, transform_gpu_forloop.cc:480-560, which enumerates every combination of loop values; here
// the bound comes from interval arithmetic over the enclosing loops, so it may be larger than the exact maximum, never
// smaller).  A buffer is never enlarged, and one with an access whose bound is unknown (a loop extent that is not a
// constant, a variable that is no loop variable) keeps its size.  Run after UpdateBufferAxes, before binding.
void ResizeBuffersToMaxVarRange(ir::LoweredFunc* func);

// The driver: map extern calls, vectorize, drop the axes a temporary does not need and shrink it, bind, free barriers
// from their guards, and record launch dimensions into func->axis_info.
void OptimizeFuncGPU(ir::LoweredFunc* func);

}  // namespace optim
}  // namespace cinn
