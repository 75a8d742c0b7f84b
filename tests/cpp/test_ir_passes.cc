// The GPU IR passes on hand-built loop nests, checked through the printed IR and the recorded launch dimensions.
// What each pass has to do is fixed by the reference: cinn/optim/map_extern_call.cc:45-115,
// cinn/optim/transform_gpu_forloop.cc:53-171 and 628-661, cinn/optim/vectorize_loops.cc:60-307.
#include <cstdio>
#include <cstdlib>
#include <string>

#include "common/target.h"
#include "common/type.h"
#include "ir/ir.h"
#include "optim/optimize.h"

using namespace cinn;      // NOLINT
using namespace cinn::ir;  // NOLINT

static int failures = 0;
#define EXPECT(cond)                                                  \
  do {                                                                \
    if (!(cond)) {                                                    \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
      ++failures;                                                     \
    }                                                                 \
  } while (0)

static bool Has(const std::string& text, const std::string& what) { return text.find(what) != std::string::npos; }

static void TestMapExternCall() {
  const common::Type f32 = common::Float(32), f16 = common::Float(16), i32 = common::Int(32), b = common::Bool();
  Expr x = MakeVar("x", f32), h = MakeVar("h", f16), n = MakeVar("n", i32);
  const auto& gpu = common::DefaultAMDGPUTarget();
  // the type of the first argument picks the function; nested calls are mapped inside out
  Expr e = MakeCall(f32, "exp", {MakeCall(f32, "tanh", {x})});
  std::string s = ToString(optim::MapExternCall(e, gpu));
  EXPECT(Has(s, "cinn_hip_exp_fp32(cinn_hip_tanh_fp32(x))"));
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(f16, "sigmoid", {h}), gpu)), "cinn_hip_sigmoid_fp16(h)"));
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(b, "isnan", {x}), gpu)), "cinn_hip_isnan_fp32(x)"));
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(i32, "left_shift", {n, MakeIntImm(i32, 3)}), gpu)), "cinn_hip_left_shift_int32(n, 3)"));
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(i32, "popc", {n}), gpu)), "cinn_hip_popc_int32(n)"));
  // pow with the constants 0.5 and -0.5 (map_extern_call.cc:95-110); any other exponent stays a pow
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(f32, "pow", {x, MakeFloatImm(f32, 0.5)}), gpu)), "cinn_hip_sqrt_fp32(x)"));
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(f32, "pow", {x, MakeFloatImm(f32, -0.5)}), gpu)), "cinn_hip_rsqrt_fp32(x)"));
  s = ToString(optim::MapExternCall(MakeCall(f32, "pow", {x, MakeFloatImm(f32, 2.0)}), gpu));
  EXPECT(Has(s, "cinn_hip_pow_fp32(x, "));
  // names outside the tables, calls without arguments, and other targets: untouched
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(f32, "cinn_hip_block_reduce_sum_fp32_internal", {x}), gpu)), "cinn_hip_block_reduce_sum_fp32_internal(x)"));
  EXPECT(ToString(optim::MapExternCall(MakeCall(common::Type(), "__syncthreads", {}), gpu)) == ToString(MakeCall(common::Type(), "__syncthreads", {})));
  EXPECT(Has(ToString(optim::MapExternCall(MakeCall(f32, "exp", {x}), common::DefaultHostTarget())), "exp(x)"));
  EXPECT(!Has(ToString(optim::MapExternCall(MakeCall(f32, "exp", {x}), common::DefaultHostTarget())), "cinn_hip"));
}

static void TestSyncThreadsDropIfThenElse() {
  const common::Type i32 = common::Int(32);
  Expr tid  = MakeVar("threadIdx.x", i32);
  Expr sync = MakeCall(common::Type(), "__syncthreads", {});
  BufferRef out = MakeBuffer("out", common::Float(32), MemoryType::Global, 64);
  Expr store = MakeStore(out, MakeFloatImm(common::Float(32), 1.0), tid);
  // `if (tid == 0) __syncthreads();` between two stores: the barrier loses its guard, the guarded store keeps its own
  Expr body = MakeBlock({store, MakeIf(tid == Expr(0), MakeBlock({sync})), MakeIf(tid == Expr(0), store)});
  std::string before = ToString(body), after = ToString(optim::SyncThreadsDropIfThenElse(body));
  auto count = [](const std::string& s, const std::string& w) { int c = 0; for (size_t p = 0; (p = s.find(w, p)) != std::string::npos; p += w.size()) ++c; return c; };
  EXPECT(count(before, "if (") == 2 && count(after, "if (") == 1);
  EXPECT(count(after, "__syncthreads") == 1);
  // a barrier under any other condition is left for the author to fix
  Expr other = MakeIf(tid < Expr(4), sync);
  EXPECT(count(ToString(optim::SyncThreadsDropIfThenElse(other)), "if (") == 1);
}

static void TestBindAndVectorize() {
  const common::Type i32 = common::Int(32), f32 = common::Float(32);
  BufferRef a = MakeBuffer("a", f32, MemoryType::Global, 4096), o = MakeBuffer("o", f32, MemoryType::Global, 4096);
  Expr bx = MakeVar("bx", i32), tx = MakeVar("tx", i32), v = MakeVar("v", i32), t2 = MakeVar("t2", i32);
  Expr base = (bx * Expr(64) + tx) * Expr(4);
  Expr copy = MakeFor(v, Expr(0), Expr(4), ForType::Vectorized, MakeStore(o, MakeLoad(a, base + v), base + v));
  BindInfo bind_t{ForType::GPUThread, 0}, bind_b{ForType::GPUBlock, 0};
  // a second loop bound to threadIdx.x with a smaller extent gets a guard; a math call inside it is mapped
  Expr tail = MakeFor(t2, Expr(0), Expr(16), ForType::GPUThread,
                      MakeStore(o, MakeCall(f32, "exp", {MakeLoad(a, t2)}), t2), bind_t);
  auto func  = std::make_shared<LoweredFunc>();
  func->name = "k";
  func->body = MakeFor(bx, Expr(0), Expr(16), ForType::GPUBlock,
                       MakeBlock({MakeFor(tx, Expr(0), Expr(64), ForType::GPUThread, copy, bind_t), tail}), bind_b);
  optim::OptimizeFuncGPU(func.get());
  std::string s = ToString(func->body);
  EXPECT(func->axis_info.valid && func->axis_info.grid[0] == 16 && func->axis_info.block[0] == 64 && func->axis_info.block[1] == 1);
  EXPECT(!Has(s, "for ("));
  EXPECT(Has(s, "blockIdx.x") && Has(s, "threadIdx.x"));
  EXPECT(Has(s, "if ((threadIdx.x < 16))") || Has(s, "if (threadIdx.x < 16)"));
  EXPECT(Has(s, "cinn_hip_exp_fp32("));
  if (failures) std::printf("%s\n", s.c_str());
}

int main() {
  TestMapExternCall();
  TestSyncThreadsDropIfThenElse();
  TestBindAndVectorize();
  if (failures) return 1;
  std::printf("ok\n");
  return 0;
}
