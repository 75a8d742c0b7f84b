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

// A schedule writes its temporaries as slices of the full-size tensor: under a block loop i (16) and a thread loop j
// (64), a per-thread accumulator acc[i*64 + j] and a per-block staging tile[i*512 + j*8 + k].  One thread touches one
// element of acc, one block 512 of tile: the block / thread terms leave the indices and the buffers shrink
// (cinn/optim/transform_gpu_forloop.cc:257-560).  Global buffers keep their indices.
static void TestBufferAxesAndResize() {
  const common::Type i32 = common::Int(32), f32 = common::Float(32);
  BufferRef a = MakeBuffer("a", f32, MemoryType::Global, 8192), o = MakeBuffer("o", f32, MemoryType::Global, 1024);
  BufferRef acc = MakeBuffer("acc", f32, MemoryType::GPULocal, 1024), tile = MakeBuffer("tile", f32, MemoryType::GPUShared, 8192);
  Expr i = MakeVar("i", i32), j = MakeVar("j", i32), k = MakeVar("k", i32), k2 = MakeVar("k2", i32), u = MakeVar("u", i32);
  Expr lin = i * Expr(64) + j;
  Expr stage = MakeFor(k, Expr(0), Expr(8), ForType::Serial,
                       MakeStore(tile, MakeLoad(a, lin * Expr(8) + k), i * Expr(512) + j * Expr(8) + k));
  Expr init = MakeStore(acc, MakeFloatImm(f32, 0.0), lin);
  // a loop that runs once: u is its first value, 3
  Expr sum = MakeFor(u, Expr(3), Expr(1), ForType::Serial,
                     MakeFor(k2, Expr(0), Expr(8), ForType::Serial,
                             MakeStore(acc, MakeLoad(acc, lin) + MakeLoad(tile, i * Expr(512) + j * Expr(8) + k2) * MakeCast(f32, u), lin)));
  Expr out = MakeStore(o, MakeLoad(acc, lin), lin);
  BindInfo bind_t{ForType::GPUThread, 0}, bind_b{ForType::GPUBlock, 0};
  auto func  = std::make_shared<LoweredFunc>();
  func->name = "k";
  func->temp_bufs = {acc, tile};
  func->body = MakeFor(i, Expr(0), Expr(16), ForType::GPUBlock,
                       MakeFor(j, Expr(0), Expr(64), ForType::GPUThread, MakeBlock({stage, init, sum, out}), bind_t), bind_b);
  Expr axes = optim::UpdateBufferAxes(func->body);
  std::string s = ToString(axes);
  EXPECT(Has(s, "acc[0]") && !Has(s, "acc[(") && !Has(s, "acc[i") );
  EXPECT(Has(s, "tile[((j * 8) + k)]") && Has(s, "tile[((j * 8) + k2)]"));
  EXPECT(Has(s, "o[((i * 64) + j)]") && Has(s, "a[((((i * 64) + j) * 8) + k)]"));
  EXPECT(Has(s, "* 3.0f)") && !Has(s, "u)"));  // the loop over u stays as a scope, its variable is gone from the body
  if (failures) std::printf("%s\n", s.c_str());
  func->body = axes;
  optim::ResizeBuffersToMaxVarRange(func.get());
  EXPECT(acc->num_elements == 1);
  EXPECT(tile->num_elements == 512);

  // the driver does the same and binds: no loop variable of a bound loop is left in a temporary's index
  acc->num_elements = 1024, tile->num_elements = 8192;
  func->body = MakeFor(i, Expr(0), Expr(16), ForType::GPUBlock,
                       MakeFor(j, Expr(0), Expr(64), ForType::GPUThread, MakeBlock({stage, init, sum, out}), bind_t), bind_b);
  optim::OptimizeFuncGPU(func.get());
  s = ToString(func->body);
  EXPECT(Has(s, "acc[0]") && Has(s, "tile[((threadIdx.x * 8) + k)]") && Has(s, "o[((blockIdx.x * 64) + threadIdx.x)]"));
  EXPECT(acc->num_elements == 1 && tile->num_elements == 512);
  if (failures) std::printf("%s\n", s.c_str());

  // an index whose range is unknown (n is no loop variable) leaves the buffer alone; a buffer is never enlarged
  BufferRef small = MakeBuffer("small", f32, MemoryType::GPULocal, 4), odd = MakeBuffer("odd", f32, MemoryType::GPULocal, 64);
  Expr n = MakeVar("n", i32), q = MakeVar("q", i32);
  auto g  = std::make_shared<LoweredFunc>();
  g->name = "g";
  g->temp_bufs = {small, odd};
  g->body = MakeFor(q, Expr(0), Expr(8), ForType::Serial,
                    MakeBlock({MakeStore(small, MakeFloatImm(f32, 1.0), q % Expr(4)), MakeStore(odd, MakeFloatImm(f32, 1.0), q + n)}));
  optim::ResizeBuffersToMaxVarRange(g.get());
  EXPECT(small->num_elements == 4 && odd->num_elements == 64);
}

// What must stay as written: the passes only drop a variable when no two accesses that met in an element stop meeting
// and no value has to survive in the dropped direction.
static void TestBufferAxesKeepWhatIsNeeded() {
  const common::Type i32 = common::Int(32), f32 = common::Float(32);
  BufferRef a = MakeBuffer("a", f32, MemoryType::Global, 4096), o = MakeBuffer("o", f32, MemoryType::Global, 4096);
  Expr j = MakeVar("j", i32), ko = MakeVar("ko", i32), ki = MakeVar("ki", i32), k2 = MakeVar("k2", i32);
  BindInfo bind_t{ForType::GPUThread, 0};
  auto run = [&](Expr inner) { return ToString(optim::UpdateBufferAxes(MakeFor(j, Expr(0), Expr(64), ForType::GPUThread, inner, bind_t))); };

  // one slice per iteration of ko, filled and consumed inside it: the iterations share the slice
  BufferRef tmp = MakeBuffer("tmp", f32, MemoryType::GPULocal, 64 * 16 * 4);
  Expr at   = (j * Expr(16) + ko) * Expr(4);
  Expr fill = MakeFor(ki, Expr(0), Expr(4), ForType::Serial, MakeStore(tmp, MakeLoad(a, at + ki), at + ki));
  Expr use  = MakeFor(k2, Expr(0), Expr(4), ForType::Serial, MakeStore(o, MakeLoad(tmp, at + k2), at + k2));
  std::string s = run(MakeFor(ko, Expr(0), Expr(16), ForType::Serial, MakeBlock({fill, use})));
  EXPECT(Has(s, "tmp[ki] = ") && Has(s, "= tmp[k2]"));
  if (failures) std::printf("%s\n", s.c_str());

  // a slice that overlaps the next iteration's (step 2, four elements): ko stays, the thread's own offset goes
  Expr at2 = j * Expr(64) + ko * Expr(2);
  fill     = MakeFor(ki, Expr(0), Expr(4), ForType::Serial, MakeStore(tmp, MakeLoad(a, at + ki), at2 + ki));
  use      = MakeFor(k2, Expr(0), Expr(4), ForType::Serial, MakeStore(o, MakeLoad(tmp, at2 + k2), at + k2));
  s        = run(MakeFor(ko, Expr(0), Expr(16), ForType::Serial, MakeBlock({fill, use})));
  EXPECT(Has(s, "tmp[((ko * 2) + ki)] = ") && Has(s, "= tmp[((ko * 2) + k2)]"));
  if (failures) std::printf("%s\n", s.c_str());

  // two halves used in turn (this iteration writes one, reads the other): not a constant step, ko stays
  Expr half_w = (ko % Expr(2)) * Expr(4), half_r = ((ko + Expr(1)) % Expr(2)) * Expr(4);
  fill        = MakeFor(ki, Expr(0), Expr(4), ForType::Serial, MakeStore(tmp, MakeLoad(a, at + ki), half_w + ki));
  use         = MakeFor(k2, Expr(0), Expr(4), ForType::Serial, MakeStore(o, MakeLoad(tmp, half_r + k2), at + k2));
  s           = run(MakeFor(ko, Expr(0), Expr(16), ForType::Serial, MakeBlock({fill, use})));
  EXPECT(Has(s, "tmp[(((ko % 2) * 4) + ki)]") && Has(s, "tmp[((((ko + 1) % 2) * 4) + k2)]"));
  if (failures) std::printf("%s\n", s.c_str());

  // a block's shared buffer keeps the thread's offset and the serial loop: other threads read what this one wrote
  BufferRef sh = MakeBuffer("sh", f32, MemoryType::GPUShared, 64 * 16 * 4);
  fill         = MakeFor(ki, Expr(0), Expr(4), ForType::Serial, MakeStore(sh, MakeLoad(a, at + ki), at + ki));
  use          = MakeFor(k2, Expr(0), Expr(4), ForType::Serial, MakeStore(o, MakeLoad(sh, at + k2), at + k2));
  s            = run(MakeFor(ko, Expr(0), Expr(16), ForType::Serial, MakeBlock({fill, use})));
  EXPECT(Has(s, "sh[((((j * 16) + ko) * 4) + ki)] = "));
  if (failures) std::printf("%s\n", s.c_str());

  // a thread's buffer read with another thread's offset (the schedule's mistake or a rotation): steps differ, untouched
  BufferRef loc = MakeBuffer("loc", f32, MemoryType::GPULocal, 256);
  s = run(MakeBlock({MakeStore(loc, MakeLoad(a, j), j), MakeStore(o, MakeLoad(loc, j * Expr(2)), j)}));
  EXPECT(Has(s, "loc[j] = ") && Has(s, "loc[(j * 2)]"));
  if (failures) std::printf("%s\n", s.c_str());
}

int main() {
  TestMapExternCall();
  TestSyncThreadsDropIfThenElse();
  TestBindAndVectorize();
  TestBufferAxesAndResize();
  TestBufferAxesKeepWhatIsNeeded();
  if (failures) return 1;
  std::printf("ok\n");
  return 0;
}
