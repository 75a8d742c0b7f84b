// Scope / Tensor / Instruction / Program / GraphCompiler of the GPU path.  Interfaces follow
// cinn/hlir/framework/{scope.h,tensor.h,buffer.h,memory.cc,instruction.h,graph_compiler.h}:
//   * a Tensor owns a cinn_buffer_t whose `memory` is device memory obtained through the runtime's
//     allocator (role of CudaMemoryMng, memory.cc:43-64) - or, for the tensors of a compiled program, a
//     slice of the program's one device allocation (DeviceArena below), in which intermediates whose
//     lifetimes do not overlap share bytes;
//   * an Instruction holds the names of its arguments and a lower_func_ptr_g; Run() packs the
//     cinn_pod_value_t argument array once and calls the function (instruction.cc:77-138);
//   * Program::Execute runs the instructions in order on one stream and synchronises when no
//     stream was given (graph_compiler.cc:212-222);
//   * GraphCompiler::Build lowers every fusion group, builds one module and creates the
//     instructions (graph_compiler.cc:745-792).
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "backends/compiler.h"
#include "cinn_hip_runtime.h"
#include "hlir/graph.h"
#include "hlir/kernel_merge.h"
#include "hlir/lowering.h"

namespace cinn {
namespace hlir {
namespace framework {

// One device allocation that holds every tensor of a compiled program (GraphCompiler::Build plans it): a few large
// pages instead of one allocation per variable, and intermediates placed by lifetime so that a program's working set
// is the largest set of values alive at once, not the sum of all of them.  Freed when the last tensor placed in it
// and the scope that made it are gone.
class DeviceArena {
 public:
  explicit DeviceArena(size_t bytes);
  ~DeviceArena();
  DeviceArena(const DeviceArena&) = delete;
  char* base() const { return base_; }
  size_t bytes() const { return bytes_; }

 private:
  char* base_{nullptr};
  size_t bytes_{0};
};

class _Tensor_ {
 public:
  _Tensor_();
  ~_Tensor_();
  _Tensor_(const _Tensor_&) = delete;

  void Resize(const ShapeType& shape);
  const ShapeType& shape() const { return shape_; }
  const common::Type& type() const { return type_; }
  void set_type(const common::Type& t);
  int64_t numel() const { return ShapeNumel(shape_); }
  size_t bytes() const { return static_cast<size_t>(numel()) * type_.bytes(); }

  // device pointer; allocates on first use
  void* mutable_data(const common::Target& target);
  // This tensor becomes another view (its own shape, the same number of bytes) of `source`'s device memory: no
  // allocation of its own, `source` stays the owner.  What a reshape of a dense row-major tensor is.
  void ShareBufferWith(const std::shared_ptr<_Tensor_>& source);
  bool is_view() const { return source_ != nullptr; }
  const std::shared_ptr<_Tensor_>& source() const { return source_; }
  // This tensor lives at `offset` of `arena` from now on (capacity bytes are its own while it is alive; a tensor that
  // is later resized beyond them goes back to an allocation of its own).  transient: other tensors of the program
  // occupy the same bytes before its producer and after its last consumer have run, so its contents mean something
  // only in between - reading or writing it from the host by name is refused.
  void PlaceIn(std::shared_ptr<DeviceArena> arena, size_t offset, size_t capacity, bool transient);
  bool is_transient() const { return arena_ && transient_; }
  bool in_arena() const { return arena_ != nullptr; }
  void* data() const { return source_ ? source_->data() : buffer_.memory; }
  cinn_buffer_t* buffer() { return &buffer_; }

  // synchronous copies between host memory and the device buffer
  void CopyFromHost(const void* src, size_t bytes, const common::Target& target);
  void CopyToHost(void* dst, size_t bytes) const;

 private:
  void Free();
  ShapeType shape_;
  common::Type type_{common::Float(32)};
  cinn_buffer_t buffer_;
  size_t allocated_{0};
  std::shared_ptr<_Tensor_> source_;  // set by ShareBufferWith
  std::shared_ptr<DeviceArena> arena_;  // set by PlaceIn
  size_t arena_offset_{0}, arena_capacity_{0};
  bool transient_{false};
};
using Tensor = std::shared_ptr<_Tensor_>;

class Scope {
 public:
  static std::shared_ptr<Scope> Create() { return std::make_shared<Scope>(); }
  // creates the tensor when it does not exist
  Tensor Var(const std::string& name);
  Tensor FindVar(const std::string& name) const;
  Tensor GetTensor(const std::string& name) const;
  std::vector<std::string> var_names() const;

 private:
  std::map<std::string, Tensor> data_;
};

class Instruction {
 public:
  Instruction(const common::Target& target, Scope* scope, std::vector<std::string> in_args,
              std::vector<std::string> out_args, std::string function_name)
      : target_(target), scope_(scope), in_args_(std::move(in_args)), out_args_(std::move(out_args)),
        function_name_(std::move(function_name)) {}

  void SetLoweredFunc(void* fn) { fn_ = reinterpret_cast<lower_func_ptr_g>(fn); }
  void Run(void* stream = nullptr);
  const std::string& function_name() const { return function_name_; }
  const std::vector<std::string>& in_args() const { return in_args_; }
  const std::vector<std::string>& out_args() const { return out_args_; }
  // device addresses of the input / output tensors (allocates them if need be): what two instructions must not share
  // to run side by side
  std::vector<const void*> ArgAddresses(bool outputs) const;
  // runs once ahead of the first execution instead of in every one (cinn/hlir/framework/instruction.h:129)
  bool pre_run{false};

 private:
  void UpdateArgsCache();
  void CheckResults();
  common::Target target_;
  Scope* scope_;
  std::vector<std::string> in_args_, out_args_;
  std::string function_name_;
  lower_func_ptr_g fn_{nullptr};
  std::vector<cinn_pod_value_t> args_cache_;
};

// true when a debug flag makes every instruction wait for its kernel (no HIP graph capture then)
bool InstructionsBlockTheStream();

class Program {
 public:
  // splits off the pre-run instructions (cinn/hlir/framework/graph_compiler.cc:66-76)
  Program(std::shared_ptr<Scope> scope, std::vector<std::unique_ptr<Instruction>> instrs);
  ~Program();
  // allocate every tensor the instructions touch
  void PreRun(const common::Target& target);
  // Runs the pre-run instructions (those whose inputs are all const, e.g. filter layout changes and folded
  // batch-norm statistics).  Execute / ExecuteGraph call it once by themselves; call it again after the data of
  // a const input has been replaced.
  void RunPreRunInstructions(void* stream = nullptr);
  // Runs all instructions on `stream`; with stream == nullptr the null stream is used and the device
  // is synchronised afterwards.
  void Execute(void* stream = nullptr);
  // Same work replayed from a HIP graph captured on first use (removes the per-kernel launch cost
  // of programs with many small kernels).  Falls back to Execute when capture is not possible.
  // With FLAGS_cinn_hip_graph_branches=1, instructions that do not depend on the one before them (the projection
  // shortcut of a residual block next to the block's main branch) are recorded on a second stream, so the graph holds
  // them as parallel branches; by default the graph is a single chain.
  void ExecuteGraph(void* stream);
  // stream lane (0: the caller's stream, 1: the side stream) of every run instruction in a graph replay
  const std::vector<int>& GraphLanes();
  size_t size() const { return instrs_.size(); }
  const std::vector<std::unique_ptr<Instruction>>& GetRunInstructions() const { return instrs_; }
  const std::vector<std::unique_ptr<Instruction>>& GetPreRunInstructions() const { return prerun_instrs_; }
  std::shared_ptr<Scope> scope() const { return scope_; }

 private:
  std::shared_ptr<Scope> scope_;
  std::vector<std::unique_ptr<Instruction>> instrs_;
  std::vector<std::unique_ptr<Instruction>> prerun_instrs_;
  bool prerun_done_{false};
  void* graph_exec_{nullptr};
  void* graph_{nullptr};
  // two-lane schedule of a graph replay
  void PlanLanes();
  void RunLanes(void* stream);
  bool lanes_planned_{false};
  bool any_side_{false};
  std::vector<int> lane_;                  // per run instruction
  std::vector<int> wait_for_;              // instruction on the other lane to wait for, or -1
  std::vector<void*> done_event_;          // recorded after the instruction when the other lane waits for it
  void* side_stream_{nullptr};
  void* fork_event_{nullptr};
  void* join_event_{nullptr};
};

struct GraphCompileOptions {
  bool with_instantiate_variables{true};
  bool reshape_as_view{true};  // groups made of reshapes only become views of their operand instead of copy kernels
  // consecutive generated kernels that do not depend on each other run as one launch (kernel_merge.h);
  // FLAGS_cinn_hip_merge_kernels=0 switches it off for a process
  bool merge_independent_kernels{true};
  // every tensor the instructions touch is a slice of one device allocation (DeviceArena); off: one allocation each
  bool memory_arena{true};
  // within the arena, intermediates (produced and consumed by run instructions, neither fed, fetched nor const) whose
  // lifetimes do not overlap share bytes; such a tensor cannot be read from the host - name it in the outputs
  bool reuse_intermediates{true};
  LoweringOptions lowering{LoweringOptions::FromEnv()};
};

class GraphCompiler final {
 public:
  using CompileOptions = GraphCompileOptions;
  GraphCompiler(const common::Target& target, std::shared_ptr<Scope> scope, std::shared_ptr<Graph> graph)
      : target_(target), scope_(std::move(scope)), graph_(std::move(graph)) {}

  std::unique_ptr<Program> Build(const CompileOptions& options = CompileOptions());
  // device source of the whole graph without loading anything
  std::string GenSourceCode(const CompileOptions& options = CompileOptions());
  const std::string& source_code() const { return source_code_; }
  // bytes of the program's device arena after Build (0: none was made), and what one allocation per tensor would take
  size_t arena_bytes() const { return arena_bytes_; }
  size_t unshared_bytes() const { return unshared_bytes_; }

 private:
  size_t arena_bytes_{0}, unshared_bytes_{0};
  ir::Module LowerGraph(const CompileOptions& options);
  // places the tensors of the instructions in one DeviceArena; returns its size
  size_t PlanMemory(const std::vector<std::unique_ptr<Instruction>>& instrs, const CompileOptions& options);
  common::Target target_;
  std::shared_ptr<Scope> scope_;
  std::shared_ptr<Graph> graph_;
  std::unique_ptr<backends::Compiler> compiler_;
  std::string source_code_;
  std::vector<LaunchUnit> units_;  // the program's instructions, filled by LowerGraph

 public:
  // the Compiler owns the loaded code objects and host stubs; a Program must not outlive it
  std::unique_ptr<backends::Compiler> ReleaseCompiler() { return std::move(compiler_); }
};

// creates scope tensors (shape + dtype) for every variable of the graph
std::shared_ptr<Scope> BuildScope(const common::Target& target, const std::shared_ptr<Graph>& graph,
                                  std::shared_ptr<Scope> scope = nullptr);

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
