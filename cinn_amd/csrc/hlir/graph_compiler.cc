#include "hlir/graph_compiler.h"

#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <set>

#include "hlir/accuracy_checker.h"
#include "hlir/memory_plan.h"
#include "optim/optimize.h"

namespace cinn {
namespace hlir {
namespace framework {

#define CINN_HIP_STATUS(expr)                                                                       \
  do {                                                                                              \
    int cinn_status__ = (expr);                                                                     \
    CINN_CHECK_EQ(cinn_status__, 0) << #expr << " failed: " << cinn_hip_error_string(cinn_status__); \
  } while (0)

// ---- DeviceArena ----------------------------------------------------------------------------------
DeviceArena::DeviceArena(size_t bytes) : bytes_(bytes) {
  void* p = nullptr;
  CINN_HIP_STATUS(cinn_hip_malloc(&p, bytes ? bytes : 256));
  base_ = static_cast<char*>(p);
}
DeviceArena::~DeviceArena() {
  if (base_) cinn_hip_free(base_);
}

// ---- Tensor ---------------------------------------------------------------------------------------
_Tensor_::_Tensor_() { cinn_hip_buffer_init(&buffer_, nullptr, cinn_type_float, 32, nullptr, 0); }
_Tensor_::~_Tensor_() { Free(); }

void _Tensor_::ShareBufferWith(const std::shared_ptr<_Tensor_>& source) {
  CINN_CHECK(source && source.get() != this) << "a tensor cannot be a view of itself";
  Free();
  source_ = source;
}

void _Tensor_::PlaceIn(std::shared_ptr<DeviceArena> arena, size_t offset, size_t capacity, bool transient) {
  CINN_CHECK(!source_) << "a view is placed with its source";
  CINN_CHECK(arena && offset + capacity <= arena->bytes()) << "tensor placed outside its arena";
  Free();
  arena_          = std::move(arena);
  arena_offset_   = offset;
  arena_capacity_ = capacity;
  transient_      = transient;
}

void _Tensor_::Free() {
  if (source_) {  // a view owns nothing
    buffer_.memory = nullptr;
    return;
  }
  if (arena_ && allocated_ == 0) {  // a slice of the arena: nothing of its own to free
    buffer_.memory = nullptr;
    return;
  }
  if (buffer_.memory) {
    cinn_hip_free(buffer_.memory);
    buffer_.memory = nullptr;
    allocated_     = 0;
  }
}

void _Tensor_::Resize(const ShapeType& shape) {
  CINN_CHECK_LE(shape.size(), static_cast<size_t>(CINN_BUFFER_MAX_DIMS)) << "tensors have at most 8 dimensions";
  shape_ = shape;
}

void _Tensor_::set_type(const common::Type& t) { type_ = t; }

void* _Tensor_::mutable_data(const common::Target& target) {
  CINN_CHECK(target.arch == common::Target::Arch::AMDGPU) << "device tensors need the AMDGPU target";
  size_t need = bytes();
  if (source_) {
    CINN_CHECK_EQ(need, source_->bytes()) << "a view must cover exactly its source's bytes";
    void* p = source_->mutable_data(target);
    if (buffer_.memory != p) {
      int code = type_.is_bool() ? cinn_type_int : (type_.is_bfloat16() ? cinn_type_bfloat : static_cast<int>(type_.code));
      cinn_hip_buffer_init(&buffer_, p, code, type_.is_bool() ? 1 : type_.bits, shape_.data(), static_cast<int>(shape_.size()));
      buffer_.memory_size = need;
    }
    return buffer_.memory;
  }
  if (arena_ && allocated_ == 0) {
    if (need <= arena_capacity_) {
      void* p = arena_->base() + arena_offset_;
      if (buffer_.memory != p || buffer_.memory_size != need) {
        int code = type_.is_bool() ? cinn_type_int : (type_.is_bfloat16() ? cinn_type_bfloat : static_cast<int>(type_.code));
        cinn_hip_buffer_init(&buffer_, p, code, type_.is_bool() ? 1 : type_.bits, shape_.data(), static_cast<int>(shape_.size()));
        buffer_.memory_size = need;
      }
      return buffer_.memory;
    }
    // resized beyond its slice: back to an allocation of its own
    buffer_.memory = nullptr;
    arena_.reset();
    transient_ = false;
  }
  if (!buffer_.memory || allocated_ < need) {
    Free();
    void* p = nullptr;
    CINN_HIP_STATUS(cinn_hip_malloc(&p, need));
    allocated_ = need;
    // runtime tag: bool is a 1-bit cinn_type_int there (cinn/runtime/cinn_runtime.cc cinn_bool_t)
    int code = type_.is_bool() ? cinn_type_int : (type_.is_bfloat16() ? cinn_type_bfloat : static_cast<int>(type_.code));
    cinn_hip_buffer_init(&buffer_, p, code, type_.is_bool() ? 1 : type_.bits, shape_.data(), static_cast<int>(shape_.size()));
    buffer_.memory_size = need;
  }
  return buffer_.memory;
}

void _Tensor_::CopyFromHost(const void* src, size_t n, const common::Target& target) {
  CINN_CHECK_EQ(n, bytes()) << "host data size does not match the tensor";
  void* dst = mutable_data(target);
  CINN_HIP_STATUS(cinn_hip_memcpy_h2d(dst, src, n, nullptr));
}
void _Tensor_::CopyToHost(void* dst, size_t n) const {
  CINN_CHECK_EQ(n, bytes()) << "host buffer size does not match the tensor";
  CINN_CHECK(data()) << "tensor has no device memory yet";
  CINN_HIP_STATUS(cinn_hip_memcpy_d2h(dst, data(), n, nullptr));
}

// ---- Scope ----------------------------------------------------------------------------------------
Tensor Scope::Var(const std::string& name) {
  auto it = data_.find(name);
  if (it != data_.end()) return it->second;
  auto t      = std::make_shared<_Tensor_>();
  data_[name] = t;
  return t;
}
Tensor Scope::FindVar(const std::string& name) const {
  auto it = data_.find(name);
  return it == data_.end() ? nullptr : it->second;
}
Tensor Scope::GetTensor(const std::string& name) const {
  auto t = FindVar(name);
  CINN_CHECK(t) << "no variable called '" << name << "' in the scope";
  return t;
}
std::vector<std::string> Scope::var_names() const {
  std::vector<std::string> names;
  for (auto& kv : data_) names.push_back(kv.first);
  return names;
}

// ---- Instruction ----------------------------------------------------------------------------------
void Instruction::UpdateArgsCache() {
  args_cache_.clear();
  auto add = [&](const std::string& name) {
    auto t = scope_->GetTensor(name);
    t->mutable_data(target_);
    cinn_pod_value_t v;
    cinn_hip_pod_from_buffer(&v, t->buffer());
    args_cache_.push_back(v);
  };
  for (auto& a : in_args_) add(a);
  for (auto& a : out_args_) add(a);
}

std::vector<const void*> Instruction::ArgAddresses(bool outputs) const {
  std::vector<const void*> out;
  for (auto& a : outputs ? out_args_ : in_args_) out.push_back(scope_->GetTensor(a)->mutable_data(target_));
  return out;
}

namespace {

// Debug switches of Instruction::Run, read once from the environment like the reference's flags
// (cinn/runtime/flags.cc): FLAGS_cinn_sync_run waits for every instruction, FLAGS_cinn_self_check_accuracy also
// reports its tensors (accuracy_checker.h), FLAGS_cinn_profiler_state != 0 brackets every instruction in a roctx
// range (the reference's RecordEvent / nvtx ranges, cinn/utils/profiler.cc:58-85) that rocprofv3 --marker-trace
// shows; the marker library is looked up at run time, a missing one disables the ranges.
struct RunFlags {
  bool sync_run{false};
  bool self_check{false};
  int (*range_push)(const char*){nullptr};
  int (*range_pop)(){nullptr};
  RunFlags() {
    auto on = [](const char* name) {
      const char* v = getenv(name);
      return v && *v && std::strcmp(v, "0") != 0 && std::strcmp(v, "false") != 0;
    };
    sync_run   = on("FLAGS_cinn_sync_run");
    self_check = SelfCheckSink::Get().enabled();
    if (on("FLAGS_cinn_profiler_state")) {
      void* lib = nullptr;
      for (const char* name : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"}) {
        lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
        if (lib) break;
      }
      if (lib) {
        range_push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
        range_pop  = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
        if (!range_push || !range_pop) range_push = nullptr, range_pop = nullptr;
      }
    }
  }
  bool blocking() const { return sync_run || self_check; }
};
const RunFlags& Flags() {
  static const RunFlags flags;
  return flags;
}

}  // namespace

bool InstructionsBlockTheStream() { return Flags().blocking(); }

void Instruction::Run(void* stream) {
  CINN_CHECK(fn_) << "instruction " << function_name_ << " has no compiled function";
  if (args_cache_.empty()) UpdateArgsCache();
  const RunFlags& flags = Flags();
  if (flags.range_push) flags.range_push(function_name_.c_str());
  fn_(args_cache_.data(), static_cast<int32_t>(args_cache_.size()), stream);
  if (flags.blocking()) CINN_HIP_STATUS(static_cast<int>(hipStreamSynchronize(static_cast<hipStream_t>(stream))));
  if (flags.self_check) CheckResults();
  if (flags.range_pop) flags.range_pop();
}

// the report of cinn/hlir/framework/instruction.cc:280-330: inputs and outputs in name order
void Instruction::CheckResults() {
  SelfCheckSink& sink = SelfCheckSink::Get();
  std::string text    = "Instruction {\n  Function " + function_name_ + ":\n";
  auto describe = [&](std::vector<std::string> names, const char* role) {
    std::sort(names.begin(), names.end());
    for (auto& n : names) text += std::string("    ") + role + ": " + DescribeTensor(scope_->GetTensor(n), n, sink.print_num()) + "\n";
  };
  describe(in_args_, "input");
  describe(out_args_, "output");
  text += "}";
  sink.Write(text);
}

// ---- Program --------------------------------------------------------------------------------------
Program::Program(std::shared_ptr<Scope> scope, std::vector<std::unique_ptr<Instruction>> instrs)
    : scope_(std::move(scope)) {
  for (auto& ins : instrs) {
    if (ins->pre_run) {
      prerun_instrs_.push_back(std::move(ins));
    } else {
      instrs_.push_back(std::move(ins));
    }
  }
}

Program::~Program() {
  if (graph_exec_) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec_));
  if (graph_) (void)hipGraphDestroy(static_cast<hipGraph_t>(graph_));
  for (void* e : done_event_)
    if (e) (void)hipEventDestroy(static_cast<hipEvent_t>(e));
  if (fork_event_) (void)hipEventDestroy(static_cast<hipEvent_t>(fork_event_));
  if (join_event_) (void)hipEventDestroy(static_cast<hipEvent_t>(join_event_));
  if (side_stream_) {
    (void)cinn_hip_scratch_release_stream(side_stream_);  // the library's per-stream scratch does not outlive the stream
    (void)hipStreamDestroy(static_cast<hipStream_t>(side_stream_));
  }
}

// Two stream lanes for a graph replay.  Instruction i depends on an earlier one that wrote what i reads or writes, or
// read what i writes (by device address, so two names for one allocation count as one).  In program order, an
// instruction that depends - directly or through others - on the last instruction of lane 0 continues lane 0; one
// that does not can run next to it and goes to lane 1.  Across lanes an instruction waits for the latest instruction
// of the other lane it depends on (stream order covers the earlier ones).
void Program::PlanLanes() {
  if (lanes_planned_) return;
  lanes_planned_ = true;
  const int n    = static_cast<int>(instrs_.size());
  lane_.assign(n, 0);
  wait_for_.assign(n, -1);
  done_event_.assign(n, nullptr);
  // Off unless asked for: on ResNet-50 (batch 32, fp16) the four forks and joins cost more than the overlap of the
  // shortcut convolutions with their main branches gains (1.022 ms per batch against 1.004 ms as a single chain).
  const char* flag = getenv("FLAGS_cinn_hip_graph_branches");
  if (!flag || std::strcmp(flag, "1") != 0) return;
  std::map<const void*, int> last_writer;
  std::map<const void*, std::vector<int>> readers;  // since the last write
  std::vector<std::vector<bool>> reach(n);          // reach[i][j]: i depends on j, directly or not
  int tail[2] = {-1, -1};
  for (int i = 0; i < n; ++i) {
    std::vector<int> deps;
    const auto ins  = instrs_[i]->ArgAddresses(false);
    const auto outs = instrs_[i]->ArgAddresses(true);
    for (const void* a : ins) {
      auto w = last_writer.find(a);
      if (w != last_writer.end()) deps.push_back(w->second);
    }
    for (const void* a : outs) {
      auto w = last_writer.find(a);
      if (w != last_writer.end()) deps.push_back(w->second);
      for (int r : readers[a]) deps.push_back(r);
    }
    reach[i].assign(n, false);
    for (int j : deps) {
      reach[i][j] = true;
      for (int k = 0; k < j; ++k)
        if (reach[j][k]) reach[i][k] = true;
    }
    const int l = (tail[0] < 0 || reach[i][tail[0]]) ? 0 : 1;
    lane_[i]    = l;
    tail[l]     = i;
    for (int j : deps)
      if (lane_[j] != l && j > wait_for_[i]) wait_for_[i] = j;
    for (const void* a : ins) readers[a].push_back(i);
    for (const void* a : outs) {
      last_writer[a] = i;
      readers[a].clear();
    }
    if (l == 1) any_side_ = true;
  }
  if (!any_side_) return;
  auto new_event = [] {
    hipEvent_t e = nullptr;
    CINN_HIP_STATUS(static_cast<int>(hipEventCreateWithFlags(&e, hipEventDisableTiming)));
    return static_cast<void*>(e);
  };
  for (int i = 0; i < n; ++i)
    if (wait_for_[i] >= 0 && !done_event_[wait_for_[i]]) done_event_[wait_for_[i]] = new_event();
  fork_event_ = new_event();
  join_event_ = new_event();
  hipStream_t side = nullptr;
  CINN_HIP_STATUS(static_cast<int>(hipStreamCreateWithFlags(&side, hipStreamNonBlocking)));  // default priority
  side_stream_ = side;
}

const std::vector<int>& Program::GraphLanes() {
  PlanLanes();
  return lane_;
}

// every run instruction on its lane; the side stream starts after what `stream` holds so far and is joined at the end
// (the fork / join a stream capture needs to take the second stream in and to end on the first)
void Program::RunLanes(void* stream) {
  PlanLanes();
  if (!any_side_) {
    for (auto& ins : instrs_) ins->Run(stream);
    return;
  }
  auto main_s = static_cast<hipStream_t>(stream);
  auto side_s = static_cast<hipStream_t>(side_stream_);
  CINN_HIP_STATUS(static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(fork_event_), main_s)));
  CINN_HIP_STATUS(static_cast<int>(hipStreamWaitEvent(side_s, static_cast<hipEvent_t>(fork_event_), 0)));
  for (size_t i = 0; i < instrs_.size(); ++i) {
    hipStream_t s = lane_[i] ? side_s : main_s;
    if (wait_for_[i] >= 0)
      CINN_HIP_STATUS(static_cast<int>(hipStreamWaitEvent(s, static_cast<hipEvent_t>(done_event_[wait_for_[i]]), 0)));
    instrs_[i]->Run(s);
    if (done_event_[i]) CINN_HIP_STATUS(static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(done_event_[i]), s)));
  }
  CINN_HIP_STATUS(static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(join_event_), side_s)));
  CINN_HIP_STATUS(static_cast<int>(hipStreamWaitEvent(main_s, static_cast<hipEvent_t>(join_event_), 0)));
}

void Program::PreRun(const common::Target& target) {
  for (auto* list : {&prerun_instrs_, &instrs_}) {
    for (auto& ins : *list) {
      for (auto& a : ins->in_args()) scope_->GetTensor(a)->mutable_data(target);
      for (auto& a : ins->out_args()) scope_->GetTensor(a)->mutable_data(target);
    }
  }
}

void Program::RunPreRunInstructions(void* stream) {
  for (auto& ins : prerun_instrs_) ins->Run(stream);
  prerun_done_ = true;
}

void Program::Execute(void* stream) {
  if (!prerun_done_) RunPreRunInstructions(stream);
  for (auto& ins : instrs_) ins->Run(stream);
  if (!stream) CINN_HIP_STATUS(cinn_hip_device_synchronize());
}

void Program::ExecuteGraph(void* stream) {
  CINN_CHECK(stream) << "graph replay needs an explicit stream";
  if (InstructionsBlockTheStream()) {
    // FLAGS_cinn_sync_run / FLAGS_cinn_self_check_accuracy wait after every instruction, which a capture forbids
    Execute(stream);
    return;
  }
  auto s = static_cast<hipStream_t>(stream);
  if (!prerun_done_) RunPreRunInstructions(stream);
  if (!graph_exec_) {
    // Library-call kernels allocate what they need on first use (the page of zeros, per-stream scratch), which a
    // capturing stream does not allow: run the program once before recording it, on the streams it will be recorded
    // on.
    RunLanes(stream);
    CINN_HIP_STATUS(static_cast<int>(hipStreamSynchronize(s)));
    // That run also sized the library's per-stream scratch (split-K partial sums, transposed operands), so the
    // recorded calls find it large enough; scratch a later call outgrows is retired, never freed, and the addresses
    // recorded here stay valid for every replay.
    hipGraph_t graph = nullptr;
    CINN_HIP_STATUS(static_cast<int>(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal)));
    try {
      RunLanes(stream);
    } catch (...) {
      // never leave the caller's stream in capture mode
      hipGraph_t partial = nullptr;
      (void)hipStreamEndCapture(s, &partial);
      if (partial) (void)hipGraphDestroy(partial);
      throw;
    }
    CINN_HIP_STATUS(static_cast<int>(hipStreamEndCapture(s, &graph)));
    hipGraphExec_t exec = nullptr;
    CINN_HIP_STATUS(static_cast<int>(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0)));
    graph_      = graph;
    graph_exec_ = exec;
  }
  CINN_HIP_STATUS(static_cast<int>(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec_), s)));
}

// ---- GraphCompiler --------------------------------------------------------------------------------
std::shared_ptr<Scope> BuildScope(const common::Target& target, const std::shared_ptr<Graph>& graph,
                                  std::shared_ptr<Scope> scope) {
  if (!scope) scope = Scope::Create();
  for (auto* v : graph->AllVars()) {
    auto t = scope->Var(v->id);
    t->Resize(v->shape);
    t->set_type(v->dtype);
  }
  (void)target;
  return scope;
}

namespace {
// one input, one output of the same type and size, and nothing but reshape operators in between
bool IsReshapeOnly(const Group& g) {
  if (g.inputs.size() != 1 || g.outputs.size() != 1 || g.nodes.empty()) return false;
  for (auto* n : g.nodes)
    if (n->op_type() != "reshape") return false;
  const auto* in  = g.inputs[0];
  const auto* out = g.outputs[0];
  return in->dtype == out->dtype && in->numel() == out->numel();
}
}  // namespace

ir::Module GraphCompiler::LowerGraph(const CompileOptions& options) {
  if (graph_->groups.empty()) graph_->BuildFusionGroups();
  OpLowerer lowerer(target_, options.lowering);
  ir::Module module;
  module.name   = "cinn_hip_module";
  module.target = target_;
  std::vector<ir::LoweredFuncRef> funcs;
  std::vector<bool> barrier;
  for (auto& g : graph_->groups) {
    auto func = lowerer.Lower(*g);
    if (func->is_device) optim::OptimizeFuncGPU(func.get());
    funcs.push_back(func);
    barrier.push_back(options.reshape_as_view && IsReshapeOnly(*g));  // becomes a view: no kernel to merge
  }
  KernelMergeOptions merge;
  const char* flag = getenv("FLAGS_cinn_hip_merge_kernels");
  merge.enabled    = options.merge_independent_kernels && !(flag && flag[0] == '0');
  if (merge.enabled && options.lowering.merged_rows_per_wave > 1) {
    // Which groups will share a launch is known once every kernel exists; row-reduce members are then lowered again
    // with that knowledge (a member's schedule may differ from the one it has alone, its block shape does not).
    std::vector<ir::LoweredFuncRef> trial;
    for (auto& unit : MergeIndependentKernels(graph_->groups, funcs, barrier, merge, &trial)) {
      if (unit.members.size() < 2) continue;
      for (const Group* member : unit.members) {
        if (member->kind != GroupKind::kRowReduce) continue;
        for (size_t i = 0; i < graph_->groups.size(); ++i) {
          if (graph_->groups[i].get() != member) continue;
          auto func = lowerer.Lower(*member, /*merged_member=*/true);
          if (func->is_device) optim::OptimizeFuncGPU(func.get());
          funcs[i] = func;
        }
      }
    }
  }
  units_           = MergeIndependentKernels(graph_->groups, funcs, barrier, merge, &module.functions);
  return module;
}

std::string GraphCompiler::GenSourceCode(const CompileOptions& options) {
  auto module  = LowerGraph(options);
  auto comp    = backends::Compiler::Create(target_);
  source_code_ = comp->GetSourceCode(module);
  return source_code_;
}

std::unique_ptr<Program> GraphCompiler::Build(const CompileOptions& options) {
  auto module = LowerGraph(options);
  compiler_   = backends::Compiler::Create(target_);
  compiler_->Build(module);
  source_code_ = compiler_->source_code();

  std::vector<std::unique_ptr<Instruction>> instrs;
  for (auto& u : units_) {
    if (u.members.size() == 1 && options.reshape_as_view && IsReshapeOnly(*u.members[0])) {
      // a reshape of a dense row-major tensor moves nothing: the result shares its operand's memory and no kernel
      // runs (the reference copies, cinn/hlir/op/transform.cc Reshape)
      scope_->Var(u.outputs[0]->id)->ShareBufferWith(scope_->Var(u.inputs[0]->id));
      continue;
    }
    std::vector<std::string> ins, outs;
    for (auto* v : u.inputs) ins.push_back(v->id);
    for (auto* v : u.outputs) outs.push_back(v->id);
    auto instr = std::make_unique<Instruction>(target_, scope_.get(), ins, outs, u.func_name);
    void* fn   = compiler_->Lookup(u.func_name);
    CINN_CHECK(fn) << "compiled function " << u.func_name << " not found";
    instr->SetLoweredFunc(fn);
    instr->pre_run = u.pre_run;
    instrs.push_back(std::move(instr));
  }
  int device_count = 0;
  if (options.with_instantiate_variables) cinn_hip_device_count(&device_count);
  if (device_count > 0 && options.memory_arena) arena_bytes_ = PlanMemory(instrs, options);
  auto program = std::make_unique<Program>(scope_, std::move(instrs));
  if (device_count > 0) program->PreRun(target_);
  return program;
}

// Memory plan of a compiled program.  Every tensor that an instruction reads or writes (views count as their source)
// and that has no memory yet gets a slice of one allocation:
//   * persistent slices, one each, for what the host or another execution may look at: fed inputs, fetched outputs,
//     const values and everything pre-run instructions touch;
//   * transient slices (PlanMemorySlots, memory_plan.h) for the rest - values produced by run instruction `def` and
//     last read by run instruction `last`.
// Slices are 256-byte aligned, the alignment the runtime's allocator gives and the kernels' 16-byte accesses rely on.
size_t GraphCompiler::PlanMemory(const std::vector<std::unique_ptr<Instruction>>& instrs, const CompileOptions& options) {
  constexpr size_t kAlign = 256;
  std::vector<MemorySlot> slots;
  std::vector<_Tensor_*> tensors;       // tensors[i] owns slots[i]
  std::map<_Tensor_*, size_t> index_of;
  std::vector<bool> written;            // by a run instruction
  auto root_of = [&](const std::string& name) {
    _Tensor_* t = scope_->GetTensor(name).get();
    while (t->source()) t = t->source().get();
    return t;
  };
  auto slot_of = [&](const std::string& name) -> size_t {
    _Tensor_* t = root_of(name);
    auto it     = index_of.find(t);
    if (it != index_of.end()) return it->second;
    MemorySlot s;
    s.bytes = std::max<size_t>(kAlign, (t->bytes() + kAlign - 1) / kAlign * kAlign);
    s.def = s.last = 0;
    slots.push_back(s);
    tensors.push_back(t);
    written.push_back(false);
    index_of[t] = slots.size() - 1;
    return slots.size() - 1;
  };
  // what must keep bytes of its own, by root tensor
  std::set<_Tensor_*> keep;
  for (auto* v : graph_->AllVars()) {
    if (!scope_->FindVar(v->id)) continue;
    if (v->producer == nullptr || v->is_fetch || v->is_const || !options.reuse_intermediates) keep.insert(root_of(v->id));
  }
  int index = 0;
  for (auto& ins : instrs) {
    if (ins->pre_run) {
      for (auto* list : {&ins->in_args(), &ins->out_args()})
        for (auto& a : *list) slots[slot_of(a)].persistent = true;
      continue;
    }
    for (auto& a : ins->in_args()) {
      const size_t i = slot_of(a);
      if (!written[i]) slots[i].persistent = true;  // read before any run instruction wrote it
      slots[i].last = index;
    }
    for (auto& a : ins->out_args()) {
      const size_t i = slot_of(a);
      if (!written[i]) slots[i].def = index;
      written[i]    = true;
      slots[i].last = index;
    }
    ++index;
  }
  // tensors the caller gave memory already stay where they are
  std::vector<MemorySlot> plan;
  std::vector<_Tensor_*> planned;
  unshared_bytes_ = 0;
  for (size_t i = 0; i < slots.size(); ++i) {
    if (tensors[i]->data() != nullptr) continue;
    if (keep.count(tensors[i])) slots[i].persistent = true;
    unshared_bytes_ += slots[i].bytes;
    plan.push_back(slots[i]);
    planned.push_back(tensors[i]);
  }
  if (plan.empty()) return 0;
  const size_t total = PlanMemorySlots(&plan);
  auto arena         = std::make_shared<DeviceArena>(total);
  for (size_t i = 0; i < plan.size(); ++i) planned[i]->PlaceIn(arena, plan[i].offset, plan[i].bytes, !plan[i].persistent);
  return total;
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
