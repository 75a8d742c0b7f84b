#include "hlir/graph_compiler.h"

#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "hlir/accuracy_checker.h"
#include "optim/optimize.h"

namespace cinn {
namespace hlir {
namespace framework {

#define CINN_HIP_STATUS(expr)                                                                       \
  do {                                                                                              \
    int cinn_status__ = (expr);                                                                     \
    CINN_CHECK_EQ(cinn_status__, 0) << #expr << " failed: " << cinn_hip_error_string(cinn_status__); \
  } while (0)

// ---- Tensor ---------------------------------------------------------------------------------------
_Tensor_::_Tensor_() { cinn_hip_buffer_init(&buffer_, nullptr, cinn_type_float, 32, nullptr, 0); }
_Tensor_::~_Tensor_() { Free(); }

void _Tensor_::ShareBufferWith(const std::shared_ptr<_Tensor_>& source) {
  CINN_CHECK(source && source.get() != this) << "a tensor cannot be a view of itself";
  Free();
  source_ = source;
}

void _Tensor_::Free() {
  if (source_) {  // a view owns nothing
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
    // Library-call kernels build per-shape tables and set function attributes on their first launch, which a
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

ir::Module GraphCompiler::LowerGraph(const CompileOptions& options) {
  if (graph_->groups.empty()) graph_->BuildFusionGroups();
  OpLowerer lowerer(target_, options.lowering);
  ir::Module module;
  module.name   = "cinn_hip_module";
  module.target = target_;
  for (auto& g : graph_->groups) {
    auto func = lowerer.Lower(*g);
    if (func->is_device) optim::OptimizeFuncGPU(func.get());
    module.functions.push_back(func);
  }
  return module;
}

std::string GraphCompiler::GenSourceCode(const CompileOptions& options) {
  auto module  = LowerGraph(options);
  auto comp    = backends::Compiler::Create(target_);
  source_code_ = comp->GetSourceCode(module);
  return source_code_;
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

std::unique_ptr<Program> GraphCompiler::Build(const CompileOptions& options) {
  auto module = LowerGraph(options);
  compiler_   = backends::Compiler::Create(target_);
  compiler_->Build(module);
  source_code_ = compiler_->source_code();

  std::vector<std::unique_ptr<Instruction>> instrs;
  for (auto& g : graph_->groups) {
    if (options.reshape_as_view && IsReshapeOnly(*g)) {
      // a reshape of a dense row-major tensor moves nothing: the result shares its operand's memory and no kernel
      // runs (the reference copies, cinn/hlir/op/transform.cc Reshape)
      scope_->Var(g->outputs[0]->id)->ShareBufferWith(scope_->Var(g->inputs[0]->id));
      continue;
    }
    std::vector<std::string> ins, outs;
    for (auto* v : g->inputs) ins.push_back(v->id);
    for (auto* v : g->outputs) outs.push_back(v->id);
    auto instr = std::make_unique<Instruction>(target_, scope_.get(), ins, outs, g->func_name);
    void* fn   = compiler_->Lookup(g->func_name);
    CINN_CHECK(fn) << "compiled function " << g->func_name << " not found";
    instr->SetLoweredFunc(fn);
    instr->pre_run = g->pre_run;
    instrs.push_back(std::move(instr));
  }
  auto program = std::make_unique<Program>(scope_, std::move(instrs));
  if (options.with_instantiate_variables) {
    int device_count = 0;
    cinn_hip_device_count(&device_count);
    if (device_count > 0) program->PreRun(target_);
  }
  return program;
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
