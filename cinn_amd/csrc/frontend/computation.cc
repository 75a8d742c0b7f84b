#include "frontend/computation.h"

#include "frontend/decomposer.h"
#include "frontend/layout_pass.h"
#include "frontend/reduce_split_pass.h"

namespace cinn {
namespace frontend {

using hlir::framework::Graph;
using hlir::framework::GraphCompiler;

std::shared_ptr<CinnComputation> CinnComputation::BuildAndCompile(const common::Target& target, NetBuilder& builder,
                                                                  const CompileOptions& options,
                                                                  const std::vector<Variable>& outputs, void* stream) {
  Program program = builder.Build();
  return Compile(target, program, options, outputs, stream);
}

std::shared_ptr<CinnComputation> CinnComputation::Compile(const common::Target& target, Program& program,
                                                          const CompileOptions& options,
                                                          const std::vector<Variable>& outputs, void* stream) {
  CINN_CHECK(target.arch == common::Target::Arch::AMDGPU) << "CinnComputation of this build compiles for AMDGPU only";
  CINN_CHECK_GT(program.size(), 0u) << "cannot compile an empty program";
  auto comp     = std::make_shared<CinnComputation>();
  comp->target_ = target;
  comp->stream_ = stream;

  std::set<std::string> fetch_ids;
  if (outputs.empty()) {
    // the output variable of the last instruction is used (computation.cc:78-83)
    for (auto& o : program[program.size() - 1]->outputs) {
      fetch_ids.insert(o->id);
      comp->output_names_.push_back(o->id);
    }
  } else {
    for (auto& o : outputs) {
      fetch_ids.insert(o->id);
      comp->output_names_.push_back(o->id);
    }
  }
  for (auto& in : program.GetInputs()) comp->input_names_.push_back(in->id);

  Program lowered = PretransposeConstMatmulWeights(program);
  if (options.conv_layout_nhwc) lowered = ConvertConvLayoutToNHWC(lowered, fetch_ids);
  if (options.fuse_conv_bn_relu) lowered = FuseConvBatchNorm(lowered, fetch_ids, options.fuse_stem_pool);
  if (options.fuse_matmul_bias) lowered = FuseMatmulBias(lowered, fetch_ids);
  if (options.fuse_conv_bn_relu && options.fuse_conv_chain) lowered = FuseConvChain(lowered, fetch_ids);
  if (options.fuse_conv_bn_relu && options.fuse_shortcut_projection) lowered = FuseShortcutProjection(lowered, fetch_ids);
  if (options.use_decomposer) lowered = ApplyDecomposer(lowered);
  if (options.split_reductions) lowered = SplitReductions(lowered, target.get_multi_processor_count());
  comp->graph_    = std::make_shared<Graph>(lowered, fetch_ids, target);
  comp->graph_->BuildFusionGroups();
  comp->scope_ = hlir::framework::BuildScope(target, comp->graph_);

  GraphCompiler gc(target, comp->scope_, comp->graph_);
  GraphCompiler::CompileOptions gopts = options;
  gopts.with_instantiate_variables    = options.do_prerun && options.with_instantiate_variables;
  comp->program_                      = gc.Build(gopts);
  comp->source_code_                  = gc.source_code();
  comp->arena_bytes_                  = gc.arena_bytes();
  comp->unshared_bytes_               = gc.unshared_bytes();
  comp->compiler_                     = gc.ReleaseCompiler();
  return comp;
}

std::vector<std::string> CinnComputation::GetAllTensorNames() { return scope_->var_names(); }
hlir::framework::Tensor CinnComputation::GetTensor(const std::string& name) { return scope_->GetTensor(name); }
std::vector<hlir::framework::Tensor> CinnComputation::GetInputTensors() {
  std::vector<hlir::framework::Tensor> out;
  for (auto& n : input_names_) out.push_back(GetTensor(n));
  return out;
}
std::vector<hlir::framework::Tensor> CinnComputation::GetOutputTensors() {
  std::vector<hlir::framework::Tensor> out;
  for (auto& n : output_names_) out.push_back(GetTensor(n));
  return out;
}
namespace {
// An intermediate whose bytes other values of the program reuse holds nothing the host could rely on.
void CheckHostVisible(const hlir::framework::Tensor& t, const char* what) {
  const hlir::framework::_Tensor_* root = t.get();
  while (root->source()) root = root->source().get();
  CINN_CHECK(!root->is_transient())
      << what << ": this tensor is an intermediate of the compiled program whose device memory is shared with other "
      << "intermediates (compile option reuse_intermediates); name it in the outputs of build_and_compile, or compile "
      << "with reuse_intermediates=0, to give it memory of its own";
}
}  // namespace

void CinnComputation::SetTensorData(hlir::framework::Tensor& t, void* data, size_t size) {
  CheckHostVisible(t, "SetTensorData");
  t->CopyFromHost(data, size, target_);
}
void CinnComputation::SetTensorData(const std::string& tname, void* data, size_t size) {
  auto t = GetTensor(tname);
  SetTensorData(t, data, size);
}
void CinnComputation::GetTensorData(hlir::framework::Tensor& t, void* data, size_t size) {
  CheckHostVisible(t, "GetTensorData");
  t->CopyToHost(data, size);
}
void CinnComputation::GetTensorData(const std::string& tname, void* data, size_t size) {
  auto t = GetTensor(tname);
  GetTensorData(t, data, size);
}
void CinnComputation::Execute() { program_->Execute(stream_); }
void CinnComputation::ExecuteGraph() { program_->ExecuteGraph(stream_); }
void CinnComputation::PreRun() { program_->RunPreRunInstructions(stream_); }

}  // namespace frontend
}  // namespace cinn
