// CinnComputation: build, compile and run a program on the GPU.  Interface of
// cinn/frontend/computation.h:27-159 (BuildAndCompile / Compile / Execute / GetTensor /
// SetTensorData / GetTensorData); the compile pipeline is the one of CompileProgram
// (cinn/frontend/computation.cc:43-95) with the gfx950 GraphCompiler underneath.
#pragma once
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "frontend/net_builder.h"
#include "hlir/graph_compiler.h"

namespace cinn {
namespace frontend {

class CinnComputation {
 public:
  struct CompileOptions : public hlir::framework::GraphCompiler::CompileOptions {
    // composite ops (softmax, batch_norm) are always decomposed on this backend: its kernels are
    // generated from primitives only
    bool use_decomposer{true};
    bool do_prerun{true};
    // fold `conv2d -> batch_norm [-> + residual] [-> relu]` on channels-last tensors into one convolution call whose
    // epilogue applies the folded batch norm in fp32 on the accumulators (frontend/layout_pass.h).  The result
    // differs from the unfused operation order by rounding only; switch it off to get that order exactly.
    bool fuse_conv_bn_relu{true};
    bool fuse_stem_pool{true};  // fold the max pooling after an image convolution into it
    // `matmul(x, W) + bias` with a const 2-D W and a const bias in a 16-bit type: the bias is added in the product's
    // epilogue (frontend/layout_pass.h); the result differs from the two operators by one rounding
    bool fuse_matmul_bias{true};
    // two folded 1x1 convolutions in a row whose channel counts the chain kernel takes become one call that writes
    // both results (frontend/layout_pass.h); same results as the two calls
    bool fuse_conv_chain{true};
    // a folded 1x1 convolution that adds a folded 1x1 projection of another tensor (a bottleneck block's last layer and
    // its projection shortcut) becomes one call over both inputs, the batch-norm scales multiplied into the filters
    // (needs fuse_conv_bn_relu)
    bool fuse_shortcut_projection{true};
    // move conv2d chains written in NCHW to channels-last tensors, the layout the MFMA convolution kernels read
    // with 16-byte accesses (frontend/layout_pass.h); off: every conv2d runs in the layout it was written in
    bool conv_layout_nhwc{true};
    // rewrite reductions over non-trailing axes into chains of per-run (and, for small outputs, two-step) reductions
    // that fill the chip (frontend/reduce_split_pass.h); off: such a reduction is one kernel whatever its grid size
    bool split_reductions{true};
  };
  static CompileOptions DefaultCompileOptions() { return CompileOptions(); }

  static std::shared_ptr<CinnComputation> BuildAndCompile(const common::Target& target, NetBuilder& builder,
                                                          const CompileOptions& options        = DefaultCompileOptions(),
                                                          const std::vector<Variable>& outputs = {},
                                                          void* stream                         = nullptr);
  static std::shared_ptr<CinnComputation> Compile(const common::Target& target, Program& program,
                                                  const CompileOptions& options        = DefaultCompileOptions(),
                                                  const std::vector<Variable>& outputs = {}, void* stream = nullptr);

  std::vector<std::string> GetAllTensorNames();
  hlir::framework::Tensor GetTensor(const std::string& name);
  std::vector<hlir::framework::Tensor> GetInputTensors();
  std::vector<hlir::framework::Tensor> GetOutputTensors();
  void SetTensorData(hlir::framework::Tensor& t, void* data, size_t size);
  void SetTensorData(const std::string& tname, void* data, size_t size);
  void GetTensorData(hlir::framework::Tensor& t, void* data, size_t size);
  void GetTensorData(const std::string& tname, void* data, size_t size);

  // run the compiled program once (synchronises when the computation has no stream)
  void Execute();
  // replay through a captured HIP graph; needs a stream
  void ExecuteGraph();
  // runs the pre-run instructions again (after the data of a const input was replaced)
  void PreRun();

  const std::string& source_code() const { return source_code_; }
  std::string group_debug_string() const { return graph_->DebugGroupString(); }
  size_t num_instructions() const { return program_->size(); }
  // size of the program's one device allocation (0: tensors are allocated one by one) and the sum of the sizes its
  // tensors would have without sharing
  size_t arena_bytes() const { return arena_bytes_; }
  size_t unshared_bytes() const { return unshared_bytes_; }
  // stream lane (0 / 1) of every run instruction in a graph replay
  const std::vector<int>& GraphLanes() { return program_->GraphLanes(); }
  const std::vector<std::string>& output_names() const { return output_names_; }
  const std::vector<std::string>& input_names() const { return input_names_; }
  void* stream() const { return stream_; }
  hlir::framework::Program* program() const { return program_.get(); }

 private:
  common::Target target_;
  void* stream_{nullptr};
  std::shared_ptr<hlir::framework::Graph> graph_;
  std::shared_ptr<hlir::framework::Scope> scope_;
  std::unique_ptr<hlir::framework::Program> program_;
  std::unique_ptr<backends::Compiler> compiler_;
  std::vector<std::string> input_names_, output_names_;
  std::string source_code_;
  size_t arena_bytes_{0}, unshared_bytes_{0};
};

}  // namespace frontend
}  // namespace cinn
