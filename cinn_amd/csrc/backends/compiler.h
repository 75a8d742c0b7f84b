// JIT driver of the gfx950 backend; interface of backends::Compiler (cinn/backends/compiler.h:53-93).
// Build() runs the sequence the reference runs in Compiler::CompileCudaModule
// (cinn/backends/compiler.cc:107-148) with the HIP pieces substituted:
//   split host/device -> CodeGenHIP_Dev -> hiprtc -> code object -> hipModuleLoadData ->
//   kernel handles registered as "<kernel>_ptr_" symbols -> host functions lowered to stubs.
// Lookup(name) returns the lower_func_ptr_g of a host function.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "cinn_hip_runtime.h"
#include "ir/ir.h"

namespace cinn {
namespace backends {

class Compiler final {
 public:
  static std::unique_ptr<Compiler> Create(const common::Target& target) {
    return std::unique_ptr<Compiler>(new Compiler(target));
  }
  ~Compiler();

  // Compile a module.  `code` may carry device source text to use instead of the generated one
  // (as the reference allows, compiler.h:62-66).  Without a visible GPU the device source is still
  // generated and compiled to a code object (so that "does it compile" is testable anywhere), but
  // Lookup()ed functions refuse to run.
  void Build(const ir::Module& module, const std::string& code = "");
  // device source text CodeGenHIP_Dev generates for the module
  std::string GetSourceCode(const ir::Module& module);
  // source of the last Build()
  const std::string& source_code() const { return source_code_; }
  size_t code_object_size() const { return code_object_size_; }

  void* Lookup(const std::string& fn_name);

 private:
  explicit Compiler(const common::Target& target) : target_(target) {}
  Compiler(const Compiler&) = delete;
  common::Target target_;
  std::vector<cinn_hip_module_t> modules_;
  std::map<std::string, lower_func_ptr_g> functions_;
  std::string source_code_;
  size_t code_object_size_{0};
};

// Dump of generated sources when FLAGS_cinn_source_code_save_path names a file, as SourceCodePrint
// does (cinn/backends/compiler.cc:38-68).
void SaveSourceCode(const std::string& source);

}  // namespace backends
}  // namespace cinn
