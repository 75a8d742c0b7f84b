// Run-time self-check of an instruction's tensors, the debugging aid behind FLAGS_cinn_self_check_accuracy
// (cinn/hlir/framework/accuracy_checker.{h,cc}, instruction.cc:280-330): every tensor is copied to the host and
// described as "name=..., dtype=..., shape=..., data=[first values, ... , last values], <verdict>" with the verdict
// NaN, Inf, Zero (all zero), One (all one) or OK.
#pragma once
#include <string>

#include "hlir/graph_compiler.h"

namespace cinn {
namespace hlir {
namespace framework {

// elements printed from each end of a tensor (FLAGS_cinn_self_check_accuracy_num: default 5, < 0 prints all)
std::string DescribeTensor(const Tensor& tensor, const std::string& name, int print_num);

// where FLAGS_cinn_self_check_accuracy sends the reports: unset / false: nowhere; true / 1: stderr; anything else
// is a file name
class SelfCheckSink {
 public:
  static SelfCheckSink& Get();
  bool enabled() const { return enabled_; }
  int print_num() const { return print_num_; }
  void Write(const std::string& text);

 private:
  SelfCheckSink();
  ~SelfCheckSink();
  bool enabled_{false};
  int print_num_{5};
  void* file_{nullptr};
};

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
