// Rebuilding traversal over the IR: Mutate() returns the same node when no child changed and a
// fresh node otherwise, so passes never modify shared sub-trees in place.
#pragma once
#include <functional>

#include "ir/ir.h"

namespace cinn {
namespace ir {

class IrMutator {
 public:
  virtual ~IrMutator() = default;
  virtual Expr Mutate(const Expr& e);

 protected:
  Expr MutateChildren(const Expr& e);
};

// replace every occurrence of the variable named `name` by `value`
Expr Substitute(const Expr& e, const std::string& name, const Expr& value);
// true when a variable named `name` occurs in e
bool UsesVar(const Expr& e, const std::string& name);
// pre-order visit of every node
void Walk(const Expr& e, const std::function<void(const Expr&)>& fn);

}  // namespace ir
}  // namespace cinn
