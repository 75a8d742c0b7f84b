// Program-level data structures of the front end: Variable, Instruction, Program.  They mirror
// cinn/frontend/syntax.h (a Program is an ordered list of Instructions over Variables carrying a
// static shape and an element type; ids are unique strings).
#pragma once
#include <map>
#include <memory>
#include <string>
#include <variant>
#include <vector>

#include "common/type.h"

namespace cinn {
namespace utils {
using ShapeType    = std::vector<int>;
using Attribute    = std::variant<bool, int, float, double, std::string, std::vector<int>, std::vector<float>,
                               std::vector<std::string>>;
using AttributeMap = std::map<std::string, Attribute>;

// "key:tag=value;..." with tags b i f d s vi vf vs; used by the C API to carry attributes
AttributeMap ParseAttributeString(const std::string& text);
std::string AttributeToString(const Attribute& a);
}  // namespace utils

namespace frontend {

struct _Variable_ {
  std::string id;
  utils::ShapeType shape;
  common::Type type;
  bool is_const{false};
};

class Variable {
 public:
  Variable() = default;
  explicit Variable(const std::string& id) : p_(std::make_shared<_Variable_>()) { p_->id = id; }
  _Variable_* operator->() const { return p_.get(); }
  _Variable_* get() const { return p_.get(); }
  bool defined() const { return p_ != nullptr; }
  bool operator==(const Variable& o) const { return p_ == o.p_; }

 private:
  std::shared_ptr<_Variable_> p_;
};

// a fed input of the program
using Placeholder = Variable;

struct _Instruction_ {
  std::string op_type;
  std::vector<Variable> inputs;
  std::vector<Variable> outputs;
  utils::AttributeMap attrs;
};

class Instruction {
 public:
  Instruction() = default;
  explicit Instruction(const std::string& op_type) : p_(std::make_shared<_Instruction_>()) { p_->op_type = op_type; }
  _Instruction_* operator->() const { return p_.get(); }
  _Instruction_* get() const { return p_.get(); }

  template <typename T>
  T GetAttrs(const std::string& key) const {
    auto it = p_->attrs.find(key);
    CINN_CHECK(it != p_->attrs.end()) << "instruction " << p_->op_type << " has no attribute '" << key << "'";
    CINN_CHECK(std::holds_alternative<T>(it->second))
        << "attribute '" << key << "' of " << p_->op_type << " has another type";
    return std::get<T>(it->second);
  }
  bool HasAttr(const std::string& key) const { return p_->attrs.count(key) != 0; }
  std::string debug_string() const;

 private:
  std::shared_ptr<_Instruction_> p_;
};

class Program {
 public:
  Program() = default;
  Program(std::vector<Instruction> instrs, std::vector<Variable> inputs, std::string name = "")
      : instrs_(std::move(instrs)), inputs_(std::move(inputs)), name_(std::move(name)) {}
  // name of the builder that made the program; generated kernels carry it in their names
  const std::string& name() const { return name_; }
  size_t size() const { return instrs_.size(); }
  const Instruction& operator[](size_t i) const { return instrs_[i]; }
  const std::vector<Instruction>& instructions() const { return instrs_; }
  const std::vector<Variable>& GetInputs() const { return inputs_; }
  void SetInstructions(std::vector<Instruction> instrs) { instrs_ = std::move(instrs); }
  std::string debug_string() const;

 private:
  std::vector<Instruction> instrs_;
  std::vector<Variable> inputs_;
  std::string name_;
};

}  // namespace frontend
}  // namespace cinn
