#include "frontend/syntax.h"

#include <sstream>

namespace cinn {
namespace utils {

namespace {
std::vector<std::string> SplitString(const std::string& s, char sep) {
  std::vector<std::string> out;
  std::string cur;
  for (char c : s) {
    if (c == sep) {
      out.push_back(cur);
      cur.clear();
    } else {
      cur.push_back(c);
    }
  }
  out.push_back(cur);
  return out;
}
}  // namespace

AttributeMap ParseAttributeString(const std::string& text) {
  AttributeMap attrs;
  if (text.empty()) return attrs;
  for (auto& item : SplitString(text, ';')) {
    if (item.empty()) continue;
    auto colon = item.find(':');
    auto eq    = item.find('=', colon == std::string::npos ? 0 : colon);
    CINN_CHECK(colon != std::string::npos && eq != std::string::npos) << "malformed attribute '" << item << "'";
    std::string key = item.substr(0, colon);
    std::string tag = item.substr(colon + 1, eq - colon - 1);
    std::string val = item.substr(eq + 1);
    if (tag == "b") {
      attrs[key] = (val == "1" || val == "true" || val == "True");
    } else if (tag == "i") {
      attrs[key] = std::stoi(val);
    } else if (tag == "f") {
      attrs[key] = std::stof(val);
    } else if (tag == "d") {
      attrs[key] = std::stod(val);
    } else if (tag == "s") {
      attrs[key] = val;
    } else if (tag == "vi") {
      std::vector<int> v;
      if (!val.empty())
        for (auto& e : SplitString(val, ',')) v.push_back(std::stoi(e));
      attrs[key] = v;
    } else if (tag == "vf") {
      std::vector<float> v;
      if (!val.empty())
        for (auto& e : SplitString(val, ',')) v.push_back(std::stof(e));
      attrs[key] = v;
    } else if (tag == "vs") {
      std::vector<std::string> v;
      if (!val.empty()) v = SplitString(val, ',');
      attrs[key] = v;
    } else {
      CINN_CHECK(false) << "unknown attribute tag '" << tag << "' in '" << item << "'";
    }
  }
  return attrs;
}

std::string AttributeToString(const Attribute& a) {
  std::ostringstream os;
  std::visit(
      [&](auto&& v) {
        using T = std::decay_t<decltype(v)>;
        if constexpr (std::is_same_v<T, std::vector<int>> || std::is_same_v<T, std::vector<float>> ||
                      std::is_same_v<T, std::vector<std::string>>) {
          os << "[";
          for (size_t i = 0; i < v.size(); ++i) os << (i ? "," : "") << v[i];
          os << "]";
        } else {
          os << v;
        }
      },
      a);
  return os.str();
}

}  // namespace utils

namespace frontend {

std::string Instruction::debug_string() const {
  std::ostringstream os;
  for (size_t i = 0; i < p_->outputs.size(); ++i) os << (i ? ", " : "") << p_->outputs[i]->id;
  os << " = " << p_->op_type << "(";
  for (size_t i = 0; i < p_->inputs.size(); ++i) os << (i ? ", " : "") << p_->inputs[i]->id;
  for (auto& kv : p_->attrs) os << ", " << kv.first << "=" << utils::AttributeToString(kv.second);
  os << ")";
  return os.str();
}

std::string Program::debug_string() const {
  std::ostringstream os;
  for (auto& ins : instrs_) os << ins.debug_string() << "\n";
  return os.str();
}

}  // namespace frontend
}  // namespace cinn
