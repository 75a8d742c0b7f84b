#include "frontend/layout_pass.h"

#include <algorithm>
#include <map>
#include <set>

#include "cinn_hip_runtime.h"
#include "frontend/pass_util.h"
#include "hlir/op.h"
#include "kernels/conv_chain.h"
#include "kernels/stem_pool.h"

namespace cinn {
namespace frontend {

namespace {

using hlir::framework::GetAttr;
using hlir::framework::OpPatternKind;
using hlir::framework::OpRegistry;
using utils::AttributeMap;
using utils::ShapeType;

ShapeType ToNhwc(const ShapeType& s) { return {s[0], s[2], s[3], s[1]}; }

bool MfmaType(const common::Type& t) { return t.is_float(32) || t.is_float(16) || t.is_bfloat16(); }

class LayoutConverter {
 public:
  LayoutConverter(const Program& program, const std::set<std::string>& fetch_ids)
      : program_(program), fetch_ids_(fetch_ids), emit_(&out_, "nhwc_") {}

  Program Run() {
    for (auto& in : program_.GetInputs()) have_nchw_.insert(in->id);
    for (auto& ins : program_.instructions()) {
      for (auto& o : ins->outputs) vars_[o->id] = o;
      Visit(ins);
    }
    for (auto& id : fetch_ids_) {
      auto it = vars_.find(id);
      if (it != vars_.end()) EnsureNchw(it->second);
    }
    return Program(std::move(out_), program_.GetInputs(), program_.name());
  }

 private:
  bool HasTwin(const Variable& v) const { return nhwc_.count(v->id) != 0; }

  // channels-last version of a 4-D NCHW value
  Variable GetNhwc(const Variable& v) {
    auto it = nhwc_.find(v->id);
    if (it != nhwc_.end()) return it->second;
    Variable t;
    auto bc = channel_broadcast_.find(v->id);
    if (bc != channel_broadcast_.end() && !have_nchw_.count(v->id)) {
      // a per-channel vector replicated over an NCHW tensor: replicate it over the NHWC one instead
      t = emit_.Emit1("broadcast_to", {bc->second->inputs[0]},
                      {{"out_shape", ToNhwc(v->shape)}, {"broadcast_axes", ShapeType{3}}});
    } else {
      EnsureNchw(v);
      if (v->shape[1] == 1 || (v->shape[2] == 1 && v->shape[3] == 1)) {
        t = emit_.Emit1("reshape", {v}, {{"shape", ToNhwc(v->shape)}});
      } else {
        t = emit_.Emit1("transpose", {v}, {{"axis", ShapeType{0, 2, 3, 1}}});
      }
    }
    nhwc_[v->id] = t;
    return t;
  }

  // makes sure the original (NCHW) variable is defined by an emitted instruction
  void EnsureNchw(const Variable& v) {
    if (have_nchw_.count(v->id)) return;
    auto bc = channel_broadcast_.find(v->id);
    if (bc != channel_broadcast_.end()) {
      out_.push_back(bc->second);
    } else {
      auto it = nhwc_.find(v->id);
      CINN_CHECK(it != nhwc_.end()) << "variable " << v->id << " is used before it is defined";
      if (v->shape[1] == 1 || (v->shape[2] == 1 && v->shape[3] == 1)) {
        emit_.EmitInto(v, "reshape", {it->second}, {{"shape", v->shape}});
      } else {
        emit_.EmitInto(v, "transpose", {it->second}, {{"axis", ShapeType{0, 3, 1, 2}}});
      }
    }
    have_nchw_.insert(v->id);
  }

  Variable FilterToOhwi(const Variable& w) {
    auto it = filters_.find(w->id);
    if (it != filters_.end()) return it->second;
    EnsureNchw(w);
    Variable t;
    if (w->shape[2] == 1 && w->shape[3] == 1) {
      t = emit_.Emit1("reshape", {w}, {{"shape", ShapeType{w->shape[0], 1, 1, w->shape[1]}}});
    } else {
      t = emit_.Emit1("transpose", {w}, {{"axis", ShapeType{0, 2, 3, 1}}});
    }
    filters_[w->id] = t;
    return t;
  }

  void KeepAsIs(const Instruction& ins) {
    for (auto& in : ins->inputs) {
      if (in->shape.size() == 4 || channel_broadcast_.count(in->id)) EnsureNchw(in);
    }
    out_.push_back(ins);
    for (auto& o : ins->outputs) have_nchw_.insert(o->id);
  }

  void Visit(const Instruction& ins) {
    const std::string& op = ins->op_type;
    if (op == "conv2d") {
      auto x = ins->inputs[0], w = ins->inputs[1];
      bool nchw    = GetAttr<std::string>(ins->attrs, "data_format", "NCHW") == "NCHW";
      bool forward = GetAttr<std::string>(ins->attrs, "conv_type", "forward") == "forward";
      int groups   = GetAttr<int>(ins->attrs, "groups", 1);
      const int chunk = 16 / x->type.bytes();
      // depthwise: one filter per channel (the channels-last kernel wants whole 16-byte channel vectors)
      const bool depthwise = groups > 1 && x->shape.size() == 4 && w->shape.size() == 4 && groups == x->shape[1] &&
                             groups == w->shape[0] && w->shape[1] == 1 && x->shape[1] % chunk == 0;
      if (nchw && forward && (groups == 1 || depthwise) && x->shape.size() == 4 && MfmaType(x->type)) {
        AttributeMap attrs   = ins->attrs;
        attrs["data_format"] = std::string("NHWC");
        Variable y;
        if (x->shape[1] % chunk == 0) {
          y = emit_.Emit1("conv2d", {GetNhwc(x), FilterToOhwi(w)}, attrs);
        } else {
          // a channel count that is not a whole number of 16-byte chunks (an image, or LeNet-style 6 / 12 channels,
          // also when the producer left only a channels-last twin): the kernel reads the NCHW tensor and the
          // [O][I][KH][KW] filter as they are
          EnsureNchw(x);
          EnsureNchw(w);
          attrs["input_layout"] = std::string("NCHW");
          y                     = emit_.Emit1("conv2d", {x, w}, attrs);
        }
        nhwc_[ins->outputs[0]->id] = y;
        return;
      }
    } else if (op == "batch_norm") {
      auto x = ins->inputs[0];
      if (GetAttr<std::string>(ins->attrs, "data_layout", "NCHW") == "NCHW" && x->shape.size() == 4 && HasTwin(x)) {
        AttributeMap attrs   = ins->attrs;
        attrs["data_layout"] = std::string("NHWC");
        std::vector<Variable> inputs = ins->inputs;
        inputs[0]                    = GetNhwc(x);
        auto outs                    = emit_.Emit("batch_norm", inputs, attrs);
        nhwc_[ins->outputs[0]->id]   = outs[0];
        return;
      }
    } else if (op == "pool2d") {
      auto x = ins->inputs[0];
      if (GetAttr<std::string>(ins->attrs, "data_format", "NCHW") == "NCHW" && x->shape.size() == 4 && HasTwin(x)) {
        AttributeMap attrs   = ins->attrs;
        attrs["data_format"] = std::string("NHWC");
        nhwc_[ins->outputs[0]->id] = emit_.Emit1("pool2d", {GetNhwc(x)}, attrs);
        return;
      }
    } else if (op == "broadcast_to") {
      auto x    = ins->inputs[0];
      auto axes = GetAttr<ShapeType>(ins->attrs, "broadcast_axes", {});
      auto& out = ins->outputs[0];
      if (out->shape.size() == 4 && x->shape.size() == 1 && axes.size() == 1 && axes[0] == 1 &&
          x->shape[0] == out->shape[1]) {
        // decided by the first consumer: emitted as it is, or replicated over the channels-last shape
        channel_broadcast_[out->id] = ins;
        return;
      }
    } else {
      const auto* def = OpRegistry::Global().Find(op);
      if (def && def->pattern == OpPatternKind::kElementWise && ins->outputs.size() == 1 &&
          ins->outputs[0]->shape.size() == 4 && !ins->inputs.empty()) {
        bool same_shape = true, any_twin = false;
        for (auto& in : ins->inputs) {
          same_shape = same_shape && in->shape == ins->outputs[0]->shape;
          any_twin   = any_twin || (HasTwin(in) && !have_nchw_.count(in->id));
        }
        if (same_shape && any_twin) {
          std::vector<Variable> inputs;
          for (auto& in : ins->inputs) inputs.push_back(GetNhwc(in));
          nhwc_[ins->outputs[0]->id] = emit_.Emit1(op, inputs, ins->attrs);
          return;
        }
      }
    }
    KeepAsIs(ins);
  }

  const Program& program_;
  const std::set<std::string>& fetch_ids_;
  std::vector<Instruction> out_;
  Emitter emit_;
  std::map<std::string, Variable> vars_;     // every variable an instruction of the program defines
  std::map<std::string, Variable> nhwc_;     // NCHW variable id -> its channels-last twin
  std::map<std::string, Variable> filters_;  // filter id -> [O][KH][KW][I] copy
  std::set<std::string> have_nchw_;          // ids whose NCHW form is defined in the output program
  std::map<std::string, Instruction> channel_broadcast_;  // deferred per-channel broadcast_to instructions
};

}  // namespace

Program ConvertConvLayoutToNHWC(const Program& program, const std::set<std::string>& fetch_ids) {
  bool has_conv = false;
  for (auto& ins : program.instructions()) has_conv = has_conv || ins->op_type == "conv2d";
  if (!has_conv) return program;
  return LayoutConverter(program, fetch_ids).Run();
}

Program PretransposeConstMatmulWeights(const Program& program) {
  std::vector<Instruction> out;
  Emitter emit(&out, "wt_");
  std::map<std::string, Variable> transposed;
  for (auto& ins : program.instructions()) {
    if (ins->op_type == "matmul" && ins->inputs.size() == 2 && ins->inputs[1]->is_const &&
        ins->inputs[1]->shape.size() == 2 && !GetAttr<bool>(ins->attrs, "trans_b", false)) {
      auto w  = ins->inputs[1];
      auto it = transposed.find(w->id);
      if (it == transposed.end())
        it = transposed.emplace(w->id, emit.Emit1("transpose", {w}, {{"axis", ShapeType{1, 0}}})).first;
      AttributeMap attrs = ins->attrs;
      attrs["trans_b"]   = true;
      Instruction m("matmul");
      m->inputs  = {ins->inputs[0], it->second};
      m->attrs   = attrs;
      m->outputs = ins->outputs;
      out.push_back(m);
    } else {
      out.push_back(ins);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

namespace {
// conv: channels-last convolution of an NCHW image; pool: its only consumer (after batch norm and relu).  True when the
// image-convolution kernel can take the pooling along (conv_stem7_mfma.hip): 7x7 / stride 2 / padding 3 over three
// channels in a 16-bit type, followed by max pooling 3x3 / stride 2 / padding 1 without ceil mode.
bool StemMaxPoolFusable(const Instruction& conv, const Instruction& pool) {
  if (GetAttr<std::string>(conv->attrs, "input_layout", "NHWC") != "NCHW") return false;
  if (GetAttr<std::string>(pool->attrs, "data_format", "NCHW") != "NHWC") return false;
  if (GetAttr<std::string>(pool->attrs, "pool_type", "max") != "max" || GetAttr<bool>(pool->attrs, "global_pooling", false) ||
      GetAttr<bool>(pool->attrs, "adaptive", false) || GetAttr<bool>(pool->attrs, "ceil_mode", false))
    return false;
  auto ksize = GetAttr<std::vector<int>>(pool->attrs, "kernel_size", {1, 1});
  auto pstr  = GetAttr<std::vector<int>>(pool->attrs, "stride_size", {1, 1});
  auto ppad  = GetAttr<std::vector<int>>(pool->attrs, "padding_size", {0, 0, 0, 0});
  if (ksize != std::vector<int>{3, 3} || pstr != std::vector<int>{2, 2}) return false;
  for (int v : ppad)
    if (v != 1) return false;
  auto stride   = GetAttr<std::vector<int>>(conv->attrs, "stride", {1, 1});
  auto padding  = GetAttr<std::vector<int>>(conv->attrs, "padding", {0, 0});
  auto dilation = GetAttr<std::vector<int>>(conv->attrs, "dilation", {1, 1});
  const auto& x = conv->inputs[0]->shape;  // NCHW
  const auto& w = conv->inputs[1]->shape;  // OIHW
  if (x.size() != 4 || w.size() != 4 || GetAttr<int>(conv->attrs, "groups", 1) != 1) return false;
  const auto& t = conv->inputs[0]->type;
  if (!t.is_floating()) return false;
  return cinn_hip_kernels::StemPoolFusableShape(x[0], x[1], x[2], x[3], w[0], w[2], w[3], stride[0], stride[1], padding[0],
                                                padding[1], dilation[0], dilation[1],
                                                t.is_bfloat16() ? cinn_type_bfloat : cinn_type_float, t.bits);
}
}  // namespace

Program FuseConvBatchNorm(const Program& program, const std::set<std::string>& fetch_ids, bool fuse_stem_pool) {
  const auto& instrs = program.instructions();
  // consumers of every variable
  std::map<std::string, std::vector<size_t>> users;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& in : instrs[i]->inputs) users[in->id].push_back(i);
  std::map<std::string, size_t> defined_at;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& o : instrs[i]->outputs) defined_at[o->id] = i;
  auto single_user = [&](const Variable& v) -> int {
    if (fetch_ids.count(v->id)) return -1;
    auto it = users.find(v->id);
    if (it == users.end() || it->second.size() != 1) return -1;
    return static_cast<int>(it->second[0]);
  };

  std::vector<bool> dropped(instrs.size(), false);
  std::map<size_t, std::vector<Instruction>> replacement;  // position of the last instruction of a match
  int serial = 0;
  for (size_t i = 0; i < instrs.size(); ++i) {
    auto& conv = instrs[i];
    if (conv->op_type != "conv2d" || dropped[i]) continue;
    if (GetAttr<std::string>(conv->attrs, "data_format", "NCHW") != "NHWC") continue;
    if (GetAttr<std::string>(conv->attrs, "conv_type", "forward") != "forward") continue;
    // grouped convolutions in channels-last form are depthwise ones (the layout pass converts no others); their kernel
    // has the same epilogue
    int bn_at = single_user(conv->outputs[0]);
    if (bn_at < 0 || instrs[bn_at]->op_type != "batch_norm" || !(instrs[bn_at]->inputs[0] == conv->outputs[0])) continue;
    auto& bn = instrs[bn_at];
    if (GetAttr<std::string>(bn->attrs, "data_layout", "NCHW") != "NHWC") continue;
    size_t last     = bn_at;
    Variable result = bn->outputs[0];
    Variable residual;
    bool relu = false;
    int next  = single_user(result);
    if (next >= 0 && !dropped[next] && instrs[next]->op_type == "elementwise_add" && instrs[next]->inputs.size() == 2) {
      auto& add     = instrs[next];
      Variable other = add->inputs[0] == result ? add->inputs[1] : add->inputs[0];
      // the other operand must exist when this convolution's inputs do: of two convolution branches meeting in an
      // addition, the later one takes the addition
      auto def          = defined_at.find(other->id);
      bool other_earlier = def == defined_at.end() || def->second < i;
      if (!(other == result) && other->shape == result->shape && other_earlier) {
        residual = other;
        dropped[next] = true;
        last     = next;
        result   = add->outputs[0];
        next     = single_user(result);
      }
    }
    if (next >= 0 && !dropped[next] && instrs[next]->op_type == "relu") {
      relu          = true;
      dropped[next] = true;
      last          = next;
      result        = instrs[next]->outputs[0];
      next          = single_user(result);
    }
    // a 3x3, stride 2, padding 1 max pooling after the image convolution's relu runs inside the convolution kernel
    bool max_pool = false;
    if (fuse_stem_pool && relu && !residual.defined() && next >= 0 && !dropped[next] && instrs[next]->op_type == "pool2d" &&
        StemMaxPoolFusable(conv, instrs[next])) {
      max_pool      = true;
      dropped[next] = true;
      last          = next;
      result        = instrs[next]->outputs[0];
    }
    dropped[i]     = true;
    dropped[bn_at] = true;

    // s = scale / sqrt(variance + eps), t = bias - mean * s, in fp32
    std::vector<Instruction> seq;
    Emitter e(&seq, "cbr" + std::to_string(serial++) + "_");
    float eps  = GetAttr<float>(bn->attrs, "epsilon", 1e-5f);
    auto to_f32 = [&](const Variable& v) {
      if (v->type == common::Float(32)) return v;
      return e.Emit1("cast", {v}, {{"dtype", std::string("float32")}});
    };
    auto scale = to_f32(bn->inputs[1]), bias = to_f32(bn->inputs[2]), mean = to_f32(bn->inputs[3]),
         var   = to_f32(bn->inputs[4]);
    auto epsv  = e.Emit1("fill_constant", {},
                         {{"shape", var->shape}, {"value", static_cast<double>(eps)}, {"dtype", std::string("float32")}, {"force_cpu", false}});
    auto denom = e.Emit1("sqrt", {e.Emit1("elementwise_add", {var, epsv}, {{"axis", -1}})}, {});
    auto s     = e.Emit1("divide", {scale, denom}, {{"axis", -1}});
    auto t     = e.Emit1("subtract", {bias, e.Emit1("elementwise_mul", {mean, s}, {{"axis", -1}})}, {{"axis", -1}});
    AttributeMap attrs = conv->attrs;
    attrs["relu"]      = relu;
    attrs["max_pool"]  = max_pool;
    std::vector<Variable> inputs = {conv->inputs[0], conv->inputs[1], s, t};
    if (residual.defined()) inputs.push_back(residual);
    e.EmitInto(result, "hip_conv2d_bn_relu", inputs, attrs);
    replacement[last] = seq;
  }
  std::vector<Instruction> out;
  for (size_t i = 0; i < instrs.size(); ++i) {
    auto it = replacement.find(i);
    if (it != replacement.end()) {
      out.insert(out.end(), it->second.begin(), it->second.end());
    } else if (!dropped[i]) {
      out.push_back(instrs[i]);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

Program FuseMatmulBias(const Program& program, const std::set<std::string>& fetch_ids) {
  const auto& instrs = program.instructions();
  std::map<std::string, std::vector<size_t>> users;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& in : instrs[i]->inputs) users[in->id].push_back(i);
  // values known before the first run: const inputs and what is computed from them alone
  std::set<std::string> known;
  for (auto& v : program.GetInputs())
    if (v->is_const) known.insert(v->id);
  std::map<std::string, size_t> defined_at;
  for (size_t i = 0; i < instrs.size(); ++i) {
    bool all = true;
    for (auto& in : instrs[i]->inputs) all = all && (in->is_const || known.count(in->id));
    for (auto& o : instrs[i]->outputs) {
      defined_at[o->id] = i;
      if (all) known.insert(o->id);
    }
  }
  std::vector<bool> dropped(instrs.size(), false);
  std::map<size_t, std::vector<Instruction>> replacement;
  int serial = 0;
  for (size_t i = 0; i < instrs.size(); ++i) {
    auto& mm = instrs[i];
    if (mm->op_type != "matmul" || mm->inputs.size() != 2 || mm->outputs.size() != 1) continue;
    const Variable &x = mm->inputs[0], &w = mm->inputs[1], &prod = mm->outputs[0];
    if (x->shape.size() != 2 || w->shape.size() != 2 || prod->shape.size() != 2) continue;
    if (GetAttr<bool>(mm->attrs, "trans_a", false) || !GetAttr<bool>(mm->attrs, "trans_b", false) ||
        GetAttr<float>(mm->attrs, "alpha", 1.0f) != 1.0f)
      continue;
    if (!(x->type.is_float16() || x->type.is_bfloat16()) || !(w->type == x->type)) continue;
    const int m = x->shape[0], k = x->shape[1], n = w->shape[0];
    if (w->shape[1] != k || prod->shape != ShapeType{m, n}) continue;
    if (fetch_ids.count(prod->id)) continue;
    auto u = users.find(prod->id);
    if (u == users.end() || u->second.size() != 1) continue;
    const size_t add_at = u->second[0];
    auto& add           = instrs[add_at];
    if (add->op_type != "elementwise_add" || add->inputs.size() != 2 || dropped[add_at]) continue;
    Variable bias  = add->inputs[0] == prod ? add->inputs[1] : add->inputs[0];
    const int axis = GetAttr<int>(add->attrs, "axis", -1);
    if (bias == prod) continue;
    // the builder's addition broadcasts the bias to [M][N] first (broadcast_to over axis 1)
    int bcast_at = -1;
    auto bdef    = defined_at.find(bias->id);
    if (bias->shape == ShapeType{m, n} && bdef != defined_at.end() && instrs[bdef->second]->op_type == "broadcast_to") {
      auto& bc  = instrs[bdef->second];
      auto axes = GetAttr<std::vector<int>>(bc->attrs, "broadcast_axes", {});
      auto bu   = users.find(bias->id);
      if (bc->inputs.size() != 1 || axes.size() != 1 || (axes[0] != 1 && axes[0] != -1) || fetch_ids.count(bias->id) ||
          bu == users.end() || bu->second.size() != 1 || dropped[bdef->second])
        continue;
      bcast_at = static_cast<int>(bdef->second);
      bias     = bc->inputs[0];
    } else if (axis != -1 && axis != 1) {
      continue;
    }
    if (bias->shape != ShapeType{n}) continue;
    if (!(bias->is_const || known.count(bias->id))) continue;
    auto def = defined_at.find(bias->id);
    if (def != defined_at.end() && def->second > i) continue;
    if (add->outputs[0]->shape != ShapeType{m, n} || !(add->outputs[0]->type == x->type)) continue;

    std::vector<Instruction> seq;
    Emitter e(&seq, "mmb" + std::to_string(serial++) + "_");
    auto x4   = e.Emit1("reshape", {x}, {{"shape", ShapeType{m, 1, 1, k}}});
    auto w4   = e.Emit1("reshape", {w}, {{"shape", ShapeType{n, 1, 1, k}}});
    auto ones = e.Emit1("fill_constant", {},
                        {{"shape", ShapeType{n}}, {"value", 1.0}, {"dtype", std::string("float32")}, {"force_cpu", false}});
    auto shift = bias->type == common::Float(32) ? bias : e.Emit1("cast", {bias}, {{"dtype", std::string("float32")}});
    AttributeMap attrs = {{"stride", std::vector<int>{1, 1}},   {"padding", std::vector<int>{0, 0}},
                          {"dilation", std::vector<int>{1, 1}}, {"groups", 1},
                          {"data_format", std::string("NHWC")}, {"relu", false},
                          {"max_pool", false}};
    auto y4 = e.Emit1("hip_conv2d_bn_relu", {x4, w4, ones, shift}, attrs);
    e.EmitInto(add->outputs[0], "reshape", {y4}, {{"shape", ShapeType{m, n}}});
    dropped[i]      = true;
    dropped[add_at] = true;
    if (bcast_at >= 0) dropped[bcast_at] = true;
    replacement[add_at] = seq;
  }
  if (replacement.empty()) return program;
  std::vector<Instruction> out;
  for (size_t i = 0; i < instrs.size(); ++i) {
    auto it = replacement.find(i);
    if (it != replacement.end()) {
      out.insert(out.end(), it->second.begin(), it->second.end());
    } else if (!dropped[i]) {
      out.push_back(instrs[i]);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

Program FuseConvChain(const Program& program, const std::set<std::string>& fetch_ids) {
  (void)fetch_ids;  // both results of a pair stay outputs of the new call, fetched or not
  const auto& instrs = program.instructions();
  std::map<std::string, std::vector<size_t>> users;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& in : instrs[i]->inputs) users[in->id].push_back(i);
  // a folded convolution that is a matrix product over the channels of each pixel
  auto pointwise = [](const Instruction& ins) {
    if (ins->op_type != "hip_conv2d_bn_relu" || ins->inputs.size() < 4) return false;
    const auto& a = ins->attrs;
    if (GetAttr<std::string>(a, "data_format", "NCHW") != "NHWC" || GetAttr<std::string>(a, "input_layout", "NHWC") != "NHWC") return false;
    if (GetAttr<bool>(a, "max_pool", false) || GetAttr<int>(a, "groups", 1) != 1) return false;
    if (GetAttr<std::vector<int>>(a, "stride", {1, 1}) != std::vector<int>{1, 1} ||
        GetAttr<std::vector<int>>(a, "padding", {0, 0}) != std::vector<int>{0, 0} ||
        GetAttr<std::vector<int>>(a, "dilation", {1, 1}) != std::vector<int>{1, 1})
      return false;
    const auto& x = ins->inputs[0];
    const auto& w = ins->inputs[1];
    if (x->shape.size() != 4 || w->shape.size() != 4 || w->shape[1] != 1 || w->shape[2] != 1 || w->shape[3] != x->shape[3]) return false;
    return x->type.is_floating() && x->type.bits == 16 && w->type == x->type;
  };
  std::map<std::string, size_t> defined_at;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& o : instrs[i]->outputs) defined_at[o->id] = i;
  std::vector<bool> dropped(instrs.size(), false);
  // what is emitted in front of instruction i: hoisted parameter computations of the second convolution, then the call
  std::map<size_t, std::vector<Instruction>> before;
  for (size_t i = 0; i < instrs.size(); ++i) {
    const auto& first = instrs[i];
    if (dropped[i] || !pointwise(first)) continue;
    const Variable& e = first->outputs[0];
    auto it = users.find(e->id);
    if (it == users.end()) continue;
    std::vector<size_t> readers = it->second;
    std::sort(readers.begin(), readers.end());
    // the second convolution: the first reader of e that qualifies
    size_t at = instrs.size();
    for (size_t r : readers) {
      const auto& c = instrs[r];
      if (r <= i || dropped[r] || !pointwise(c) || c->inputs.size() != 4) continue;
      if (!(c->inputs[0] == e) || c->inputs[1] == e || c->inputs[2] == e || c->inputs[3] == e) continue;
      const int64_t m = static_cast<int64_t>(e->shape[0]) * e->shape[1] * e->shape[2];
      if (!cinn_hip_kernels::ConvChainShape(m, first->inputs[0]->shape[3], e->shape[3], c->outputs[0]->shape[3])) continue;
      at = r;
      break;
    }
    if (at == instrs.size()) continue;
    const auto& second = instrs[at];
    // The call produces e, so it goes in front of e's earliest reader.  What the second convolution's filter, scale and
    // shift are computed from between there and its own position comes along, provided none of it reads e.
    const size_t where = readers.front();
    if (where <= i || before.count(where)) continue;
    std::set<size_t> hoist;
    bool ok = true;
    std::vector<Variable> work(second->inputs.begin() + 1, second->inputs.end());
    while (ok && !work.empty()) {
      Variable v = work.back();
      work.pop_back();
      auto def = defined_at.find(v->id);
      if (def == defined_at.end() || def->second < where) continue;  // a program input, or ready in time
      if (def->second >= at || dropped[def->second]) {
        ok = false;
        break;
      }
      if (!hoist.insert(def->second).second) continue;
      for (auto& in : instrs[def->second]->inputs) {
        if (in == e) ok = false;
        work.push_back(in);
      }
    }
    if (!ok) continue;
    Instruction chain("hip_conv2d_bn_relu_chain");
    chain->inputs = first->inputs;  // x, w1, scale1, shift1[, residual]
    chain->inputs.insert(chain->inputs.end(), second->inputs.begin() + 1, second->inputs.end());
    chain->outputs = {e, second->outputs[0]};
    chain->attrs["relu"]       = GetAttr<bool>(first->attrs, "relu", false);
    chain->attrs["relu_after"] = GetAttr<bool>(second->attrs, "relu", false);
    std::vector<Instruction> seq;
    for (size_t h : hoist) {
      seq.push_back(instrs[h]);
      dropped[h] = true;
    }
    seq.push_back(chain);
    dropped[i]    = true;
    dropped[at]   = true;
    before[where] = seq;
  }
  if (before.empty()) return program;
  std::vector<Instruction> out;
  for (size_t i = 0; i < instrs.size(); ++i) {
    auto it = before.find(i);
    if (it != before.end()) out.insert(out.end(), it->second.begin(), it->second.end());
    if (!dropped[i]) out.push_back(instrs[i]);
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

Program FuseShortcutProjection(const Program& program, const std::set<std::string>& fetch_ids) {
  const auto& instrs = program.instructions();
  std::map<std::string, std::vector<size_t>> users;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& in : instrs[i]->inputs) users[in->id].push_back(i);
  std::map<std::string, size_t> defined_at;
  for (size_t i = 0; i < instrs.size(); ++i)
    for (auto& o : instrs[i]->outputs) defined_at[o->id] = i;
  // a folded 1x1 convolution without padding or dilation on channels-last 16-bit tensors, at any stride
  auto pointwise = [](const Instruction& ins) {
    if (ins->op_type != "hip_conv2d_bn_relu" || ins->inputs.size() < 4) return false;
    const auto& a = ins->attrs;
    if (GetAttr<std::string>(a, "data_format", "NCHW") != "NHWC" || GetAttr<std::string>(a, "input_layout", "NHWC") != "NHWC") return false;
    if (GetAttr<bool>(a, "max_pool", false) || GetAttr<int>(a, "groups", 1) != 1) return false;
    if (GetAttr<std::vector<int>>(a, "padding", {0, 0}) != std::vector<int>{0, 0} ||
        GetAttr<std::vector<int>>(a, "dilation", {1, 1}) != std::vector<int>{1, 1})
      return false;
    const auto& x = ins->inputs[0];
    const auto& w = ins->inputs[1];
    if (x->shape.size() != 4 || w->shape.size() != 4 || w->shape[1] != 1 || w->shape[2] != 1 || w->shape[3] != x->shape[3]) return false;
    return x->type.is_floating() && x->type.bits == 16 && w->type == x->type;
  };
  std::vector<bool> dropped(instrs.size(), false);
  std::map<size_t, std::vector<Instruction>> replacement;
  int serial = 0;
  // the filters of two layers side by side along their channels, each times its scale: multiplied in fp32, rounded once
  // to the storage type
  auto scaled_side_by_side = [](Emitter& e, const Variable& w1, const Variable& s1, const Variable& w2, const Variable& s2) {
    const std::string store = w1->type.is_bfloat16() ? "bfloat16" : "float16";
    auto scaled = [&](const Variable& w, const Variable& s) {
      auto w32 = e.Emit1("cast", {w}, {{"dtype", std::string("float32")}});
      auto sb  = e.Emit1("broadcast_to", {s}, {{"out_shape", w->shape}, {"broadcast_axes", ShapeType{0}}});
      auto ws  = e.Emit1("elementwise_mul", {w32, sb}, {{"axis", -1}});
      return e.Emit1("cast", {ws}, {{"dtype", store}});
    };
    return e.Emit1("concat", {scaled(w1, s1), scaled(w2, s2)}, {{"axis", 3}});
  };
  // the projection behind residual r of the instruction at position i, or null: a folded 1x1 projection without relu
  // that nothing else reads
  auto projection_of = [&](const Variable& r, size_t i) -> const Instruction* {
    auto def = defined_at.find(r->id);
    if (def == defined_at.end() || def->second >= i || dropped[def->second]) return nullptr;
    const auto& proj = instrs[def->second];
    if (!pointwise(proj) || proj->inputs.size() != 4 || GetAttr<bool>(proj->attrs, "relu", false)) return nullptr;
    auto ru = users.find(r->id);
    if (fetch_ids.count(r->id) || ru == users.end() || ru->second.size() != 1) return nullptr;
    return &proj;
  };
  for (size_t i = 0; i < instrs.size(); ++i) {
    const auto& main = instrs[i];
    if (main->op_type == "hip_conv2d_bn_relu_chain" && main->inputs.size() == 8) {
      // x, w1, scale1, shift1, residual, w2, scale2, shift2 -> e, y: the residual becomes a second input of the first layer
      const Variable& r = main->inputs[4];
      const Instruction* pp = projection_of(r, i);
      if (!pp) continue;
      const auto& proj = *pp;
      const Variable &x = main->inputs[0], &x2 = proj->inputs[0], &e_out = main->outputs[0], &y = main->outputs[1];
      if (x == r || !(x2->type == x->type) || r->shape != e_out->shape) continue;
      if (GetAttr<std::vector<int>>(proj->attrs, "stride", {1, 1}) != std::vector<int>{1, 1}) continue;
      if (x2->shape[0] != x->shape[0] || x2->shape[1] != x->shape[1] || x2->shape[2] != x->shape[2]) continue;
      const int64_t m = static_cast<int64_t>(x->shape[0]) * x->shape[1] * x->shape[2];
      if (!cinn_hip_kernels::ConvChainShape2(m, x->shape[3], x2->shape[3], e_out->shape[3], y->shape[3])) continue;
      std::vector<Instruction> seq;
      Emitter e(&seq, "csp" + std::to_string(serial++) + "_");
      auto w_both = scaled_side_by_side(e, main->inputs[1], main->inputs[2], proj->inputs[1], proj->inputs[2]);
      auto shift  = e.Emit1("elementwise_add", {main->inputs[3], proj->inputs[3]}, {{"axis", -1}});
      Instruction chain("hip_conv2d_pair_chain");
      chain->inputs  = {x, x2, w_both, shift, main->inputs[5], main->inputs[6], main->inputs[7]};
      chain->outputs = main->outputs;
      chain->attrs["relu"]       = GetAttr<bool>(main->attrs, "relu", false);
      chain->attrs["relu_after"] = GetAttr<bool>(main->attrs, "relu_after", false);
      seq.push_back(chain);
      dropped[defined_at[r->id]] = true;
      dropped[i]                 = true;
      replacement[i]             = seq;
      continue;
    }
    if (!pointwise(main) || main->inputs.size() != 5) continue;
    if (GetAttr<std::vector<int>>(main->attrs, "stride", {1, 1}) != std::vector<int>{1, 1}) continue;
    const Variable& r = main->inputs[4];
    const Instruction* pp = projection_of(r, i);
    if (!pp) continue;
    const auto& proj = *pp;
    const Variable &x = main->inputs[0], &x2 = proj->inputs[0], &y = main->outputs[0];
    if (x == r || !(x2->type == x->type) || r->shape != y->shape) continue;
    auto stride2 = GetAttr<std::vector<int>>(proj->attrs, "stride", {1, 1});
    if (stride2.size() != 2 || (x->shape[1] - 1) * stride2[0] >= x2->shape[1] || (x->shape[2] - 1) * stride2[1] >= x2->shape[2]) continue;
    const int64_t m = static_cast<int64_t>(x->shape[0]) * x->shape[1] * x->shape[2];
    if (!cinn_hip_kernels::ConvPairShape(m, x->shape[3], x2->shape[3], y->shape[3])) continue;

    // y = act(s1 (w1 x) + t1 + s2 (w2 x2) + t2) = act([s1 w1 | s2 w2] [x; x2] + (t1 + t2)): the scales go into the filters
    // (multiplied in fp32, rounded once to the storage type), the filters side by side along their channels
    std::vector<Instruction> seq;
    Emitter e(&seq, "csp" + std::to_string(serial++) + "_");
    auto w_both = scaled_side_by_side(e, main->inputs[1], main->inputs[2], proj->inputs[1], proj->inputs[2]);
    auto shift  = e.Emit1("elementwise_add", {main->inputs[3], proj->inputs[3]}, {{"axis", -1}});
    e.EmitInto(y, "hip_conv2d_pointwise_pair", {x, x2, w_both, shift},
               {{"second_stride", stride2}, {"relu", GetAttr<bool>(main->attrs, "relu", false)}});
    dropped[defined_at[r->id]] = true;
    dropped[i]                 = true;
    replacement[i]             = seq;
  }
  if (replacement.empty()) return program;
  std::vector<Instruction> out;
  for (size_t i = 0; i < instrs.size(); ++i) {
    auto it = replacement.find(i);
    if (it != replacement.end()) {
      out.insert(out.end(), it->second.begin(), it->second.end());
    } else if (!dropped[i]) {
      out.push_back(instrs[i]);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

}  // namespace frontend
}  // namespace cinn
