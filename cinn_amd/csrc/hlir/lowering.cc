#include "hlir/lowering.h"

#include <algorithm>
#include <cstdlib>
#include <functional>
#include <limits>
#include <set>

namespace cinn {
namespace hlir {
namespace framework {

using common::Type;
using ir::BufferRef;
using ir::Expr;
using ir::ForType;
using ir::MemoryType;

namespace {

// ---------------------------------------------------------------------------------------------------
// small helpers
// ---------------------------------------------------------------------------------------------------
Expr I32(int64_t v) { return ir::MakeIntImm(common::Int(32), v); }

std::string CName(const std::string& id) {
  std::string out;
  for (char c : id) out.push_back((isalnum(static_cast<unsigned char>(c)) || c == '_') ? c : '_');
  if (out.empty() || isdigit(static_cast<unsigned char>(out[0]))) out = "v_" + out;
  // a tensor may be named like a keyword or a built-in of the kernel language ("short", "float", "threadIdx"): as a
  // parameter name that would not compile
  static const std::set<std::string> reserved = {
      "alignas", "alignof", "and", "asm", "auto", "bool", "break", "case", "catch", "char", "class", "const", "constexpr",
      "continue", "default", "delete", "do", "double", "else", "enum", "explicit", "export", "extern", "false", "float", "for",
      "friend", "goto", "if", "inline", "int", "long", "mutable", "namespace", "new", "not", "nullptr", "operator", "or",
      "private", "protected", "public", "register", "return", "short", "signed", "sizeof", "static", "struct", "switch",
      "template", "this", "throw", "true", "try", "typedef", "typename", "union", "unsigned", "using", "virtual", "void",
      "volatile", "while", "xor", "half", "float16", "bfloat16", "threadIdx", "blockIdx", "blockDim", "gridDim", "warpSize",
      "int8_t", "int16_t", "int32_t", "int64_t", "uint8_t", "uint16_t", "uint32_t", "uint64_t", "size_t", "min", "max"};
  if (reserved.count(out)) out = "v_" + out;
  // ... or like a name the generated code uses for its own variables: the loop and index variables, the numbered
  // temporaries (<hint>_<n>) and the members of a merged kernel (m<k>_...)
  auto all_digits = [](const std::string& t) {
    return !t.empty() && std::all_of(t.begin(), t.end(), [](char c) { return isdigit(static_cast<unsigned char>(c)); });
  };
  static const std::set<std::string> loop_vars = {"i",  "j",  "k",  "r",  "u",   "io",  "ki",  "kc", "kl", "ks", "rr",
                                                  "tx", "ty", "bx", "bid", "row", "col", "kernel_args", "kernel_args_num",
                                                  "kernel_stream"};
  bool local = loop_vars.count(out) > 0;
  const size_t us = out.rfind('_');
  if (!local && us != std::string::npos && all_digits(out.substr(us + 1))) {
    static const std::set<std::string> hints = {"acc", "acc_idx", "t",  "o",  "base", "red", "rcp",  "r",  "q0",
                                                "n0",  "last",    "kv", "cv", "b",    "a",   "x",    "tile", "res"};
    local = hints.count(out.substr(0, us)) > 0;
  }
  if (!local && out.size() >= 3 && out[0] == 'm') {
    const size_t first_us = out.find('_');
    local = first_us != std::string::npos && all_digits(out.substr(1, first_us - 1));
  }
  if (local) out = "v_" + out;
  return out;
}

int EnvInt(const char* name, int dflt) {
  const char* v = getenv(name);
  if (!v || !*v) return dflt;
  return atoi(v);
}

ir::BindInfo BlockAxis(int axis) { return ir::BindInfo{ForType::GPUBlock, axis}; }
ir::BindInfo ThreadAxis(int axis) { return ir::BindInfo{ForType::GPUThread, axis}; }

// position inside a row-major tensor: either a flat offset, or per-dimension coordinates, or both
struct Index {
  Expr flat;
  std::vector<Expr> coords;
  bool identity{false};  // still the group's own iteration index (enables staged vector loads)
};

std::vector<Expr> Decompose(const Expr& flat, const ShapeType& shape) {
  std::vector<Expr> coords(shape.size());
  int64_t stride = 1;
  for (int i = static_cast<int>(shape.size()) - 1; i >= 0; --i) {
    if (shape[i] == 1) {
      coords[i] = I32(0);
    } else {
      Expr q = stride == 1 ? flat : flat / I32(stride);
      // the outermost non-unit dimension needs no modulo
      bool outermost = true;
      for (int j = 0; j < i; ++j) outermost &= (shape[j] == 1);
      coords[i] = outermost ? q : q % I32(shape[i]);
    }
    stride *= shape[i];
  }
  return coords;
}

Expr Compose(const std::vector<Expr>& coords, const ShapeType& shape) {
  Expr flat      = I32(0);
  int64_t stride = 1;
  for (int i = static_cast<int>(shape.size()) - 1; i >= 0; --i) {
    if (shape[i] != 1) flat = flat + coords[i] * I32(stride);
    stride *= shape[i];
  }
  return flat;
}

Expr FlatOf(const Index& idx, const ShapeType& shape) {
  if (idx.flat.defined()) return idx.flat;
  return Compose(idx.coords, shape);
}
std::vector<Expr> CoordsOf(const Index& idx, const ShapeType& shape) {
  if (!idx.coords.empty()) return idx.coords;
  return Decompose(idx.flat, shape);
}

// index of the operand of an index-transforming node, given the index into its output
Index TransformIndex(const Node& n, size_t input_slot, const Index& out_idx) {
  const ShapeType& out_shape = n.outputs[0]->shape;
  const ShapeType& in_shape  = n.inputs[input_slot]->shape;
  Index in;
  const std::string& op = n.op_type();
  if (op == "reshape") {
    in.flat     = FlatOf(out_idx, out_shape);
    in.identity = out_idx.identity;
    return in;
  }
  auto out_coords = CoordsOf(out_idx, out_shape);
  int out_rank    = static_cast<int>(out_shape.size());
  if (op == "broadcast_to") {
    auto axes = GetAttr<std::vector<int>>(n.attrs, "broadcast_axes", {});
    if (ShapeNumel(in_shape) == ShapeNumel(out_shape)) {
      // nothing is replicated: the flat position is unchanged
      in.flat     = FlatOf(out_idx, out_shape);
      in.identity = out_idx.identity;
      return in;
    }
    in.coords.resize(in_shape.size());
    for (size_t i = 0; i < in_shape.size(); ++i) {
      int ax       = axes[i] < 0 ? axes[i] + out_rank : axes[i];
      in.coords[i] = in_shape[i] == 1 ? I32(0) : out_coords[ax];
    }
    return in;
  }
  if (op == "transpose") {
    auto axis = GetAttr<std::vector<int>>(n.attrs, "axis", {});
    in.coords.resize(in_shape.size());
    for (size_t i = 0; i < axis.size(); ++i) {
      int ax        = axis[i] < 0 ? axis[i] + out_rank : axis[i];
      in.coords[ax] = out_coords[i];
    }
    return in;
  }
  if (op == "slice") {
    auto axes    = GetAttr<std::vector<int>>(n.attrs, "axes", {});
    auto starts  = GetAttr<std::vector<int>>(n.attrs, "starts", {});
    auto strides = GetAttr<std::vector<int>>(n.attrs, "strides", {});
    in.coords    = out_coords;
    for (size_t i = 0; i < axes.size(); ++i) {
      int ax  = axes[i] < 0 ? axes[i] + out_rank : axes[i];
      int dim = in_shape[ax];
      int s   = starts[i] < 0 ? starts[i] + dim : starts[i];
      s       = std::min(std::max(s, 0), dim);
      int st  = i < strides.size() ? strides[i] : 1;
      in.coords[ax] = out_coords[ax] * I32(st) + I32(s);
    }
    return in;
  }
  CINN_CHECK(false) << "no index transform for op " << op;
  return in;
}

// ---------------------------------------------------------------------------------------------------
// shared state of one group lowering
// ---------------------------------------------------------------------------------------------------
struct GroupContext {
  const Group& group;
  std::set<const NodeData*> produced;
  std::map<const NodeData*, BufferRef> global_bufs;
  ir::LoweredFuncRef func;
  int name_counter{0};

  explicit GroupContext(const Group& g) : group(g) {
    func       = std::make_shared<ir::LoweredFunc>();
    func->name = g.func_name;
    for (Node* n : g.nodes)
      for (auto* o : n->outputs) produced.insert(o);
    for (auto* v : g.inputs) AddArg(v, ir::Argument::IO::kInput);
    for (auto* v : g.outputs) AddArg(v, ir::Argument::IO::kOutput);
  }
  void AddArg(NodeData* v, ir::Argument::IO io) {
    CINN_CHECK_LT(v->numel(), static_cast<int64_t>(std::numeric_limits<int32_t>::max()))
        << "tensor " << v->id << " is too large for 32-bit indexing";
    auto buf = ir::MakeBuffer(CName(v->id), v->dtype, MemoryType::Global, v->numel());
    global_bufs[v] = buf;
    ir::Argument arg;
    arg.buffer = buf;
    arg.io     = io;
    func->args.push_back(arg);
  }
  bool IsOutput(const NodeData* v) const {
    return std::find(group.outputs.begin(), group.outputs.end(), v) != group.outputs.end();
  }
  BufferRef NewLocal(const std::string& hint, Type t, int64_t size, MemoryType m = MemoryType::GPULocal) {
    auto buf = ir::MakeBuffer(hint + "_" + std::to_string(name_counter++), t, m, size);
    func->temp_bufs.push_back(buf);
    return buf;
  }
  Expr NewVar(const std::string& hint, Type t) { return ir::MakeVar(hint + "_" + std::to_string(name_counter++), t); }
};

Expr ComputeElementwise(const Node& n, const std::vector<Expr>& inputs) {
  CINN_CHECK(n.op->compute) << "op " << n.op_type() << " has no scalar compute";
  return n.op->compute(inputs, n.attrs, n.outputs[0]->dtype);
}

// identity element of a reduction, values of the reference table
// (cinn/runtime/cuda/cinn_cuda_runtime_source.cuh:372-457)
Expr ReduceIdentity(const std::string& kind, const Type& t) {
  if (kind == "sum") return ir::MakeConst(t, 0);
  if (kind == "prod") return ir::MakeConst(t, 1);
  if (kind == "all") return Expr(true);
  if (kind == "any") return Expr(false);
  bool is_max = kind == "max";
  if (t.is_float(32)) return ir::MakeFloatImm(t, is_max ? -3.40282e+38 : 3.40282e+38);
  if (t.is_float(64)) return ir::MakeFloatImm(t, is_max ? -1.79769e+308 : 1.79769e+308);
  if (t.is_float16() || t.is_bfloat16()) {
    // raw patterns 0xfbff / 0x7bff
    return ir::MakeCall(t, t.is_float16() ? "cinn_hip_raw_to_fp16" : "cinn_hip_raw_to_bf16",
                        {ir::MakeIntImm(common::UInt(16), is_max ? 0xfbff : 0x7bff)});
  }
  if (t.is_int(32)) return ir::MakeIntImm(t, is_max ? std::numeric_limits<int32_t>::min() : std::numeric_limits<int32_t>::max());
  if (t.is_int(64)) return ir::MakeIntImm(t, is_max ? std::numeric_limits<int64_t>::min() : std::numeric_limits<int64_t>::max());
  CINN_CHECK(false) << "no " << kind << " identity for type " << common::Type2Str(t);
  return Expr();
}

// type a reduction accumulates in: 16-bit float sums / products run in fp32 and round once
Type AccumType(const std::string& kind, const Type& t) {
  if ((kind == "sum" || kind == "prod") && (t.is_float16() || t.is_bfloat16())) return common::Float(32);
  return t;
}

Expr Combine(const std::string& kind, const Expr& acc, const Expr& v) {
  if (kind == "sum") return acc + v;
  if (kind == "prod") return acc * v;
  if (kind == "max") return ir::Max(acc, v);
  if (kind == "min") return ir::Min(acc, v);
  if (kind == "all") return acc && v;
  if (kind == "any") return acc || v;
  CINN_CHECK(false) << "unknown reduce kind " << kind;
  return Expr();
}

std::string ReduceSuffix(const std::string& kind, const Type& t) {
  if (kind == "all" || kind == "any") return kind;
  return kind + "_" + common::TypeSuffix(t);
}

}  // namespace

LoweringOptions LoweringOptions::FromEnv() {
  LoweringOptions o;
  o.max_cached_elems_per_thread = EnvInt("FLAGS_cinn_hip_reduce_cached_elems", o.max_cached_elems_per_thread);
  o.wave_row_elems_per_lane     = EnvInt("FLAGS_cinn_hip_reduce_wave_elems", o.wave_row_elems_per_lane);
  o.block_row_elems_per_thread  = EnvInt("FLAGS_cinn_hip_reduce_block_elems", o.block_row_elems_per_thread);
  o.nontemporal_store_bytes     = static_cast<int64_t>(EnvInt("FLAGS_cinn_hip_nontemporal_store_mb", 8)) << 20;
  o.nontemporal_load_bytes      = static_cast<int64_t>(EnvInt("FLAGS_cinn_hip_nontemporal_load_mb", 0)) << 20;
  o.rows_per_wave               = EnvInt("FLAGS_cinn_hip_reduce_rows_per_wave", o.rows_per_wave);
  o.merged_rows_per_wave        = EnvInt("FLAGS_cinn_hip_merged_rows_per_wave", o.merged_rows_per_wave);
  o.elementwise_block           = EnvInt("FLAGS_cinn_hip_elementwise_block", o.elementwise_block);
  o.rows_per_block              = EnvInt("FLAGS_cinn_hip_reduce_rows_per_block", o.rows_per_block);
  o.column_reduce               = EnvInt("FLAGS_cinn_hip_column_reduce", 1) != 0;
  o.tiled_transpose             = EnvInt("FLAGS_cinn_hip_tiled_transpose", 1) != 0;
  o.sub_wave_rows               = EnvInt("FLAGS_cinn_hip_sub_wave_rows", 1) != 0;
  return o;
}

OpLowerer::OpLowerer(const common::Target& target, const LoweringOptions& options) : target_(target), options_(options) {
  CINN_CHECK(target.arch == common::Target::Arch::AMDGPU) << "this lowering targets AMDGPU only";
}

std::vector<NodeData*> OpLowerer::ArgumentsOf(const Group& group) {
  std::vector<NodeData*> args = group.inputs;
  args.insert(args.end(), group.outputs.begin(), group.outputs.end());
  return args;
}

ir::LoweredFuncRef OpLowerer::Lower(const Group& group, bool merged_member) const {
  switch (group.kind) {
    case GroupKind::kElementwise: return LowerElementwise(group);
    case GroupKind::kRowReduce: return LowerRowReduce(group, merged_member);
    case GroupKind::kGeneralReduce: return LowerGeneralReduce(group);
    case GroupKind::kLibraryCall: return LowerLibraryCall(group);
  }
  return nullptr;
}

// ---------------------------------------------------------------------------------------------------
// element-wise groups
// ---------------------------------------------------------------------------------------------------
namespace {

class ElementwiseEmitter {
 public:
  ElementwiseEmitter(GroupContext* ctx, std::vector<Expr>* stmts) : ctx_(ctx), stmts_(stmts) {}

  // values of group inputs that were staged into registers by a vector load: local buffer + lane
  std::map<const NodeData*, std::pair<BufferRef, Expr>> staged;
  // values that are already at hand at the identity index (a tile staged through LDS)
  std::map<const NodeData*, Expr> forced;

  Expr ValueAt(NodeData* v, const Index& idx) {
    if (idx.identity) {
      auto f = forced.find(v);
      if (f != forced.end()) return f->second;
      auto it = cache_.find(v);
      if (it != cache_.end()) return it->second;
    }
    Expr value;
    if (!ctx_->produced.count(v)) {
      auto st = staged.find(v);
      if (idx.identity && st != staged.end()) {
        value = ir::MakeLoad(st->second.first, st->second.second);
      } else {
        value = ir::MakeLoad(ctx_->global_bufs.at(v), FlatOf(idx, v->shape));
      }
    } else {
      Node* n = v->producer;
      if (n->op->pattern == OpPatternKind::kElementWise) {
        std::vector<Expr> inputs;
        for (auto* in : n->inputs) inputs.push_back(ValueAt(in, idx));
        value = ComputeElementwise(*n, inputs);
      } else if (n->op_type() == "concat") {
        value = Concat(*n, idx);
      } else {
        value = ValueAt(n->inputs[0], TransformIndex(*n, 0, idx));
      }
    }
    if (idx.identity) {
      // name the value once so that several consumers share it
      if (!value.is_constant() && !value.As<ir::Var>()) {
        Expr var = ctx_->NewVar("t", value.type());
        stmts_->push_back(ir::MakeLet(var, value));
        value = var;
      }
      cache_[v] = value;
    }
    return value;
  }

 private:
  Expr Concat(const Node& n, const Index& idx) {
    const ShapeType& out_shape = n.outputs[0]->shape;
    int axis = GetAttr<int>(n.attrs, "axis", 0);
    if (axis < 0) axis += static_cast<int>(out_shape.size());
    auto coords = CoordsOf(idx, out_shape);
    // walk the operands from the last to the first: select(c < offset_i, operand_{i-1}..., operand_i)
    std::vector<int> offsets;
    int off = 0;
    for (auto* in : n.inputs) {
      offsets.push_back(off);
      off += in->shape[axis];
    }
    Expr result;
    for (int i = static_cast<int>(n.inputs.size()) - 1; i >= 0; --i) {
      Index in;
      in.coords       = coords;
      in.coords[axis] = coords[axis] - I32(offsets[i]);
      Expr v          = ValueAt(n.inputs[i], in);
      if (!result.defined()) {
        result = v;
      } else {
        result = ir::MakeSelect(coords[axis] < I32(offsets[i + 1]), v, result);
      }
    }
    return result;
  }

  GroupContext* ctx_;
  std::vector<Expr>* stmts_;
  std::map<const NodeData*, Expr> cache_;
};

// True when every use of the group input `v` inside the group happens at the group's own flat index,
// i.e. it is reached from the outputs through element-wise ops, reshape and non-replicating
// broadcasts only.
bool UsedAtIdentityOnly(const Group& g, const NodeData* v, int64_t numel) {
  if (v->numel() != numel) return false;
  for (Node* n : g.nodes) {
    for (auto* in : n->inputs) {
      if (in != v) continue;
      if (n->op->pattern == OpPatternKind::kElementWise || n->op_type() == "reshape") continue;
      return false;
    }
  }
  return true;
}

}  // namespace

namespace {
void MarkStreamingInputs(GroupContext* ctx, int64_t threshold_bytes) {
  if (threshold_bytes <= 0) return;
  for (auto* v : ctx->group.inputs) {
    if (v->numel() * v->dtype.bytes() >= threshold_bytes) ctx->global_bufs.at(v)->streaming_load = true;
  }
}
void MarkStreamingOutputs(GroupContext* ctx, int64_t threshold_bytes) {
  if (threshold_bytes <= 0) return;
  for (auto* o : ctx->group.outputs) {
    if (o->numel() * o->dtype.bytes() >= threshold_bytes) ctx->global_bufs.at(o)->streaming_store = true;
  }
}
}  // namespace

// ---------------------------------------------------------------------------------------------------
// Element-wise group around one transpose that moves the innermost axis of a group input: the input is staged
// through LDS in TILE x TILE tiles over (output axis that holds the input's innermost axis, output's innermost
// axis), so that both the reads of the input and the writes of the outputs walk contiguous memory.  Without it
// consecutive threads read the input at the stride of the moved axis.  Every other operand of the group is at the
// group's own index.  Returns false when the group does not have this form.
// ---------------------------------------------------------------------------------------------------
namespace {
bool LowerTiledTranspose(const Group& group, GroupContext* ctx) {
  Node* t = nullptr;
  for (Node* n : group.nodes) {
    if (n->op_type() == "transpose") {
      if (t) return false;
      t = n;
    } else if (n->op->pattern != OpPatternKind::kElementWise) {
      return false;
    }
  }
  if (!t) return false;
  NodeData* x = t->inputs[0];
  if (ctx->produced.count(x)) return false;
  for (Node* n : group.nodes)
    for (auto* in : n->inputs)
      if (in == x && n != t) return false;
  const ShapeType& shape = t->outputs[0]->shape;
  const int rank         = static_cast<int>(shape.size());
  auto axis              = GetAttr<std::vector<int>>(t->attrs, "axis", {});
  if (rank < 2 || static_cast<int>(axis.size()) != rank) return false;
  for (auto& a : axis)
    if (a < 0) a += rank;
  if (axis[rank - 1] == rank - 1) return false;
  int q = -1;
  for (int i = 0; i < rank; ++i)
    if (axis[i] == rank - 1) q = i;
  if (q < 0) return false;
  const int64_t Q = shape[q], N = shape[rank - 1];
  if (Q < 16 || N < 16) return false;
  for (auto* o : group.outputs)
    if (o->shape != shape) return false;
  for (auto* v : group.inputs)
    if (v != x && v->shape != shape) return false;

  const int tile   = x->dtype.bytes() >= 4 ? 32 : 64;
  const int ty_n   = 256 / tile;
  const int per    = tile / ty_n;
  const int pitch  = tile + (x->dtype.bytes() >= 4 ? 1 : 2);  // odd number of 4-byte words per row
  const int64_t gq = (Q + tile - 1) / tile, gn = (N + tile - 1) / tile;
  ShapeType batch_shape;
  for (int i = 0; i < rank - 1; ++i)
    if (i != q) batch_shape.push_back(shape[i]);
  int64_t batch = 1;
  for (int d : batch_shape) batch *= d;
  if (batch * gq * gn >= static_cast<int64_t>(std::numeric_limits<int32_t>::max())) return false;
  const bool guard = Q % tile != 0 || N % tile != 0;

  Expr bid = ir::MakeVar("bid", common::Int(32));
  Expr tx  = ir::MakeVar("tx", common::Int(32));
  Expr ty  = ir::MakeVar("ty", common::Int(32));
  BufferRef lds = ctx->NewLocal("tile", x->dtype, static_cast<int64_t>(tile) * pitch, MemoryType::GPUShared);

  std::vector<Expr> stmts;
  Expr q0 = ctx->NewVar("q0", common::Int(32));
  Expr n0 = ctx->NewVar("n0", common::Int(32));
  Expr b  = ctx->NewVar("b", common::Int(32));
  stmts.push_back(ir::MakeLet(n0, (bid % I32(gn)) * I32(tile)));
  stmts.push_back(ir::MakeLet(q0, ((bid / I32(gn)) % I32(gq)) * I32(tile)));
  stmts.push_back(ir::MakeLet(b, bid / I32(gn * gq)));
  auto batch_coords = Decompose(b, batch_shape);
  auto coords_of    = [&](const Expr& qc, const Expr& nc) {
    std::vector<Expr> c(rank);
    for (int i = 0, k = 0; i < rank - 1; ++i)
      if (i != q) c[i] = batch_coords[k++];
    c[q]        = qc;
    c[rank - 1] = nc;
    return c;
  };
  {
    // phase 1: threads along the input's innermost axis
    Expr i  = ir::MakeVar("i", common::Int(32));
    Expr ln = ty + i * I32(ty_n);
    Index out_idx;
    out_idx.coords = coords_of(q0 + tx, n0 + ln);
    Index in_idx   = TransformIndex(*t, 0, out_idx);
    Expr copy = ir::MakeStore(lds, ir::MakeLoad(ctx->global_bufs.at(x), FlatOf(in_idx, x->shape)), ln * I32(pitch) + tx);
    if (guard) copy = ir::MakeIf(((q0 + tx) < I32(Q)) && ((n0 + ln) < I32(N)), copy);
    stmts.push_back(ir::MakeFor(i, I32(0), I32(per), ForType::Unrolled, copy));
  }
  stmts.push_back(ir::MakeCall(Type(), "__syncthreads", {}));
  {
    // phase 2: threads along the outputs' innermost axis
    Expr i  = ir::MakeVar("j", common::Int(32));
    Expr lq = ty + i * I32(ty_n);
    std::vector<Expr> body;
    ElementwiseEmitter emitter(ctx, &body);
    Index idx;
    idx.coords   = coords_of(q0 + lq, n0 + tx);
    Expr flat    = ctx->NewVar("o", common::Int(32));
    body.push_back(ir::MakeLet(flat, Compose(idx.coords, shape)));
    idx.flat     = flat;
    idx.identity = true;
    emitter.forced[t->outputs[0]] = ir::MakeLoad(lds, tx * I32(pitch) + lq);
    for (auto* o : group.outputs) {
      Expr value = emitter.ValueAt(o, idx);
      body.push_back(ir::MakeStore(ctx->global_bufs.at(o), value, flat));
    }
    Expr work = ir::MakeBlock(body);
    if (guard) work = ir::MakeIf(((q0 + lq) < I32(Q)) && ((n0 + tx) < I32(N)), work);
    stmts.push_back(ir::MakeFor(i, I32(0), I32(per), ForType::Unrolled, work));
  }
  Expr threads_x  = ir::MakeFor(tx, I32(0), I32(tile), ForType::Serial, ir::MakeBlock(stmts), ThreadAxis(0));
  Expr threads_y  = ir::MakeFor(ty, I32(0), I32(ty_n), ForType::Serial, threads_x, ThreadAxis(1));
  ctx->func->body = ir::MakeFor(bid, I32(0), I32(batch * gq * gn), ForType::Serial, threads_y, BlockAxis(0));
  return true;
}
}  // namespace

ir::LoweredFuncRef OpLowerer::LowerElementwise(const Group& group) const {
  GroupContext ctx(group);
  if (options_.tiled_transpose && LowerTiledTranspose(group, &ctx)) return ctx.func;
  MarkStreamingOutputs(&ctx, options_.nontemporal_store_bytes);
  MarkStreamingInputs(&ctx, options_.nontemporal_load_bytes);
  CINN_CHECK(!group.outputs.empty());
  const int64_t numel = group.outputs[0]->numel();
  for (auto* o : group.outputs) CINN_CHECK_EQ(o->numel(), numel) << "outputs of an element-wise group differ in size";
  CINN_CHECK_GT(numel, 0);

  // vector width: 16 bytes of the narrowest tensor that is accessed at the identity index
  int min_bytes = 16;
  std::vector<NodeData*> identity_inputs;
  for (auto* v : group.inputs) {
    if (UsedAtIdentityOnly(group, v, numel)) {
      identity_inputs.push_back(v);
      min_bytes = std::min(min_bytes, v->dtype.bytes());
    }
  }
  for (auto* v : group.outputs) min_bytes = std::min(min_bytes, v->dtype.bytes());
  int vec = std::max(1, std::min(16 / min_bytes, 8));
  while (vec > 1 && numel % vec != 0) vec /= 2;
  // an output that is not produced at the identity index of the flat space cannot exist here (all
  // outputs have `numel` elements and are indexed by the flat index)
  const int block   = options_.elementwise_block;
  int64_t num_vec   = numel / vec;
  // vectors per thread: keep at least ~8 blocks per compute unit in flight
  int per_thread    = 1;
  int64_t min_blocks = static_cast<int64_t>(target_.get_multi_processor_count()) * 8;
  while (per_thread < 4 && num_vec / (static_cast<int64_t>(block) * per_thread * 2) >= min_blocks) per_thread *= 2;
  int64_t per_block = static_cast<int64_t>(block) * per_thread;
  int64_t grid      = (num_vec + per_block - 1) / per_block;
  bool need_guard   = (num_vec % per_block) != 0;

  Expr bx = ir::MakeVar("bx", common::Int(32));
  Expr tx = ir::MakeVar("tx", common::Int(32));
  Expr u  = ir::MakeVar("u", common::Int(32));
  Expr k  = ir::MakeVar("k", common::Int(32));

  Expr vec_index = bx * I32(per_block) + u * I32(block) + tx;
  Expr base      = ctx.NewVar("base", common::Int(32));

  std::vector<Expr> body;  // statements of one vector
  body.push_back(ir::MakeLet(base, vec_index * I32(vec)));

  std::vector<Expr> compute;  // statements of the per-lane loop
  ElementwiseEmitter emitter(&ctx, &compute);
  // staged loads of identity inputs
  for (auto* v : identity_inputs) {
    BufferRef local = ctx.NewLocal(CName(v->id) + "_reg", v->dtype, vec);
    Expr kk         = ir::MakeVar("kl", common::Int(32));
    body.push_back(ir::MakeFor(kk, I32(0), I32(vec), ForType::Vectorized,
                               ir::MakeStore(local, ir::MakeLoad(ctx.global_bufs.at(v), base + kk), kk)));
    emitter.staged[v] = {local, k};
  }
  Index idx;
  idx.flat     = base + k;
  idx.identity = true;
  std::vector<std::pair<NodeData*, BufferRef>> out_regs;
  for (auto* o : group.outputs) {
    Expr value      = emitter.ValueAt(o, idx);
    BufferRef local = ctx.NewLocal(CName(o->id) + "_reg", o->dtype, vec);
    compute.push_back(ir::MakeStore(local, value, k));
    out_regs.push_back({o, local});
  }
  body.push_back(ir::MakeFor(k, I32(0), I32(vec), ForType::Unrolled, ir::MakeBlock(compute)));
  for (auto& kv : out_regs) {
    Expr kk = ir::MakeVar("ks", common::Int(32));
    body.push_back(ir::MakeFor(kk, I32(0), I32(vec), ForType::Vectorized,
                               ir::MakeStore(ctx.global_bufs.at(kv.first), ir::MakeLoad(kv.second, kk), base + kk)));
  }
  Expr one_vec = ir::MakeBlock(body);
  if (need_guard) one_vec = ir::MakeIf(vec_index < I32(num_vec), one_vec);
  Expr per_thread_loop = ir::MakeFor(u, I32(0), I32(per_thread), ForType::Unrolled, one_vec);
  Expr threads = ir::MakeFor(tx, I32(0), I32(block), ForType::Serial, per_thread_loop, ThreadAxis(0));
  ctx.func->body = ir::MakeFor(bx, I32(0), I32(grid), ForType::Serial, threads, BlockAxis(0));
  return ctx.func;
}

// ---------------------------------------------------------------------------------------------------
// row-reduce groups
// ---------------------------------------------------------------------------------------------------
namespace {

struct RowReducePlan {
  int64_t rows, cols;
  int team;            // threads that share a row: a power of two up to 32 lanes, 64 (one wavefront) or the whole block
  int rows_per_block;  // > 1 only when team <= 64
  int vec;             // elements per vector access
  int chunks;          // vectors per thread and row
  bool guard_cols;     // cols is not a multiple of team * vec
  bool cached;         // the row stays in registers across phases
};

class RowReduceEmitter {
 public:
  RowReduceEmitter(GroupContext* ctx, const RowReducePlan& plan, std::map<const NodeData*, RowKind> kinds)
      : ctx_(ctx), plan_(plan), kinds_(std::move(kinds)) {
    row_ = ir::MakeVar("row", common::Int(32));
    tx_  = ir::MakeVar("tx", common::Int(32));
    j_   = ir::MakeVar("j", common::Int(32));
    k_   = ir::MakeVar("k", common::Int(32));
    col_ = ir::MakeVar("col", common::Int(32));
    ComputePhases();
    // Column operands (gamma / beta of a layer norm) that only later phases use are requested in the first phase,
    // together with the row itself, and kept in registers: otherwise their latency is paid after the reductions,
    // once more per row.  Budget: 64 registers per lane for all of them.
    if (plan_.cached && num_phases_ > 1) {
      int64_t dwords = 0;
      for (auto& kv : kinds_) {
        if (kv.second != RowKind::kCol || ctx_->produced.count(kv.first)) continue;
        dwords += (static_cast<int64_t>(plan_.chunks) * plan_.vec * kv.first->dtype.bytes() + 3) / 4;
        prefetched_cols_.push_back(const_cast<NodeData*>(kv.first));
      }
      static const bool enabled = EnvInt("FLAGS_cinn_hip_prefetch_columns", 1) != 0;
      if (!enabled || dwords > 64) prefetched_cols_.clear();
      std::sort(prefetched_cols_.begin(), prefetched_cols_.end(),
                [](const NodeData* a, const NodeData* b) { return a->id < b->id; });
    }
  }

  Expr row() const { return row_; }
  Expr tx() const { return tx_; }

  // statements executed by every thread of a team for its row
  std::vector<Expr> EmitRowBody() {
    std::vector<Expr> out;
    row_stmts_ = &out;
    for (int p = 0; p < num_phases_; ++p) {
      EmitRowValues(p);
      EmitPhaseLoop(p);
    }
    EmitRowValues(num_phases_);
    return out;
  }

 private:
  RowKind KindOf(const NodeData* v) const {
    auto it = kinds_.find(v);
    CINN_CHECK(it != kinds_.end()) << "value " << v->id << " has no row kind";
    return it->second;
  }
  bool IsElem(const NodeData* v) const { return KindOf(v) == RowKind::kElem; }

  void ComputePhases() {
    num_phases_ = 1;
    auto phase_of = [&](const NodeData* v) {
      auto it = phase_.find(v);
      return it == phase_.end() ? 0 : it->second;
    };
    for (Node* n : ctx_->group.nodes) {
      int p = 0;
      for (auto* in : n->inputs) p = std::max(p, phase_of(in));
      if (n->op->pattern == OpPatternKind::kReduction) {
        num_phases_ = std::max(num_phases_, p + 1);
        p += 1;
      }
      for (auto* o : n->outputs) phase_[o] = p;
    }
    for (auto* o : ctx_->group.outputs)
      if (IsElem(o)) num_phases_ = std::max(num_phases_, phase_of(o) + 1);
    // values that cross a phase boundary are kept in registers (cached mode only)
    if (plan_.cached) {
      for (Node* n : ctx_->group.nodes) {
        if (n->op->pattern == OpPatternKind::kReduction) continue;
        for (auto* in : n->inputs) {
          if (!IsElem(in) || !ctx_->produced.count(in)) continue;
          if (!in->producer->op->compute || in->producer->op_type() == "fill_constant") continue;
          if (phase_of(n->outputs[0]) > phase_of(in)) materialize_.insert(in);
        }
      }
    }
  }
  int PhaseOf(const NodeData* v) const {
    auto it = phase_.find(v);
    return it == phase_.end() ? 0 : it->second;
  }

  // ---- per-row scalars ----------------------------------------------------------------------------
  Expr RowValue(NodeData* v) {
    auto it = row_values_.find(v);
    if (it != row_values_.end()) return it->second;
    Expr value;
    RowKind kind = KindOf(v);
    if (!ctx_->produced.count(v)) {
      Expr index = kind == RowKind::kRow ? row_ : I32(0);
      if (plan_.rows == 1) index = I32(0);
      value = ir::MakeLoad(ctx_->global_bufs.at(v), index);
    } else {
      Node* n = v->producer;
      CINN_CHECK(n->op->pattern != OpPatternKind::kReduction) << "reduce result " << v->id << " used before its phase";
      if (n->op->pattern == OpPatternKind::kElementWise) {
        std::vector<Expr> inputs;
        for (auto* in : n->inputs) inputs.push_back(RowValue(in));
        value = ComputeElementwise(*n, inputs);
      } else {
        value = RowValue(n->inputs[0]);  // reshape / broadcast_to among per-row values
      }
    }
    if (!value.is_constant() && !value.As<ir::Var>()) {
      Expr var = ctx_->NewVar("r", value.type());
      row_stmts_->push_back(ir::MakeLet(var, value));
      value = var;
    }
    row_values_[v] = value;
    return value;
  }

  // per-row values that become available before phase loop p (or after the last loop), and per-row
  // outputs
  void EmitRowValues(int p) {
    for (Node* n : ctx_->group.nodes) {
      if (n->op->pattern == OpPatternKind::kReduction) continue;
      for (auto* o : n->outputs) {
        RowKind kind = KindOf(o);
        if (kind != RowKind::kRow && kind != RowKind::kScalar) continue;
        if (PhaseOf(o) != p) continue;
        RowValue(o);
      }
    }
    for (auto* o : ctx_->group.outputs) {
      RowKind kind = KindOf(o);
      if (kind != RowKind::kRow && kind != RowKind::kScalar) continue;
      if (PhaseOf(o) != p || stored_rows_.count(o)) continue;
      stored_rows_.insert(o);
      Expr value = RowValue(o);
      Expr index = (kind == RowKind::kRow && plan_.rows != 1) ? row_ : I32(0);
      row_stmts_->push_back(
          ir::MakeIf(tx_ == I32(0), ir::MakeStore(ctx_->global_bufs.at(o), value, index)));
    }
  }

  // ---- element values -----------------------------------------------------------------------------
  Expr LaneSlot() const { return plan_.cached ? j_ * I32(plan_.vec) + k_ : k_; }

  // pieces of at most 16 bytes that make up one chunk of `vec` elements of type t
  void EmitChunkCopy(std::vector<Expr>* out, const BufferRef& dst, const Expr& dst_base, const BufferRef& src,
                     const Expr& src_base, const Type& t) {
    int piece  = std::max(1, std::min(plan_.vec, 16 / t.bytes()));
    int pieces = plan_.vec / piece;
    for (int p = 0; p < pieces; ++p) {
      Expr kk = ctx_->NewVar("kv", common::Int(32));
      out->push_back(ir::MakeFor(kk, I32(0), I32(piece), ForType::Vectorized,
                                 ir::MakeStore(dst, ir::MakeLoad(src, src_base + I32(p * piece) + kk),
                                               dst_base + I32(p * piece) + kk)));
    }
  }

  // Register copy of a group input for the current chunk.  A row operand (kind Elem) in cached mode
  // owns registers for the whole row and is loaded in the first phase that needs it; a column
  // vector, or any operand in streaming mode, is re-read in every phase that uses it.
  Expr StagedInput(NodeData* v, bool is_col) {
    auto& slot      = stage_[v];
    bool persistent = plan_.cached && (!is_col || std::find(prefetched_cols_.begin(), prefetched_cols_.end(), v) != prefetched_cols_.end());
    if (!slot.buffer) {
      int64_t size = persistent ? static_cast<int64_t>(plan_.chunks) * plan_.vec : plan_.vec;
      slot.buffer  = ctx_->NewLocal(CName(v->id) + "_reg", v->dtype, size);
    }
    bool need_load = persistent ? slot.loaded_phase < 0 : !slot.emitted_in.count(cur_phase_);
    if (need_load) {
      Expr src_base = is_col ? col_ : row_ * I32(plan_.cols) + col_;
      Expr dst_base = persistent ? j_ * I32(plan_.vec) : I32(0);
      EmitChunkCopy(chunk_loads_, slot.buffer, dst_base, ctx_->global_bufs.at(v), src_base, v->dtype);
      slot.emitted_in.insert(cur_phase_);
      slot.loaded_phase = cur_phase_;
    }
    return ir::MakeLoad(slot.buffer, persistent ? LaneSlot() : k_);
  }

  Expr ElemValue(NodeData* v) {
    auto it = elem_cache_.find(v);
    if (it != elem_cache_.end()) return it->second;
    Expr value;
    if (!ctx_->produced.count(v)) {
      value = StagedInput(v, false);
    } else if (materialized_buf_.count(v) && materialized_phase_.at(v) < cur_phase_) {
      value = ir::MakeLoad(materialized_buf_.at(v), LaneSlot());
    } else {
      Node* n = v->producer;
      if (n->op_type() == "divide" && v->dtype.is_floating() && RowDivisor(n->inputs[1]) && !ExactDivision()) {
        // x / (per-row value) -> x * (1 / per-row value): the reciprocal is taken once per row with a
        // correctly rounded division, so the result stays within 1 ulp of the quotient while the
        // per-element cost drops from a division sequence to one multiply
        Expr rcp = RowReciprocal(RowDivisor(n->inputs[1]));
        Expr a   = ElemValue(n->inputs[0]);
        value    = ir::MakeCast(v->dtype, ir::MakeCast(rcp.type(), a) * rcp);
      } else if (n->op->pattern == OpPatternKind::kElementWise) {
        std::vector<Expr> inputs;
        for (auto* in : n->inputs) {
          RowKind kind = KindOf(in);
          inputs.push_back(kind == RowKind::kElem ? ElemValue(in) : RowValue(in));
        }
        value = ComputeElementwise(*n, inputs);
      } else if (n->op_type() == "broadcast_to") {
        NodeData* in = n->inputs[0];
        switch (KindOf(in)) {
          case RowKind::kElem: value = ElemValue(in); break;
          case RowKind::kCol: value = StagedInput(in, true); break;
          default: value = RowValue(in);
        }
      } else {  // reshape
        value = ElemValue(n->inputs[0]);
      }
      if (!value.is_constant() && !value.As<ir::Var>()) {
        Expr var = ctx_->NewVar("t", value.type());
        lane_stmts_->push_back(ir::MakeLet(var, value));
        value = var;
      }
      if (materialize_.count(v) && PhaseOf(v) == cur_phase_ && !materialized_buf_.count(v)) {
        BufferRef buf = ctx_->NewLocal(CName(v->id) + "_keep", v->dtype, static_cast<int64_t>(plan_.chunks) * plan_.vec);
        lane_stmts_->push_back(ir::MakeStore(buf, value, LaneSlot()));
        materialized_buf_[v]   = buf;
        materialized_phase_[v] = cur_phase_;
      }
    }
    elem_cache_[v] = value;
    return value;
  }

  static bool ExactDivision() { return EnvInt("FLAGS_cinn_hip_exact_division", 0) != 0; }

  // the per-row value an element operand replicates, looking through reshape / broadcast_to
  NodeData* RowDivisor(NodeData* v) const {
    while (ctx_->produced.count(v)) {
      Node* n = v->producer;
      if (n->op_type() != "broadcast_to" && n->op_type() != "reshape") return nullptr;
      v = n->inputs[0];
      RowKind kind = KindOf(v);
      if (kind == RowKind::kRow || kind == RowKind::kScalar) return v;
      if (kind != RowKind::kElem) return nullptr;
    }
    return nullptr;
  }
  Expr RowReciprocal(NodeData* row_var) {
    auto it = row_rcp_.find(row_var);
    if (it != row_rcp_.end()) return it->second;
    Expr b      = RowValue(row_var);
    Type wide   = b.type().bits < 32 ? common::Float(32) : b.type();
    Expr var    = ctx_->NewVar("rcp", wide);
    row_stmts_->push_back(ir::MakeLet(var, ir::MakeConst(wide, 1) / ir::MakeCast(wide, b)));
    row_rcp_[row_var] = var;
    return var;
  }

  struct Accumulator {
    Node* node;
    std::string kind;
    Type acc_type;
    BufferRef value;  // size-1 register buffer
    BufferRef index;  // arg-reduce only
  };

  void EmitPhaseLoop(int p) {
    cur_phase_ = p;
    elem_cache_.clear();
    std::vector<Expr> chunk_loads, lane_stmts, chunk_stores;
    chunk_loads_ = &chunk_loads;
    lane_stmts_  = &lane_stmts;

    // reductions whose operand is complete in this phase
    std::vector<Accumulator> accs;
    for (Node* n : ctx_->group.nodes) {
      if (n->op->pattern != OpPatternKind::kReduction || PhaseOf(n->inputs[0]) != p) continue;
      Accumulator a;
      a.node             = n;
      a.kind             = n->op->reduce_kind;
      const Type in_type = n->inputs[0]->dtype;
      bool is_arg        = a.kind == "argmax" || a.kind == "argmin";
      a.acc_type         = is_arg ? in_type : AccumType(a.kind, in_type);
      a.value            = ctx_->NewLocal("acc", a.acc_type, 1);
      if (is_arg) {
        a.index = ctx_->NewLocal("acc_idx", common::Int(32), 1);
        row_stmts_->push_back(ir::MakeStore(a.value, ir::MakeConst(a.acc_type, 0), I32(0)));
        row_stmts_->push_back(ir::MakeStore(a.index, I32(-1), I32(0)));
      } else {
        row_stmts_->push_back(ir::MakeStore(a.value, ir::MakeCast(a.acc_type, ReduceIdentity(a.kind, a.acc_type)), I32(0)));
      }
      accs.push_back(a);
    }
    for (auto& a : accs) {
      Expr v   = ElemValue(a.node->inputs[0]);
      Expr cur = ir::MakeLoad(a.value, I32(0));
      if (a.index) {
        Expr cur_idx = ir::MakeLoad(a.index, I32(0));
        Expr better  = a.kind == "argmax" ? (v > cur) : (v < cur);
        Expr pos     = col_ + k_;
        lane_stmts.push_back(ir::MakeIf((cur_idx < I32(0)) || better,
                                        ir::MakeBlock({ir::MakeStore(a.value, v, I32(0)), ir::MakeStore(a.index, pos, I32(0))})));
      } else {
        lane_stmts.push_back(ir::MakeStore(a.value, Combine(a.kind, cur, ir::MakeCast(a.acc_type, v)), I32(0)));
      }
    }
    // column operands of later phases, requested now
    if (p == 0 && !accs.empty())
      for (NodeData* v : prefetched_cols_) StagedInput(v, true);
    // values that later phases need (cached mode)
    for (Node* n : ctx_->group.nodes) {
      for (auto* v : n->outputs)
        if (materialize_.count(v) && PhaseOf(v) == p) ElemValue(v);
    }
    // element outputs that are complete in this phase
    for (auto* o : ctx_->group.outputs) {
      if (!IsElem(o) || PhaseOf(o) != p) continue;
      Expr value    = ElemValue(o);
      BufferRef reg = ctx_->NewLocal(CName(o->id) + "_out", o->dtype, plan_.vec);
      lane_stmts.push_back(ir::MakeStore(reg, value, k_));
      EmitChunkCopy(&chunk_stores, ctx_->global_bufs.at(o), row_ * I32(plan_.cols) + col_, reg, I32(0), o->dtype);
    }

    if (!lane_stmts.empty()) {
      std::vector<Expr> chunk;
      chunk.push_back(ir::MakeLet(col_, (j_ * I32(plan_.team) + tx_) * I32(plan_.vec)));
      std::vector<Expr> guarded = chunk_loads;
      guarded.push_back(ir::MakeFor(k_, I32(0), I32(plan_.vec), ForType::Unrolled, ir::MakeBlock(lane_stmts)));
      guarded.insert(guarded.end(), chunk_stores.begin(), chunk_stores.end());
      if (plan_.guard_cols) {
        chunk.push_back(ir::MakeIf(col_ < I32(plan_.cols), ir::MakeBlock(guarded)));
      } else {
        chunk.insert(chunk.end(), guarded.begin(), guarded.end());
      }
      row_stmts_->push_back(ir::MakeFor(j_, I32(0), I32(plan_.chunks), plan_.cached ? ForType::Unrolled : ForType::Serial,
                                        ir::MakeBlock(chunk)));
    }

    // team reductions: every thread of the team gets the result
    for (auto& a : accs) {
      NodeData* out = a.node->outputs[0];
      bool wave     = plan_.team == 64;
      bool sub_wave = plan_.team < 64;  // several rows per wavefront
      Expr result;
      if (a.index) {
        std::string fn = std::string(sub_wave ? "cinn_team_" : wave ? "cinn_wave_" : "cinn_block_") + a.kind;
        std::vector<Expr> args = {ir::MakeLoad(a.value, I32(0)), ir::MakeLoad(a.index, I32(0))};
        if (sub_wave) args.push_back(I32(plan_.team));
        result = ir::MakeCall(common::Int(32), fn, args);
      } else {
        std::string suffix = ReduceSuffix(a.kind, a.acc_type);
        std::string fn     = sub_wave ? "cinn_team_shuffle_" + suffix + "_internal"
                             : wave   ? "cinn_wave_shuffle_" + suffix + "_internal"
                                      : "cinn_block_reduce_" + suffix + "_internal";
        std::vector<Expr> args = {ir::MakeLoad(a.value, I32(0))};
        if (sub_wave) args.push_back(I32(plan_.team));
        result = ir::MakeCast(out->dtype, ir::MakeCall(a.acc_type, fn, args));
      }
      Expr var = ctx_->NewVar("red", out->dtype);
      row_stmts_->push_back(ir::MakeLet(var, result));
      row_values_[out] = var;
    }
    chunk_loads_ = nullptr;
    lane_stmts_  = nullptr;
  }

  struct Stage {
    BufferRef buffer;
    int loaded_phase{-1};
    std::set<int> emitted_in;
  };

  GroupContext* ctx_;
  RowReducePlan plan_;
  std::map<const NodeData*, RowKind> kinds_;
  std::map<const NodeData*, int> phase_;
  std::set<const NodeData*> materialize_;
  int num_phases_{1};
  Expr row_, tx_, j_, k_, col_;

  std::vector<Expr>* row_stmts_{nullptr};
  std::vector<Expr>* chunk_loads_{nullptr};
  std::vector<Expr>* lane_stmts_{nullptr};
  int cur_phase_{0};
  std::map<const NodeData*, Expr> row_values_;
  std::map<const NodeData*, Expr> row_rcp_;
  std::set<const NodeData*> stored_rows_;
  std::map<const NodeData*, Expr> elem_cache_;
  std::map<const NodeData*, Stage> stage_;
  std::vector<NodeData*> prefetched_cols_;
  std::map<const NodeData*, BufferRef> materialized_buf_;
  std::map<const NodeData*, int> materialized_phase_;
};

}  // namespace

ir::LoweredFuncRef OpLowerer::LowerRowReduce(const Group& group, bool merged_member) const {
  GroupContext ctx(group);
  MarkStreamingOutputs(&ctx, options_.nontemporal_store_bytes);
  MarkStreamingInputs(&ctx, options_.nontemporal_load_bytes);
  std::map<const NodeData*, RowKind> kinds;
  CINN_CHECK(ClassifyRowReduceGroup(group.nodes, group.rows, group.cols, &kinds))
      << "group " << group.func_name << " is not a row-reduce group";

  RowReducePlan plan;
  plan.rows = group.rows;
  plan.cols = group.cols;
  CINN_CHECK_LT(plan.rows * plan.cols, static_cast<int64_t>(std::numeric_limits<int32_t>::max()));

  // vector width from the narrowest tensor that is walked along the row
  int min_bytes = 16;
  for (auto& kv : kinds) {
    bool global = !ctx.produced.count(kv.first) || ctx.IsOutput(kv.first);
    if (!global) continue;
    if (kv.second == RowKind::kElem || kv.second == RowKind::kCol) min_bytes = std::min(min_bytes, kv.first->dtype.bytes());
  }
  plan.vec = std::max(1, std::min(16 / min_bytes, 8));
  while (plan.vec > 1 && plan.cols % plan.vec != 0) plan.vec /= 2;

  const int wave = target_.wavefront_size();
  CINN_CHECK_EQ(wave, 64) << "the row-reduce template is written for 64-lane wavefronts";
  int64_t per_lane       = (plan.cols + wave - 1) / wave;
  const int64_t row_vecs = (plan.cols + plan.vec - 1) / plan.vec;
  if (options_.sub_wave_rows && row_vecs <= wave / 2) {
    // short rows: a team of the fewest lanes that hold the row with one vector each, 64 / team rows per wavefront
    int team = 1;
    while (team < row_vecs) team *= 2;
    plan.team           = team;
    plan.rows_per_block = 256 / team;
  } else if (per_lane <= options_.wave_row_elems_per_lane) {
    plan.team           = wave;
    plan.rows_per_block = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(options_.rows_per_block, plan.rows)));
  } else {
    // whole block per row: the smallest power-of-two block (up to 1024 threads) that keeps the row
    // within the register budget
    int team = 128;
    while (team < target_.max_num_threads() && (plan.cols + team - 1) / team > options_.block_row_elems_per_thread) {
      team *= 2;
    }
    plan.team           = team;
    plan.rows_per_block = 1;
  }
  int64_t span    = static_cast<int64_t>(plan.team) * plan.vec;
  plan.chunks     = static_cast<int>((plan.cols + span - 1) / span);
  plan.guard_cols = (plan.cols % span) != 0;
  plan.cached     = static_cast<int64_t>(plan.chunks) * plan.vec <= options_.max_cached_elems_per_thread;

  RowReduceEmitter emitter(&ctx, plan, kinds);
  std::vector<Expr> row_body = emitter.EmitRowBody();

  // short rows: let a wavefront work through several rows so that more loads are in flight per lane
  int rows_per_wave = 1;
  if (plan.team == wave) {
    rows_per_wave = std::max(1, options_.rows_per_wave);
    if (merged_member && rows_per_wave == 1 && options_.merged_rows_per_wave > 1) {
      // A member of a merged launch runs at the occupancy the heaviest member's registers allow.  Wavefronts that
      // request at most 32 bytes per lane for a row and leave then have too few bytes in flight per CU: such rows are
      // taken several per wavefront.
      int64_t row_bytes = 0;  // what a lane requests per row
      for (auto& kv : kinds)
        if (!ctx.produced.count(kv.first) && kv.second == RowKind::kElem) row_bytes += per_lane * kv.first->dtype.bytes();
      while (rows_per_wave * 2 <= options_.merged_rows_per_wave && row_bytes * rows_per_wave * 2 <= 64 &&
             plan.rows % (static_cast<int64_t>(plan.rows_per_block) * rows_per_wave * 2) == 0)
        rows_per_wave *= 2;
    }
  }
  Expr bx = ir::MakeVar("bx", common::Int(32));
  Expr ty = ir::MakeVar("ty", common::Int(32));
  Expr rr = ir::MakeVar("rr", common::Int(32));
  int64_t rows_per_group = static_cast<int64_t>(plan.rows_per_block) * rows_per_wave;
  int64_t grid           = (plan.rows + rows_per_group - 1) / rows_per_group;
  Expr wave_index        = plan.rows_per_block > 1 ? bx * I32(plan.rows_per_block) + ty : bx;
  Expr row_index         = rows_per_wave > 1 ? wave_index * I32(rows_per_wave) + rr : wave_index;

  std::vector<Expr> per_row;
  per_row.push_back(ir::MakeLet(emitter.row(), row_index));
  Expr work = ir::MakeBlock(row_body);
  if (plan.rows % rows_per_group != 0) work = ir::MakeIf(emitter.row() < I32(plan.rows), work);
  per_row.push_back(work);
  Expr per_thread = ir::MakeBlock(per_row);
  if (rows_per_wave > 1) per_thread = ir::MakeFor(rr, I32(0), I32(rows_per_wave), ForType::Unrolled, per_thread);

  Expr body = ir::MakeFor(emitter.tx(), I32(0), I32(plan.team), ForType::Serial, per_thread, ThreadAxis(0));
  if (plan.rows_per_block > 1) body = ir::MakeFor(ty, I32(0), I32(plan.rows_per_block), ForType::Serial, body, ThreadAxis(1));
  ctx.func->body = ir::MakeFor(bx, I32(0), I32(grid), ForType::Serial, body, BlockAxis(0));
  return ctx.func;
}

// ---------------------------------------------------------------------------------------------------
// Reduction over one non-trailing run of axes: the input is [a][r][c] with r reduced.  A block is TX x TY
// threads: x walks the kept, contiguous axis c in vectors of 16 bytes (a wavefront reads whole rows or row
// segments), y strides over r; every thread keeps one accumulator per vector lane, rows are fetched four at a time
// so that several loads are in flight, and the TY partial results of a column meet in LDS
// (cinn_block_column_reduce_*).  Grid: a x ceil(c / (vec * TX)) blocks.  The reference assigns such reductions
// in LoopAssignReduceWithoutLast (cinn/hlir/framework/op_lowering_util.cc:485-640).
// ---------------------------------------------------------------------------------------------------
namespace {

void EmitColumnReduce(GroupContext* ctx, const common::Target& target, NodeData* in, NodeData* out,
                      const std::string& kind, int64_t a, int64_t r, int64_t c) {
  const Type acc_type = AccumType(kind, in->dtype);
  int vec             = std::max(1, std::min(16 / in->dtype.bytes(), 8));
  while (vec > 1 && c % vec != 0) vec /= 2;
  CINN_CHECK(vec <= (acc_type.bytes() >= 8 ? 2 : 8)) << "the LDS exchange of the column reduce holds 8 values per thread";
  const int64_t cv = c / vec;
  int tx_n         = 1;
  while (tx_n < 64 && tx_n < cv) tx_n *= 2;
  int ty_n = 256 / tx_n;
  while (ty_n > 1 && ty_n / 2 >= r) ty_n /= 2;
  const int64_t grid_c  = (cv + tx_n - 1) / tx_n;
  const bool col_guard  = cv % tx_n != 0;
  const int64_t full    = r / ty_n;  // rows every thread takes without a bound check
  const int unroll      = full >= 8 ? 4 : 1;
  const int64_t main_it = full / unroll;
  CINN_CHECK_LT(a * grid_c, static_cast<int64_t>(std::numeric_limits<int32_t>::max()));

  Expr bid = ir::MakeVar("bid", common::Int(32));
  Expr tx  = ir::MakeVar("tx", common::Int(32));
  Expr ty  = ir::MakeVar("ty", common::Int(32));
  Expr k   = ir::MakeVar("k", common::Int(32));
  BufferRef src = ctx->global_bufs.at(in);
  BufferRef dst = ctx->global_bufs.at(out);

  std::vector<Expr> stmts;
  Expr ai   = ctx->NewVar("a", common::Int(32));
  Expr cvi  = ctx->NewVar("cv", common::Int(32));
  Expr base = ctx->NewVar("base", common::Int(32));
  stmts.push_back(ir::MakeLet(ai, bid / I32(grid_c)));
  stmts.push_back(ir::MakeLet(cvi, (bid % I32(grid_c)) * I32(tx_n) + tx));
  stmts.push_back(ir::MakeLet(base, ai * I32(r * c) + cvi * I32(vec)));

  BufferRef acc = ctx->NewLocal("acc", acc_type, vec);
  {
    Expr ki = ir::MakeVar("ki", common::Int(32));
    stmts.push_back(ir::MakeFor(ki, I32(0), I32(vec), ForType::Unrolled,
                                ir::MakeStore(acc, ir::MakeCast(acc_type, ReduceIdentity(kind, acc_type)), ki)));
  }
  // one row: a 16-byte load into registers, then the lane-wise combine
  auto row = [&](const Expr& row_index, int slot) {
    BufferRef reg = ctx->NewLocal("x" + std::to_string(slot), in->dtype, vec);
    Expr kl       = ir::MakeVar("kl", common::Int(32));
    Expr kc       = ir::MakeVar("kc", common::Int(32));
    Expr offset   = base + row_index * I32(c);
    Expr load     = ir::MakeFor(kl, I32(0), I32(vec), ForType::Vectorized,
                                ir::MakeStore(reg, ir::MakeLoad(src, offset + kl), kl));
    Expr combine  = ir::MakeFor(
        kc, I32(0), I32(vec), ForType::Unrolled,
        ir::MakeStore(acc, Combine(kind, ir::MakeLoad(acc, kc), ir::MakeCast(acc_type, ir::MakeLoad(reg, kc))), kc));
    return ir::MakeBlock({load, combine});
  };
  std::vector<Expr> accumulate;
  if (main_it > 0) {
    Expr io = ir::MakeVar("io", common::Int(32));
    Expr u  = ir::MakeVar("u", common::Int(32));
    // the loads of the unrolled rows are independent: the compiler issues them together
    Expr body = row((io * I32(unroll) + u) * I32(ty_n) + ty, 0);
    accumulate.push_back(ir::MakeFor(io, I32(0), I32(main_it), ForType::Serial,
                                     ir::MakeFor(u, I32(0), I32(unroll), ForType::Unrolled, body)));
  }
  if (full > main_it * unroll) {
    Expr i = ir::MakeVar("i", common::Int(32));
    accumulate.push_back(ir::MakeFor(i, I32(main_it * unroll), I32(full - main_it * unroll), ForType::Serial,
                                     row(i * I32(ty_n) + ty, 1)));
  }
  if (r % ty_n != 0) {
    Expr last = ctx->NewVar("last", common::Int(32));
    accumulate.push_back(ir::MakeLet(last, I32(full * ty_n) + ty));
    accumulate.push_back(ir::MakeIf(last < I32(r), row(last, 2)));
  }
  Expr accumulate_all = ir::MakeBlock(accumulate);
  if (col_guard) accumulate_all = ir::MakeIf(cvi < I32(cv), accumulate_all);
  stmts.push_back(accumulate_all);

  // every thread of the block takes part in the exchange through LDS
  BufferRef res  = ctx->NewLocal("res", out->dtype, vec);
  std::string fn = "cinn_block_column_reduce_" + ReduceSuffix(kind, acc_type);
  {
    Expr call = ir::MakeCall(Type(), fn, {I32(vec)});
    const_cast<ir::Call*>(call.As<ir::Call>())->buffer_args.push_back(acc);
    stmts.push_back(call);
  }
  stmts.push_back(ir::MakeFor(k, I32(0), I32(vec), ForType::Unrolled,
                              ir::MakeStore(res, ir::MakeCast(out->dtype, ir::MakeLoad(acc, k)), k)));
  Expr ks    = ir::MakeVar("ks", common::Int(32));
  Expr store = ir::MakeFor(ks, I32(0), I32(vec), ForType::Vectorized,
                           ir::MakeStore(dst, ir::MakeLoad(res, ks), ai * I32(c) + cvi * I32(vec) + ks));
  Expr owner = ty == I32(0);
  if (col_guard) owner = owner && (cvi < I32(cv));
  stmts.push_back(ir::MakeIf(owner, store));

  Expr threads_x  = ir::MakeFor(tx, I32(0), I32(tx_n), ForType::Serial, ir::MakeBlock(stmts), ThreadAxis(0));
  Expr threads_y  = ir::MakeFor(ty, I32(0), I32(ty_n), ForType::Serial, threads_x, ThreadAxis(1));
  ctx->func->body = ir::MakeFor(bid, I32(0), I32(a * grid_c), ForType::Serial, threads_y, BlockAxis(0));
  (void)target;
}

// [a][r][c] of a reduction whose reduced axes (sizes > 1) form one run; false otherwise
bool SingleReduceRun(const ShapeType& shape, const std::vector<int>& dims, int64_t* a, int64_t* r, int64_t* c) {
  const int rank = static_cast<int>(shape.size());
  std::vector<bool> reduced(rank, false);
  for (int d : dims) reduced[d] = true;
  *a = *r = *c = 1;
  int state = 0;  // 0: before the run, 1: inside, 2: after
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 1) continue;
    if (reduced[i]) {
      if (state == 2) return false;
      state = 1;
      *r *= shape[i];
    } else if (state == 0) {
      *a *= shape[i];
    } else {
      state = 2;
      *c *= shape[i];
    }
  }
  return true;
}

}  // namespace

// ---------------------------------------------------------------------------------------------------
// reductions over arbitrary axes: a column-reduce kernel when the reduced axes form one run, else one thread per
// output element
// ---------------------------------------------------------------------------------------------------
ir::LoweredFuncRef OpLowerer::LowerGeneralReduce(const Group& group) const {
  CINN_CHECK_EQ(group.nodes.size(), 1u) << "a general reduce group holds exactly one reduction";
  GroupContext ctx(group);
  Node* n           = group.nodes[0];
  NodeData* in      = n->inputs[0];
  NodeData* out     = n->outputs[0];
  const auto& shape = in->shape;
  int rank          = static_cast<int>(shape.size());
  auto dims         = ReduceDimsOf(*n);
  std::vector<bool> reduced(rank, false);
  for (int d : dims) reduced[d] = true;
  const std::string& kind = n->op->reduce_kind;
  bool is_arg             = kind == "argmax" || kind == "argmin";
  if (IsReduceRun(*n)) {
    const int64_t parts = GetAttr<int>(n->attrs, "parts", 1);
    EmitColumnReduce(&ctx, target_, in, out, kind, static_cast<int64_t>(GetAttr<int>(n->attrs, "a", 1)) * parts,
                     GetAttr<int>(n->attrs, "r", 1) / parts, GetAttr<int>(n->attrs, "c", 1));
    return ctx.func;
  }
  {
    int64_t a, r, c;
    if (!is_arg && options_.column_reduce && SingleReduceRun(shape, dims, &a, &r, &c) && r > 1) {
      EmitColumnReduce(&ctx, target_, in, out, kind, a, r, c);
      return ctx.func;
    }
  }

  ShapeType kept_shape;
  for (int i = 0; i < rank; ++i)
    if (!reduced[i]) kept_shape.push_back(shape[i]);
  int64_t out_numel = out->numel();
  CINN_CHECK_EQ(ShapeNumel(kept_shape), out_numel);

  const int block = options_.elementwise_block;
  int64_t grid    = (out_numel + block - 1) / block;
  Expr bx = ir::MakeVar("bx", common::Int(32));
  Expr tx = ir::MakeVar("tx", common::Int(32));
  Expr o  = ctx.NewVar("o", common::Int(32));

  std::vector<Expr> stmts;
  stmts.push_back(ir::MakeLet(o, bx * I32(block) + tx));
  std::vector<Expr> work;
  auto kept_coords = Decompose(o, kept_shape);
  std::vector<Expr> coords(rank);
  std::vector<Expr> loop_vars;
  for (int i = 0, kc = 0; i < rank; ++i) {
    if (reduced[i]) {
      coords[i] = ir::MakeVar("r" + std::to_string(i), common::Int(32));
      loop_vars.push_back(coords[i]);
    } else {
      coords[i] = kept_coords[kc++];
    }
  }
  Type acc_type = is_arg ? in->dtype : AccumType(kind, in->dtype);
  BufferRef acc = ctx.NewLocal("acc", acc_type, 1);
  BufferRef acc_idx;
  if (is_arg) {
    acc_idx = ctx.NewLocal("acc_idx", common::Int(32), 1);
    work.push_back(ir::MakeStore(acc, ir::MakeConst(acc_type, 0), I32(0)));
    work.push_back(ir::MakeStore(acc_idx, I32(-1), I32(0)));
  } else {
    work.push_back(ir::MakeStore(acc, ir::MakeCast(acc_type, ReduceIdentity(kind, acc_type)), I32(0)));
  }
  Expr v   = ir::MakeLoad(ctx.global_bufs.at(in), Compose(coords, shape));
  Expr cur = ir::MakeLoad(acc, I32(0));
  Expr inner;
  if (is_arg) {
    Expr better = kind == "argmax" ? (v > cur) : (v < cur);
    inner       = ir::MakeIf((ir::MakeLoad(acc_idx, I32(0)) < I32(0)) || better,
                             ir::MakeBlock({ir::MakeStore(acc, v, I32(0)), ir::MakeStore(acc_idx, coords[dims[0]], I32(0))}));
  } else {
    inner = ir::MakeStore(acc, Combine(kind, cur, ir::MakeCast(acc_type, v)), I32(0));
  }
  // ascending order over the reduced axes, outermost first
  for (int i = rank - 1; i >= 0; --i) {
    if (!reduced[i]) continue;
    inner = ir::MakeFor(coords[i], I32(0), I32(shape[i]), ForType::Serial, inner);
  }
  work.push_back(inner);
  Expr result = is_arg ? ir::MakeLoad(acc_idx, I32(0)) : ir::MakeCast(out->dtype, ir::MakeLoad(acc, I32(0)));
  work.push_back(ir::MakeStore(ctx.global_bufs.at(out), result, o));
  Expr guarded = ir::MakeBlock(work);
  if (out_numel % block != 0) guarded = ir::MakeIf(o < I32(out_numel), guarded);
  stmts.push_back(guarded);
  Expr threads   = ir::MakeFor(tx, I32(0), I32(block), ForType::Serial, ir::MakeBlock(stmts), ThreadAxis(0));
  ctx.func->body = ir::MakeFor(bx, I32(0), I32(grid), ForType::Serial, threads, BlockAxis(0));
  return ctx.func;
}

// ---------------------------------------------------------------------------------------------------
// library calls: a host function whose body is one call of a runtime intrinsic with baked constants
// ---------------------------------------------------------------------------------------------------
namespace {
ShapeType PadTo4(const ShapeType& s) {
  ShapeType out(4, 1);
  CINN_CHECK_LE(s.size(), 4u) << "matmul operands of rank > 4 are not supported";
  std::copy(s.begin(), s.end(), out.begin() + (4 - s.size()));
  return out;
}
}  // namespace

ir::LoweredFuncRef OpLowerer::LowerLibraryCall(const Group& group) const {
  CINN_CHECK_EQ(group.nodes.size(), 1u);
  // The reference lowers contractions through generated compute bodies when FLAGS_cinn_use_custom_call is 0
  // (cinn/hlir/framework/op_lowering.cc); here they exist only as library calls, so that setting is an error rather
  // than a silently different path.
  CINN_CHECK(EnvInt("FLAGS_cinn_use_custom_call", 1) != 0)
      << "FLAGS_cinn_use_custom_call=0 is not supported: matmul / conv2d / pool2d are lowered to library calls only";
  Node* n         = group.nodes[0];
  auto func       = std::make_shared<ir::LoweredFunc>();
  func->name      = group.func_name;
  func->is_device = false;
  for (auto* v : ArgumentsOf(group)) {
    ir::Argument arg;
    arg.buffer = ir::MakeBuffer(CName(v->id), v->dtype, MemoryType::Global, v->numel());
    arg.io     = std::find(group.outputs.begin(), group.outputs.end(), v) != group.outputs.end() ? ir::Argument::IO::kOutput
                                                                                                  : ir::Argument::IO::kInput;
    func->args.push_back(arg);
  }
  Expr kernel_args     = ir::MakeVar("kernel_args", common::Handle());
  Expr kernel_args_num = ir::MakeVar("kernel_args_num", common::Int(32));
  Expr kernel_stream   = ir::MakeVar("kernel_stream", common::Handle());
  std::vector<Expr> args = {kernel_args, kernel_args_num};
  std::string api;
  const std::string& op = n->op_type();
  auto push_ints = [&](std::initializer_list<int> vals) {
    for (int v : vals) args.push_back(I32(v));
  };
  if (op == "matmul" || op == "mul") {
    // argument list of CustomCallArgsForCublas (cinn/hlir/op/custom_call.cc:116-217)
    api = "cinn_call_cublas";
    bool ta = false, tb = false;
    const bool trans_out = GetAttr<bool>(n->attrs, "trans_out", false);
    const float alpha    = GetAttr<float>(n->attrs, "alpha", 1.0f);
    const float beta     = GetAttr<float>(n->attrs, "beta", 0.0f);
    ShapeType a_shape, b_shape;
    if (op == "matmul") {
      ta      = GetAttr<bool>(n->attrs, "trans_a", false);
      tb      = GetAttr<bool>(n->attrs, "trans_b", false);
      a_shape = n->inputs[0]->shape;
      b_shape = n->inputs[1]->shape;
      if (a_shape.size() == 1) a_shape = ta ? ShapeType{a_shape[0], 1} : ShapeType{1, a_shape[0]};
      if (b_shape.size() == 1) b_shape = tb ? ShapeType{1, b_shape[0]} : ShapeType{b_shape[0], 1};
    } else {
      int xn = GetAttr<int>(n->attrs, "x_num_col_dims", 1), yn = GetAttr<int>(n->attrs, "y_num_col_dims", 1);
      const auto& xs = n->inputs[0]->shape;
      const auto& ys = n->inputs[1]->shape;
      if (xn < 0) xn += static_cast<int>(xs.size());
      if (yn < 0) yn += static_cast<int>(ys.size());
      int a_height = 1, a_width = 1, b_height = 1, b_width = 1;
      for (int i = 0; i < xn; ++i) a_height *= xs[i];
      for (size_t i = xn; i < xs.size(); ++i) a_width *= xs[i];
      for (int i = 0; i < yn; ++i) b_height *= ys[i];
      for (size_t i = yn; i < ys.size(); ++i) b_width *= ys[i];
      a_shape = {a_height, a_width};
      b_shape = {b_height, b_width};
      if (GetAttr<bool>(n->attrs, "is_infer", false)) {
        // y is the transposed weight [N, K] (custom_call.cc:199-202)
        CINN_CHECK_EQ(a_width, b_width) << "mul (is_infer): the K dimensions differ";
        tb = true;
      } else {
        CINN_CHECK_EQ(a_width, b_height) << "mul: the K dimensions differ";
      }
    }
    auto a4 = PadTo4(a_shape), b4 = PadTo4(b_shape);
    args.push_back(Expr(ta));
    args.push_back(Expr(tb));
    args.push_back(Expr(trans_out));
    args.push_back(Expr(alpha));
    args.push_back(Expr(beta));
    push_ints({a4[0], a4[1], a4[2], a4[3], b4[0], b4[1], b4[2], b4[3]});
  } else if (op == "conv2d" && GetAttr<std::string>(n->attrs, "conv_type", "forward") != "forward") {
    // argument lists of CustomCallArgsForCudnnConvBackwardData / ...BackwardFilter (custom_call.cc:390-500): the
    // extents of x, w and dy in n, c, h, w order, whichever of them is the output
    const bool data = GetAttr<std::string>(n->attrs, "conv_type", "forward") == "backward_data";
    api             = data ? "cinn_call_cudnn_conv2d_backward_data" : "cinn_call_cudnn_conv2d_backward_filter";
    auto stride     = GetAttr<std::vector<int>>(n->attrs, "stride", {1, 1});
    auto padding    = GetAttr<std::vector<int>>(n->attrs, "padding", {0, 0});
    auto dilation   = GetAttr<std::vector<int>>(n->attrs, "dilation", {1, 1});
    int groups      = GetAttr<int>(n->attrs, "groups", 1);
    const bool nchw = GetAttr<std::string>(n->attrs, "data_format", "NCHW") == "NCHW";
    ShapeType x  = data ? n->outputs[0]->shape : n->inputs[0]->shape;
    ShapeType w  = data ? n->inputs[0]->shape : n->outputs[0]->shape;
    ShapeType dy = n->inputs[1]->shape;
    auto ordered = [&](const ShapeType& s) { return nchw ? s : ShapeType{s[0], s[3], s[1], s[2]}; };
    x = ordered(x), w = ordered(w), dy = ordered(dy);
    args.push_back(I32(nchw ? 0 : 1));
    args.push_back(Expr(1.0f));
    args.push_back(Expr(0.0f));
    push_ints({x[0], x[1], x[2], x[3], w[0], w[1], w[2], w[3]});
    push_ints({padding[0], padding[1], stride[0], stride[1], dilation[0], dilation[1], groups});
    push_ints({dy[0], dy[1], dy[2], dy[3]});
  } else if (op == "conv2d" || op == "hip_conv2d_bn_relu") {
    // argument list of CustomCallArgsForCudnnConvForward (custom_call.cc:338-388)
    auto stride   = GetAttr<std::vector<int>>(n->attrs, "stride", {1, 1});
    auto padding  = GetAttr<std::vector<int>>(n->attrs, "padding", {0, 0});
    auto dilation = GetAttr<std::vector<int>>(n->attrs, "dilation", {1, 1});
    int groups    = GetAttr<int>(n->attrs, "groups", 1);
    auto layout   = GetAttr<std::string>(n->attrs, "data_format", "NCHW");
    const auto& x = n->inputs[0]->shape;
    const auto& w = n->inputs[1]->shape;
    const auto& y = n->outputs[0]->shape;
    bool nchw       = layout == "NCHW";
    bool nchw_input = GetAttr<std::string>(n->attrs, "input_layout", layout) == "NCHW";
    // tensor format of the intrinsic: 0 NCHW, 1 NHWC, 2 NHWC output from an NCHW input and OIHW filter
    int format = nchw ? 0 : (nchw_input ? 2 : 1);
    if (op == "conv2d") {
      api = "cinn_call_cudnn_conv2d_forward";
      args.push_back(I32(format));
      args.push_back(Expr(1.0f));
      args.push_back(Expr(0.0f));
    } else {
      api = "cinn_call_hip_conv2d_bn_relu";
      args.push_back(I32(format));
      // bit 0: relu; bit 1: 3x3 / stride 2 / padding 1 max pooling after it, inside the kernel
      args.push_back(I32((GetAttr<bool>(n->attrs, "relu", false) ? 1 : 0) | (GetAttr<bool>(n->attrs, "max_pool", false) ? 2 : 0)));
    }
    // extents are always passed in n, c, h, w order
    if (nchw_input) {
      push_ints({x[0], x[1], x[2], x[3]});
      push_ints({w[0], w[1], w[2], w[3]});
    } else {
      push_ints({x[0], x[3], x[1], x[2]});
      push_ints({w[0], w[3], w[1], w[2]});
    }
    push_ints({padding[0], padding[1], stride[0], stride[1], dilation[0], dilation[1], groups});
    if (nchw) {
      push_ints({y[0], y[1], y[2], y[3]});
    } else if (GetAttr<bool>(n->attrs, "max_pool", false)) {
      // the output tensor is the pooled one; the intrinsic takes the convolution's own output extents
      const int xh = nchw_input ? x[2] : x[1], xw = nchw_input ? x[3] : x[2];
      const int kh = nchw_input ? w[2] : w[1], kw = nchw_input ? w[3] : w[2];
      push_ints({y[0], y[3], (xh + 2 * padding[0] - ((kh - 1) * dilation[0] + 1)) / stride[0] + 1,
                 (xw + 2 * padding[1] - ((kw - 1) * dilation[1] + 1)) / stride[1] + 1});
    } else {
      push_ints({y[0], y[3], y[1], y[2]});
    }
  } else if (op == "hip_conv2d_bn_relu_chain") {
    api           = "cinn_call_hip_conv2d_bn_relu_chain";
    const auto& x = n->inputs[0]->shape;
    args.push_back(I32((GetAttr<bool>(n->attrs, "relu", false) ? 1 : 0) | (GetAttr<bool>(n->attrs, "relu_after", false) ? 2 : 0)));
    push_ints({x[0], x[1], x[2], x[3], n->outputs[0]->shape[3], n->outputs[1]->shape[3]});
  } else if (op == "hip_conv2d_pair_chain") {
    api            = "cinn_call_hip_conv2d_pair_chain";
    const auto& x  = n->inputs[0]->shape;
    args.push_back(I32((GetAttr<bool>(n->attrs, "relu", false) ? 1 : 0) | (GetAttr<bool>(n->attrs, "relu_after", false) ? 2 : 0)));
    push_ints({x[0], x[1], x[2], x[3], n->inputs[1]->shape[3], n->outputs[0]->shape[3], n->outputs[1]->shape[3]});
  } else if (op == "hip_conv2d_pointwise_pair") {
    api            = "cinn_call_hip_conv2d_pointwise_pair";
    const auto& x  = n->inputs[0]->shape;
    const auto& x2 = n->inputs[1]->shape;
    auto stride2   = GetAttr<std::vector<int>>(n->attrs, "second_stride", {1, 1});
    args.push_back(I32(GetAttr<bool>(n->attrs, "relu", false) ? 1 : 0));
    push_ints({x[0], x[1], x[2], x[3], x2[1], x2[2], x2[3], stride2[0], stride2[1], n->outputs[0]->shape[3]});
  } else if (op == "pool2d" || op == "pool2d_grad") {
    // argument list of CustomCallArgsForCudnnPoolForward / ...PoolBackward (custom_call.cc:520-640): the gradient
    // takes x, y and dy and passes the extents of x and y
    api            = op == "pool2d" ? "cinn_call_cudnn_pool2d_forward" : "cinn_call_cudnn_pool2d_backward";
    auto ksize     = GetAttr<std::vector<int>>(n->attrs, "kernel_size", {1, 1});
    auto stride    = GetAttr<std::vector<int>>(n->attrs, "stride_size", {1, 1});
    auto padding   = GetAttr<std::vector<int>>(n->attrs, "padding_size", {0, 0, 0, 0});
    auto pool_type = GetAttr<std::string>(n->attrs, "pool_type", "max");
    bool exclusive = GetAttr<bool>(n->attrs, "exclusive", true);
    bool global    = GetAttr<bool>(n->attrs, "global_pooling", false);
    bool adaptive  = GetAttr<bool>(n->attrs, "adaptive", false);
    auto layout    = GetAttr<std::string>(n->attrs, "data_format", "NCHW");
    bool nchw      = layout == "NCHW";
    const auto& x  = n->inputs[0]->shape;
    const auto& y  = op == "pool2d" ? n->outputs[0]->shape : n->inputs[1]->shape;
    int ih = nchw ? x[2] : x[1], iw = nchw ? x[3] : x[2];
    int oh = nchw ? y[2] : y[1], ow = nchw ? y[3] : y[2];
    if (global) {
      ksize   = {ih, iw};
      stride  = {ih, iw};
      padding = {0, 0, 0, 0};
    } else if (adaptive) {
      // windows of floor(extent / outputs), side by side from the first row / column; what is left over at the end is
      // not read (PoolImpl, cinn/hlir/pe/nn.cc:1073-1112)
      CINN_CHECK(oh > 0 && ow > 0 && ih >= oh && iw >= ow) << "adaptive pool2d: more outputs than inputs";
      ksize   = {ih / oh, iw / ow};
      stride  = ksize;
      padding = {0, 0, 0, 0};
    }
    if (padding.size() == 2) padding = {padding[0], padding[1], padding[0], padding[1]};
    int mode = pool_type == "max" ? 0 : (exclusive ? 2 : 1);
    args.push_back(I32(mode));
    args.push_back(I32(nchw ? 0 : 1));
    args.push_back(Expr(1.0f));
    args.push_back(Expr(0.0f));
    if (nchw) {
      push_ints({x[0], x[1], x[2], x[3]});
    } else {
      push_ints({x[0], x[3], x[1], x[2]});
    }
    push_ints({ksize[0], ksize[1], padding[0], padding[1], stride[0], stride[1]});
    if (nchw) {
      push_ints({y[0], y[1], y[2], y[3]});
    } else {
      push_ints({y[0], y[3], y[1], y[2]});
    }
  } else if (op == "argsort" || op == "sort") {
    // [outer][size][inner] around the sorted axis; argsort writes indices and positions, sort the values
    api            = "cinn_call_hip_argsort";
    const auto& x  = n->inputs[0]->shape;
    int axis       = GetAttr<int>(n->attrs, "axis", 0);
    if (axis < 0) axis += static_cast<int>(x.size());
    CINN_CHECK(axis >= 0 && axis < static_cast<int>(x.size())) << op << ": axis out of range";
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < axis; ++d) outer *= x[d];
    for (size_t d = axis + 1; d < x.size(); ++d) inner *= x[d];
    {
      // cinn_call_hip_argsort keeps a whole row of keys (and, for rows with a NaN, positions) in one block's LDS:
      // 128 KiB / (key bytes + 4).  Longer rows are refused here, when the program is compiled, not at its first run.
      const int key_bytes   = n->inputs[0]->dtype.bytes() > 4 ? 8 : 4;
      const int64_t longest = (128 * 1024) / (key_bytes + 4);
      CINN_CHECK(((static_cast<int64_t>(x[axis]) + 3) & ~int64_t(3)) <= longest)
          << op << ": " << x[axis] << " elements along the sorted axis; the GPU kernel sorts rows of at most " << longest
          << " elements of this type (one block's LDS)";
    }
    push_ints({static_cast<int>(outer), x[axis], static_cast<int>(inner), GetAttr<bool>(n->attrs, "is_ascend", true) ? 1 : 0,
               op == "argsort" ? 3 : 4});
  } else {
    CINN_CHECK(false) << "op " << op << " has no GPU lowering";
  }
  args.push_back(kernel_stream);
  func->body = ir::MakeCall(Type(), api, args, ir::CallType::Extern);
  return func;
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
