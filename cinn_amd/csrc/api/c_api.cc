#include "cinn_amd_api.h"

#include <cstring>
#include <functional>
#include <map>
#include <sstream>

#include "backends/host_stub.h"
#include "frontend/computation.h"
#include "frontend/net_builder.h"
#include "hlir/op.h"

using cinn::frontend::CinnComputation;
using cinn::frontend::NetBuilder;
using cinn::frontend::Variable;
using cinn::hlir::framework::GetAttr;
using cinn::utils::AttributeMap;
using cinn::utils::ShapeType;

struct cinn_amd_builder {
  std::unique_ptr<NetBuilder> builder;
  std::map<std::string, Variable> vars;
};
struct cinn_amd_computation {
  std::shared_ptr<CinnComputation> comp;
};

namespace {

thread_local std::string g_last_error;

template <typename Fn>
int Guard(Fn&& fn) {
  try {
    fn();
    return 0;
  } catch (const std::exception& e) {
    g_last_error = e.what();
    return 1;
  } catch (...) {
    g_last_error = "unknown C++ exception";
    return 1;
  }
}

void CopyOut(const std::string& s, char* out, size_t cap, size_t* needed = nullptr) {
  if (needed) *needed = s.size() + 1;
  if (!out || cap == 0) return;
  if (!needed) CINN_CHECK_LT(s.size(), cap) << "output buffer of " << cap << " bytes is too small";
  size_t n = std::min(s.size(), cap - 1);
  memcpy(out, s.data(), n);
  out[n] = 0;
}

std::string Join(const std::vector<std::string>& v) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + v[i];
  return s;
}

using Method = std::function<std::vector<Variable>(NetBuilder&, const std::vector<Variable>&, const AttributeMap&)>;

const std::map<std::string, Method>& Methods() {
  static const std::map<std::string, Method> table = [] {
    std::map<std::string, Method> m;
#define CINN_API_UNARY(fn, op) \
  m[#fn] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap&) { return std::vector<Variable>{b.fn(in.at(0))}; };
    CINN_NETBUILDER_UNARY_FOREACH(CINN_API_UNARY)
#undef CINN_API_UNARY
#define CINN_API_BINARY(fn, op)                                                                   \
  m[#fn] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {           \
    return std::vector<Variable>{b.fn(in.at(0), in.at(1), GetAttr<int>(a, "axis", -1))};          \
  };
    CINN_NETBUILDER_BINARY_FOREACH(CINN_API_BINARY)
#undef CINN_API_BINARY
#define CINN_API_REDUCE(fn)                                                                                         \
  m[#fn] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {                              \
    return std::vector<Variable>{b.fn(in.at(0), GetAttr<ShapeType>(a, "dim", {}), GetAttr<bool>(a, "keep_dim", false))}; \
  };
    CINN_API_REDUCE(ReduceSum)
    CINN_API_REDUCE(ReduceProd)
    CINN_API_REDUCE(ReduceMax)
    CINN_API_REDUCE(ReduceMin)
    CINN_API_REDUCE(ReduceAll)
    CINN_API_REDUCE(ReduceAny)
#undef CINN_API_REDUCE
    m["Argmax"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Argmax(in.at(0), GetAttr<int>(a, "axis", 0), GetAttr<bool>(a, "keep_dim", false))};
    };
    m["Argmin"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Argmin(in.at(0), GetAttr<int>(a, "axis", 0), GetAttr<bool>(a, "keep_dim", false))};
    };
    m["ArgSort"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return b.ArgSort(in.at(0), GetAttr<int>(a, "axis", 0), GetAttr<bool>(a, "is_ascend", true));
    };
    m["Sort"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Sort(in.at(0), GetAttr<int>(a, "axis", 0), GetAttr<bool>(a, "is_ascend", true))};
    };
    m["TopK"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return b.TopK(in.at(0), GetAttr<int>(a, "k", 1), GetAttr<int>(a, "axis", -1), GetAttr<bool>(a, "largest", true));
    };
    m["Select"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap&) {
      return std::vector<Variable>{b.Select(in.at(0), in.at(1), in.at(2))};
    };
    m["Scale"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Scale(in.at(0), GetAttr<float>(a, "scale", 1.0f), GetAttr<float>(a, "bias", 0.0f),
                                           GetAttr<bool>(a, "bias_after_scale", true))};
    };
    m["Sum"]   = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap&) { return std::vector<Variable>{b.Sum(in)}; };
    m["Relu6"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Relu6(in.at(0), GetAttr<float>(a, "threshold", 6.0f))};
    };
    m["Cast"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Cast(in.at(0), GetAttr<std::string>(a, "dtype", "float32"))};
    };
    m["FillConstant"] = [](NetBuilder& b, const std::vector<Variable>&, const AttributeMap& a) {
      return std::vector<Variable>{b.FillConstant(GetAttr<ShapeType>(a, "shape", {1}), GetAttr<float>(a, "value", 0.0f),
                                                  GetAttr<std::string>(a, "name", ""),
                                                  GetAttr<std::string>(a, "dtype", "float32"))};
    };
    m["BroadcastTo"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      auto out_shape = GetAttr<ShapeType>(a, "out_shape", {});
      if (a.count("broadcast_axes")) {
        return std::vector<Variable>{b.BroadcastTo(in.at(0), out_shape, GetAttr<ShapeType>(a, "broadcast_axes", {}))};
      }
      return std::vector<Variable>{b.BroadcastTo(in.at(0), out_shape)};
    };
    m["Reshape"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Reshape(in.at(0), GetAttr<ShapeType>(a, "shape", {}))};
    };
    m["Transpose"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Transpose(in.at(0), GetAttr<ShapeType>(a, "axis", {}))};
    };
    m["Concat"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Concat(in, GetAttr<int>(a, "axis", 0))};
    };
    m["Slice"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Slice(in.at(0), GetAttr<ShapeType>(a, "axes", {}), GetAttr<ShapeType>(a, "starts", {}),
                                           GetAttr<ShapeType>(a, "ends", {}), GetAttr<ShapeType>(a, "infer_flags", {}),
                                           GetAttr<ShapeType>(a, "strides", {}), GetAttr<ShapeType>(a, "decrease_axis", {}))};
    };
    m["Squeeze"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Squeeze(in.at(0), GetAttr<ShapeType>(a, "axes", {}))};
    };
    m["ExpandDims"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.ExpandDims(in.at(0), GetAttr<ShapeType>(a, "axes", {}))};
    };
    m["Softmax"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Softmax(in.at(0), GetAttr<ShapeType>(a, "axes", {-1}),
                                             GetAttr<std::string>(a, "mode", "fast"),
                                             GetAttr<std::string>(a, "data_format", "AnyLayout"))};
    };
    m["Matmul"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Matmul(in.at(0), in.at(1), GetAttr<bool>(a, "trans_x", false),
                                            GetAttr<bool>(a, "trans_y", false), GetAttr<float>(a, "alpha", 1.0f))};
    };
    m["Mul"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Mul(in.at(0), in.at(1), GetAttr<int>(a, "x_num_col_dims", 1),
                                         GetAttr<int>(a, "y_num_col_dims", 1), GetAttr<bool>(a, "is_infer", false))};
    };
    m["Conv2d"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Conv2d(in.at(0), in.at(1), GetAttr<std::vector<int>>(a, "strides", {1, 1}),
                                            GetAttr<std::vector<int>>(a, "paddings", {0, 0}),
                                            GetAttr<std::vector<int>>(a, "dilations", {1, 1}), GetAttr<int>(a, "groups", 1),
                                            GetAttr<std::string>(a, "data_format", "NCHW"),
                                            GetAttr<std::string>(a, "padding_algorithm", "EXPLICIT"))};
    };
    m["Conv"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Conv(in.at(0), in.at(1), GetAttr<std::vector<int>>(a, "strides", {1, 1}),
                                          GetAttr<std::vector<int>>(a, "paddings", {0, 0}),
                                          GetAttr<std::vector<int>>(a, "dilations", {1, 1}), GetAttr<int>(a, "groups", 1),
                                          GetAttr<std::string>(a, "conv_type", "forward"),
                                          GetAttr<std::string>(a, "data_format", "NCHW"),
                                          GetAttr<std::string>(a, "padding_algorithm", "EXPLICIT"),
                                          GetAttr<std::vector<int>>(a, "output_shape", {}))};
    };
    m["BatchNorm"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return b.BatchNorm(in.at(0), in.at(1), in.at(2), in.at(3), in.at(4), GetAttr<float>(a, "epsilon", 1e-5f),
                         GetAttr<float>(a, "momentum", 0.9f), GetAttr<std::string>(a, "data_layout", "NCHW"),
                         GetAttr<bool>(a, "is_test", true));
    };
    m["ReluGrad"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap&) {
      return std::vector<Variable>{b.ReluGrad(in.at(0), in.at(1))};
    };
    m["ElementwiseAddGrad"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return b.ElementwiseAddGrad(in.at(0), in.at(1), in.at(2), GetAttr<int>(a, "axis", -1));
    };
    m["BatchNormGrad"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return b.BatchNormGrad(in.at(0), in.at(1), in.at(2), in.at(3), in.at(4), GetAttr<float>(a, "epsilon", 1e-5f),
                             GetAttr<std::string>(a, "data_layout", "NCHW"));
    };
    m["Pool2d"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{
          b.Pool2d(in.at(0), GetAttr<std::string>(a, "pooling_type", "max"), GetAttr<std::vector<int>>(a, "ksize", {1, 1}),
                   GetAttr<std::vector<int>>(a, "strides", {1, 1}), GetAttr<std::vector<int>>(a, "paddings", {0, 0}),
                   GetAttr<bool>(a, "ceil_mode", false), GetAttr<bool>(a, "exclusive", true),
                   GetAttr<bool>(a, "global_pooling", false), GetAttr<std::string>(a, "data_format", "NCHW"),
                   GetAttr<bool>(a, "adaptive", false), GetAttr<std::string>(a, "padding_algorithm", "EXPLICIT"))};
    };
    m["Pool2dGrad"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      return std::vector<Variable>{b.Pool2dGrad(
          in.at(0), in.at(1), in.at(2), GetAttr<std::string>(a, "pooling_type", "max"),
          GetAttr<std::vector<int>>(a, "ksize", {1, 1}), GetAttr<std::vector<int>>(a, "strides", {1, 1}),
          GetAttr<std::vector<int>>(a, "paddings", {0, 0}), GetAttr<bool>(a, "ceil_mode", false),
          GetAttr<bool>(a, "exclusive", true), GetAttr<bool>(a, "global_pooling", false),
          GetAttr<std::string>(a, "data_format", "NCHW"), GetAttr<bool>(a, "adaptive", false),
          GetAttr<std::string>(a, "padding_algorithm", "EXPLICIT"))};
    };
    // inputs: x [, scale [, bias]]
    m["PaddleLayerNorm"] = [](NetBuilder& b, const std::vector<Variable>& in, const AttributeMap& a) {
      Variable scale = in.size() > 1 ? in[1] : Variable();
      Variable bias  = in.size() > 2 ? in[2] : Variable();
      return cinn::frontend::PaddleLayerNorm(&b, in.at(0), scale, bias, GetAttr<float>(a, "epsilon", 1e-5f),
                                             GetAttr<int>(a, "begin_norm_axis", 1));
    };
    return m;
  }();
  return table;
}

void FillInfo(const ShapeType& shape, const cinn::common::Type& type, int32_t* shape_out, int32_t* rank_out,
              char* dtype_out, size_t dtype_cap) {
  if (rank_out) *rank_out = static_cast<int32_t>(shape.size());
  if (shape_out)
    for (size_t i = 0; i < shape.size() && i < 8; ++i) shape_out[i] = shape[i];
  if (dtype_out) CopyOut(cinn::common::Type2Str(type), dtype_out, dtype_cap);
}

}  // namespace

extern "C" {

const char* cinn_amd_last_error(void) { return g_last_error.c_str(); }

int cinn_amd_builder_create(const char* name, cinn_amd_builder_t* out) {
  return Guard([&] {
    auto* b    = new cinn_amd_builder;
    b->builder = std::make_unique<NetBuilder>(name ? name : "net_builder");
    *out       = b;
  });
}
int cinn_amd_builder_destroy(cinn_amd_builder_t b) {
  delete b;
  return 0;
}

int cinn_amd_builder_create_input(cinn_amd_builder_t b, const char* dtype, const int32_t* shape, int32_t rank,
                                  const char* name_hint, char* id_out, size_t id_cap) {
  return Guard([&] {
    CINN_CHECK(b && dtype && shape) << "null argument";
    ShapeType s(shape, shape + rank);
    auto v = b->builder->CreateInput(cinn::common::Str2Type(dtype), s, name_hint ? name_hint : "");
    b->vars[v->id] = v;
    CopyOut(v->id, id_out, id_cap);
  });
}

int cinn_amd_builder_call(cinn_amd_builder_t b, const char* method, const char* const* inputs, int32_t num_inputs,
                          const char* attrs, char* ids_out, size_t ids_cap) {
  return Guard([&] {
    CINN_CHECK(b && method) << "null argument";
    std::vector<Variable> in;
    for (int i = 0; i < num_inputs; ++i) {
      auto it = b->vars.find(inputs[i]);
      CINN_CHECK(it != b->vars.end()) << "unknown variable '" << inputs[i] << "'";
      in.push_back(it->second);
    }
    AttributeMap a = cinn::utils::ParseAttributeString(attrs ? attrs : "");
    std::vector<Variable> outs;
    std::string name = method;
    if (name.rfind("CustomInstr:", 0) == 0) {
      outs = b->builder->CustomInstr(name.substr(strlen("CustomInstr:")), in, a);
    } else {
      auto it = Methods().find(name);
      CINN_CHECK(it != Methods().end()) << "NetBuilder has no method '" << name << "'";
      outs = it->second(*b->builder, in, a);
    }
    std::vector<std::string> ids;
    for (auto& o : outs) {
      b->vars[o->id] = o;
      ids.push_back(o->id);
    }
    CopyOut(Join(ids), ids_out, ids_cap);
  });
}

int cinn_amd_builder_var_info(cinn_amd_builder_t b, const char* id, int32_t* shape_out, int32_t* rank_out,
                              char* dtype_out, size_t dtype_cap) {
  return Guard([&] {
    auto it = b->vars.find(id);
    CINN_CHECK(it != b->vars.end()) << "unknown variable '" << id << "'";
    FillInfo(it->second->shape, it->second->type, shape_out, rank_out, dtype_out, dtype_cap);
  });
}

int cinn_amd_builder_set_const(cinn_amd_builder_t b, const char* id, int32_t is_const) {
  return Guard([&] {
    auto it = b->vars.find(id);
    CINN_CHECK(it != b->vars.end()) << "unknown variable '" << id << "'";
    it->second->is_const = is_const != 0;
  });
}

int cinn_amd_builder_size(cinn_amd_builder_t b, int32_t* num_instructions) {
  return Guard([&] { *num_instructions = static_cast<int32_t>(b->builder->size()); });
}

int cinn_amd_builder_program_string(cinn_amd_builder_t b, char* out, size_t cap, size_t* needed) {
  return Guard([&] { CopyOut(b->builder->Build().debug_string(), out, cap, needed); });
}

int cinn_amd_computation_build_and_compile(cinn_amd_builder_t b, const char* const* outputs, int32_t num_outputs,
                                           void* stream, const char* options, cinn_amd_computation_t* out) {
  return Guard([&] {
    CINN_CHECK(b && out) << "null argument";
    std::vector<Variable> outs;
    for (int i = 0; i < num_outputs; ++i) {
      auto it = b->vars.find(outputs[i]);
      CINN_CHECK(it != b->vars.end()) << "unknown output variable '" << outputs[i] << "'";
      outs.push_back(it->second);
    }
    auto opts = CinnComputation::DefaultCompileOptions();
    if (options && *options) {
      std::istringstream iss(options);
      std::string item;
      while (std::getline(iss, item, ';')) {
        if (item.empty()) continue;
        auto eq = item.find('=');
        CINN_CHECK(eq != std::string::npos) << "malformed option '" << item << "'";
        std::string k = item.substr(0, eq);
        int v         = std::stoi(item.substr(eq + 1));
        if (k == "do_prerun") {
          opts.do_prerun = v != 0;
        } else if (k == "fuse_conv_bn_relu") {
          opts.fuse_conv_bn_relu = v != 0;
        } else if (k == "fuse_stem_pool") {
          opts.fuse_stem_pool = v != 0;
        } else if (k == "fuse_matmul_bias") {
          opts.fuse_matmul_bias = v != 0;
        } else if (k == "fuse_conv_chain") {
          opts.fuse_conv_chain = v != 0;
        } else if (k == "fuse_shortcut_projection") {
          opts.fuse_shortcut_projection = v != 0;
        } else if (k == "reshape_as_view") {
          opts.reshape_as_view = v != 0;
        } else if (k == "merge_independent_kernels") {
          opts.merge_independent_kernels = v != 0;
        } else if (k == "memory_arena") {
          opts.memory_arena = v != 0;
        } else if (k == "reuse_intermediates") {
          opts.reuse_intermediates = v != 0;
        } else if (k == "conv_layout_nhwc") {
          opts.conv_layout_nhwc = v != 0;
        } else if (k == "split_reductions") {
          opts.split_reductions = v != 0;
        } else if (k == "reduce_cached_elems") {
          opts.lowering.max_cached_elems_per_thread = v;
        } else if (k == "reduce_wave_elems") {
          opts.lowering.wave_row_elems_per_lane = v;
        } else if (k == "elementwise_block") {
          opts.lowering.elementwise_block = v;
        } else if (k == "reduce_rows_per_block") {
          opts.lowering.rows_per_block = v;
        } else {
          CINN_CHECK(false) << "unknown compile option '" << k << "'";
        }
      }
    }
    auto comp = CinnComputation::BuildAndCompile(cinn::common::DefaultAMDGPUTarget(), *b->builder, opts, outs, stream);
    auto* c   = new cinn_amd_computation;
    c->comp   = comp;
    *out      = c;
  });
}

int cinn_amd_computation_destroy(cinn_amd_computation_t c) {
  delete c;
  return 0;
}
int cinn_amd_computation_execute(cinn_amd_computation_t c) {
  return Guard([&] { c->comp->Execute(); });
}
int cinn_amd_computation_execute_graph(cinn_amd_computation_t c) {
  return Guard([&] { c->comp->ExecuteGraph(); });
}
int cinn_amd_computation_pre_run(cinn_amd_computation_t c) {
  return Guard([&] { c->comp->PreRun(); });
}
int cinn_amd_computation_memory_info(cinn_amd_computation_t c, size_t* arena_bytes, size_t* unshared_bytes) {
  return Guard([&] {
    if (arena_bytes) *arena_bytes = c->comp->arena_bytes();
    if (unshared_bytes) *unshared_bytes = c->comp->unshared_bytes();
  });
}
int cinn_amd_computation_num_instructions(cinn_amd_computation_t c, int32_t* n) {
  return Guard([&] { *n = static_cast<int32_t>(c->comp->num_instructions()); });
}
int cinn_amd_computation_graph_lanes(cinn_amd_computation_t c, int32_t* lanes, int32_t capacity, int32_t* count) {
  return Guard([&] {
    const std::vector<int>& l = c->comp->GraphLanes();
    *count                    = static_cast<int32_t>(l.size());
    for (int32_t i = 0; i < capacity && i < *count; ++i) lanes[i] = l[i];
  });
}
int cinn_amd_computation_set_tensor(cinn_amd_computation_t c, const char* name, const void* data, size_t bytes) {
  return Guard([&] { c->comp->SetTensorData(name, const_cast<void*>(data), bytes); });
}
int cinn_amd_computation_get_tensor(cinn_amd_computation_t c, const char* name, void* data, size_t bytes) {
  return Guard([&] { c->comp->GetTensorData(name, data, bytes); });
}
int cinn_amd_computation_tensor_info(cinn_amd_computation_t c, const char* name, int32_t* shape_out,
                                     int32_t* rank_out, char* dtype_out, size_t dtype_cap, void** device_ptr) {
  return Guard([&] {
    auto t = c->comp->GetTensor(name);
    FillInfo(t->shape(), t->type(), shape_out, rank_out, dtype_out, dtype_cap);
    if (device_ptr) *device_ptr = t->data();
  });
}
int cinn_amd_computation_tensor_names(cinn_amd_computation_t c, int32_t which, char* out, size_t cap, size_t* needed) {
  return Guard([&] {
    std::vector<std::string> names = which == 0   ? c->comp->input_names()
                                     : which == 1 ? c->comp->output_names()
                                                  : c->comp->GetAllTensorNames();
    CopyOut(Join(names), out, cap, needed);
  });
}
int cinn_amd_computation_source_code(cinn_amd_computation_t c, char* out, size_t cap, size_t* needed) {
  return Guard([&] { CopyOut(c->comp->source_code(), out, cap, needed); });
}
int cinn_amd_computation_group_string(cinn_amd_computation_t c, char* out, size_t cap, size_t* needed) {
  return Guard([&] { CopyOut(c->comp->group_debug_string(), out, cap, needed); });
}
int cinn_amd_computation_instruction_info(cinn_amd_computation_t c, int32_t index, char* fn_name, size_t fn_cap,
                                          char* args, size_t args_cap) {
  return Guard([&] {
    auto& instrs = c->comp->program()->GetRunInstructions();
    CINN_CHECK(index >= 0 && index < static_cast<int32_t>(instrs.size())) << "instruction index out of range";
    auto& ins = instrs[index];
    CopyOut(ins->function_name(), fn_name, fn_cap);
    std::vector<std::string> names = ins->in_args();
    names.insert(names.end(), ins->out_args().begin(), ins->out_args().end());
    CopyOut(Join(names), args, args_cap);
  });
}
int cinn_amd_computation_run_instruction(cinn_amd_computation_t c, int32_t index) {
  return Guard([&] {
    auto& instrs = c->comp->program()->GetRunInstructions();
    CINN_CHECK(index >= 0 && index < static_cast<int32_t>(instrs.size())) << "instruction index out of range";
    instrs[index]->Run(c->comp->stream());
  });
}

int cinn_amd_list_operators(char* out, size_t cap, size_t* needed) {
  return Guard([&] { CopyOut(Join(cinn::hlir::framework::OpRegistry::Global().ListAllNames()), out, cap, needed); });
}

int cinn_amd_extern_api_names(char* out, size_t cap, size_t* needed) {
  return Guard([&] { CopyOut(Join(cinn::backends::ExternApiRegistry::Global().Names()), out, cap, needed); });
}

int cinn_amd_host_stub_create(const char* api, const char* constants, void** fn) {
  return Guard([&] {
    namespace ir = cinn::ir;
    CINN_CHECK(api && fn) << "null argument";
    std::vector<ir::Expr> args = {ir::MakeVar("kernel_args", cinn::common::Handle()),
                                  ir::MakeVar("kernel_args_num", cinn::common::Int(32))};
    std::stringstream items(constants ? constants : "");
    std::string item;
    while (std::getline(items, item, ',')) {
      if (item.empty()) continue;
      CINN_CHECK(item.size() > 2 && item[1] == ':') << "bad constant '" << item << "' (want i:<int>, f:<float> or b:<0|1>)";
      const std::string value = item.substr(2);
      switch (item[0]) {
        case 'i': args.push_back(ir::MakeIntImm(cinn::common::Int(64), std::stoll(value))); break;
        case 'f': args.push_back(ir::Expr(static_cast<float>(std::stod(value)))); break;
        case 'b': args.push_back(ir::Expr(value != "0")); break;
        default: CINN_CHECK(false) << "bad constant '" << item << "'";
      }
    }
    args.push_back(ir::MakeVar("kernel_stream", cinn::common::Handle()));
    ir::LoweredFunc func;
    func.name      = std::string("stub_of_") + api;
    func.is_device = false;
    func.body      = ir::MakeCall(cinn::common::Type(), api, args, ir::CallType::Extern);
    auto closure   = cinn::backends::LowerHostFunction(func, {});
    *fn            = reinterpret_cast<void*>(cinn::backends::HostStubPool::Global().Acquire(std::move(closure)));
  });
}

int cinn_amd_host_stub_release(void* fn) {
  return Guard([&] { cinn::backends::HostStubPool::Global().Release(reinterpret_cast<lower_func_ptr_g>(fn)); });
}

}  // extern "C"
