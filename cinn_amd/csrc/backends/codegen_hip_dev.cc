#include "backends/codegen_hip_dev.h"

#include <set>

namespace cinn {
namespace backends {

using namespace ir;  // NOLINT

CodeGenHIP_Dev::CodeGenHIP_Dev(const common::Target& target) : target_(target) {
  CINN_CHECK(target.arch == common::Target::Arch::AMDGPU) << "CodeGenHIP_Dev needs an AMDGPU target";
}

const std::string& CodeGenHIP_Dev::GetSourceHeader() {
  static const std::string header = "#include \"cinn_hip_runtime_source.h\"\n\n";
  return header;
}

std::string CodeGenHIP_Dev::Compile(const Module& module, bool for_hiprtc) {
  std::string out;
  if (for_hiprtc) out += GetSourceHeader();
  std::set<std::string> names;
  for (auto& f : module.functions) {
    if (!f->is_device) continue;
    CINN_CHECK(names.insert(f->name).second) << "duplicate kernel name " << f->name;
    out += CompileFunc(*f);
    out += "\n";
  }
  return out;
}

std::string CodeGenHIP_Dev::CompileFunc(const LoweredFunc& func) {
  CINN_CHECK(func.is_device);
  CINN_CHECK(func.axis_info.valid) << "kernel " << func.name << " has no launch dimensions";
  os_.str("");
  indent_ = 0;
  PrintFunctionDeclaration(func);
  os_ << "\n{\n";
  ++indent_;
  PrintTempBuffers(func);
  PrintStmt(func.body);
  --indent_;
  os_ << "}\n";
  return os_.str();
}

void CodeGenHIP_Dev::PrintFunctionDeclaration(const LoweredFunc& func) {
  os_ << "extern \"C\" __global__\nvoid __launch_bounds__(" << func.axis_info.block_threads() << ") " << func.name
      << "(";
  bool first = true;
  for (auto& arg : func.args) {
    if (!first) os_ << ", ";
    first = false;
    if (arg.is_buffer()) {
      if (arg.io == Argument::IO::kInput) os_ << "const ";
      os_ << common::TypeCName(arg.buffer->dtype) << "* __restrict__ " << arg.buffer->name;
    } else {
      os_ << "const " << common::TypeCName(arg.var.type()) << " " << arg.var.As<Var>()->name;
    }
  }
  os_ << ")";
}

void CodeGenHIP_Dev::PrintTempBuffers(const LoweredFunc& func) {
  for (auto& buf : func.temp_bufs) {
    Indent();
    CINN_CHECK_GT(buf->num_elements, 0) << "temporary buffer " << buf->name << " has no size";
    // the alignment specifier leads the declaration: after __shared__ (a GNU attribute) it is rejected by some
    // front-end configurations ("an attribute list cannot appear here")
    os_ << "alignas(16) ";
    switch (buf->memory_type) {
      case MemoryType::GPUShared: os_ << "__shared__ "; break;
      case MemoryType::GPULocal: break;
      default: CINN_CHECK(false) << "temporary buffer " << buf->name << " must live in LDS or registers";
    }
    os_ << common::TypeCName(buf->dtype) << " " << buf->name << "[" << buf->num_elements << "];\n";
  }
}

void CodeGenHIP_Dev::VisitVar(const Var* op) {
  const std::string& n = op->name;
  if (n.rfind("threadIdx.", 0) == 0 || n.rfind("blockIdx.", 0) == 0 || n.rfind("blockDim.", 0) == 0 ||
      n.rfind("gridDim.", 0) == 0) {
    os_ << "(" << common::TypeCName(op->type) << ")" << n;
  } else {
    os_ << n;
  }
}

void CodeGenHIP_Dev::VisitBinary(const Binary* op) {
  if (op->node_type == IrNodeTy::Min || op->node_type == IrNodeTy::Max) {
    os_ << (op->node_type == IrNodeTy::Min ? "cinn_hip_min_generic(" : "cinn_hip_max_generic(");
    Visit(op->a);
    os_ << ", ";
    Visit(op->b);
    os_ << ")";
    return;
  }
  IrPrinter::VisitBinary(op);
}

void CodeGenHIP_Dev::VisitLoad(const Load* op) {
  CINN_CHECK(!op->index.As<Ramp>()) << "a vector load may only appear as the value of a vector store";
  IrPrinter::VisitLoad(op);
}

void CodeGenHIP_Dev::VisitStore(const Store* op) {
  auto* ramp = op->index.As<Ramp>();
  if (!ramp) {
    IrPrinter::VisitStore(op);
    return;
  }
  auto* ld = op->value.As<Load>();
  CINN_CHECK(ld) << "a vector store must copy a vector load";
  auto* lramp = ld->index.As<Ramp>();
  CINN_CHECK(lramp && lramp->lanes == ramp->lanes && lramp->stride == 1 && ramp->stride == 1);
  const char* copy_fn = "cinn_hip_copy_vec";
  if (op->buffer->memory_type == MemoryType::Global && op->buffer->streaming_store) copy_fn = "cinn_hip_store_stream_vec";
  if (ld->buffer->memory_type == MemoryType::Global && ld->buffer->streaming_load) copy_fn = "cinn_hip_load_stream_vec";
  os_ << copy_fn << "<" << common::TypeCName(op->buffer->dtype) << ", " << ramp->lanes << ">(&"
      << op->buffer->name << "[";
  Visit(ramp->base);
  os_ << "], &" << ld->buffer->name << "[";
  Visit(lramp->base);
  os_ << "])";
}

void CodeGenHIP_Dev::VisitFor(const For* op) {
  CINN_CHECK(!op->bind_info.valid()) << "a loop bound to a GPU axis reached the code generator";
  if (op->for_type == ForType::Unrolled || op->for_type == ForType::Vectorized) {
    os_ << "#pragma unroll\n";
    Indent();
  }
  IrPrinter::VisitFor(op);
}

void CodeGenHIP_Dev::VisitCall(const Call* op) {
  if (op->name == "__syncthreads") {
    os_ << "__syncthreads()";
    return;
  }
  IrPrinter::VisitCall(op);
}

}  // namespace backends
}  // namespace cinn
