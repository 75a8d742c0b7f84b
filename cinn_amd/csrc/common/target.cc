#include "common/target.h"

#include <mutex>
#include <ostream>

#include "cinn_hip_runtime.h"
#include "common/check.h"

namespace cinn {
namespace common {

namespace {
const cinn_hip_target_info& DeviceInfo() {
  static cinn_hip_target_info info;
  static std::once_flag once;
  std::call_once(once, [] { cinn_hip_get_target_info(&info); });
  return info;
}
}  // namespace

int Target::wavefront_size() const { return arch == Arch::AMDGPU ? DeviceInfo().wavefront_size : 1; }

int Target::max_num_threads() const {
  CINN_CHECK(arch == Arch::AMDGPU) << "max_num_threads() is a GPU query";
  return DeviceInfo().max_threads_per_block;
}
int Target::get_multi_processor_count() const {
  CINN_CHECK(arch == Arch::AMDGPU) << "get_multi_processor_count() is a GPU query";
  return DeviceInfo().multi_processor_count;
}
int Target::get_max_threads_per_sm() const {
  CINN_CHECK(arch == Arch::AMDGPU) << "get_max_threads_per_sm() is a GPU query";
  return DeviceInfo().max_threads_per_multi_processor;
}
int Target::get_max_blocks_per_sm() const {
  CINN_CHECK(arch == Arch::AMDGPU) << "get_max_blocks_per_sm() is a GPU query";
  return DeviceInfo().max_blocks_per_multi_processor;
}
int Target::lds_bytes_per_block() const { return DeviceInfo().lds_bytes_per_block; }
int Target::lds_bytes_per_cu() const { return DeviceInfo().lds_bytes_per_multi_processor; }
int Target::num_xcd() const { return DeviceInfo().num_xcd; }
int Target::runtime_arch() const { return static_cast<int>(arch); }
std::string Target::arch_str() const { return arch == Arch::AMDGPU ? std::string(DeviceInfo().arch) : "host"; }
std::string Target::backend_key() const {
  switch (arch) {
    case Arch::AMDGPU: return "backend_amdgpu";
    case Arch::NVGPU: return "backend_nvgpu";
    case Arch::X86: return "backend_x86";
    default: return "backend_unk";
  }
}

const Target& UnkTarget() {
  static Target t(Target::OS::Unk, Target::Arch::Unk, Target::Bit::Unk);
  return t;
}
const Target& DefaultHostTarget() {
  static Target t(Target::OS::Linux, Target::Arch::X86, Target::Bit::k64);
  return t;
}
const Target& DefaultAMDGPUTarget() {
  static Target t(Target::OS::Linux, Target::Arch::AMDGPU, Target::Bit::k64);
  return t;
}
const Target& DefaultTarget() { return DefaultAMDGPUTarget(); }

int GetMaxThreads() {
  const auto& t = DefaultAMDGPUTarget();
  return t.get_multi_processor_count() * t.get_max_threads_per_sm() * 4;
}
int GetMaxBlocks() {
  const auto& t = DefaultAMDGPUTarget();
  return t.get_multi_processor_count() * t.get_max_blocks_per_sm();
}

std::ostream& operator<<(std::ostream& os, const Target& t) {
  os << "Target<";
  os << (t.os == Target::OS::Linux ? "linux" : t.os == Target::OS::Windows ? "windows" : "unk") << ",";
  switch (t.arch) {
    case Target::Arch::X86: os << "x86"; break;
    case Target::Arch::ARM: os << "arm"; break;
    case Target::Arch::NVGPU: os << "nvgpu"; break;
    case Target::Arch::AMDGPU: os << "amdgpu"; break;
    default: os << "unk";
  }
  os << "," << (t.bits == Target::Bit::k64 ? "64" : t.bits == Target::Bit::k32 ? "32" : "unk") << ">";
  return os;
}

}  // namespace common
}  // namespace cinn
