// Device descriptor consumed by schedules and by the compiler driver.  Mirrors the interface of
// common::Target (cinn/common/target.h:25-112, target.cc:55-84, 177-221) with an AMDGPU arch whose
// numbers describe gfx950: 64-lane wavefronts, 1024 threads per block, 256 compute units in 8 XCDs,
// 160 KiB of LDS per compute unit.  The values come from the live device when one is visible and
// from the MI355X datasheet otherwise, so schedules are reproducible on a GPU-less build box.
#pragma once
#include <iosfwd>
#include <string>
#include <vector>

namespace cinn {
namespace common {

struct Target {
  enum class OS : int { Unk = -1, Linux, Windows };
  enum class Arch : int { Unk = -1, X86, ARM, NVGPU, AMDGPU };
  enum class Bit : int { Unk = -1, k32, k64 };

  OS os{OS::Unk};
  Arch arch{Arch::Unk};
  Bit bits{Bit::Unk};

  Target() = default;
  Target(OS o, Arch a, Bit b) : os(o), arch(a), bits(b) {}

  bool defined() const { return os != OS::Unk && arch != Arch::Unk && bits != Bit::Unk; }
  bool is_gpu() const { return arch == Arch::AMDGPU || arch == Arch::NVGPU; }

  // lanes that execute in lock-step: 64 on gfx950
  int wavefront_size() const;
  // threads per block limit (reference: max_num_threads(), 1024 on NVGPU)
  int max_num_threads() const;
  // compute units (reference: get_multi_processor_count())
  int get_multi_processor_count() const;
  // resident threads per compute unit (reference: get_max_threads_per_sm())
  int get_max_threads_per_sm() const;
  // resident blocks per compute unit (reference: get_max_blocks_per_sm())
  int get_max_blocks_per_sm() const;
  int lds_bytes_per_block() const;
  int lds_bytes_per_cu() const;
  int num_xcd() const;
  int runtime_arch() const;
  std::string arch_str() const;  // "gfx950"
  // key used in extern-function / external-API registries ("backend_amdgpu")
  std::string backend_key() const;

  bool operator==(const Target& o) const { return os == o.os && arch == o.arch && bits == o.bits; }
  bool operator!=(const Target& o) const { return !(*this == o); }
};

const Target& UnkTarget();
const Target& DefaultHostTarget();
const Target& DefaultAMDGPUTarget();
// AMDGPU: this build only knows the gfx950 backend.
const Target& DefaultTarget();
// CUs * resident threads per CU * 4, the element-count heuristic of GetMaxThreads() (target.cc:200-210)
int GetMaxThreads();
int GetMaxBlocks();

std::ostream& operator<<(std::ostream& os, const Target& t);

}  // namespace common
}  // namespace cinn
