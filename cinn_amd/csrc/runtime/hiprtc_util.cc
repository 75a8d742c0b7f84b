// hiprtc wrapper: HIP source -> gfx950 code object.  Role of nvrtc::Compiler
// (cinn/backends/nvrtc/nvrtc_util.cc:40-152): fixed option set, device library handed over as an
// in-memory header, compile log returned on failure.  Identical sources are served from an
// in-process cache so a program that is rebuilt does not pay hiprtc twice.
#include <hip/hiprtc.h>

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "cinn_hip_runtime.h"

extern "C" const char cinn_hip_device_lib_source_text[];

namespace {
char* DupString(const std::string& s) {
  char* p = static_cast<char*>(malloc(s.size() + 1));
  memcpy(p, s.data(), s.size());
  p[s.size()] = 0;
  return p;
}
std::mutex g_cache_mu;
std::map<std::string, std::string> g_code_cache;  // key: options + '\0' + source
}  // namespace

extern "C" {

const char* cinn_hip_device_lib_source(void) { return cinn_hip_device_lib_source_text; }

int cinn_hip_rtc_compile(const char* source, int with_device_lib, const char* extra_options, char** code,
                         size_t* code_size, char** log) {
  if (code) *code = nullptr;
  if (code_size) *code_size = 0;
  if (log) *log = nullptr;
  if (!source || !code || !code_size) return -1;

  // -ffp-contract=off: generated kernels round every fp32 operation on its own, like the host path
  // they are compared against; -packed-fp32-ops off: scalar fp32 code generation only.
  std::vector<std::string> opts = {"--offload-arch=gfx950", "-std=c++17", "-O3", "-ffp-contract=off",
                                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  if (extra_options) {
    std::istringstream iss(extra_options);
    std::string tok;
    while (iss >> tok) opts.push_back(tok);
  }
  std::string key;
  for (auto& o : opts) key += o + " ";
  key.push_back(with_device_lib ? '1' : '0');
  key.push_back('\0');
  key += source;
  {
    std::lock_guard<std::mutex> lock(g_cache_mu);
    auto it = g_code_cache.find(key);
    if (it != g_code_cache.end()) {
      *code = static_cast<char*>(malloc(it->second.size()));
      memcpy(*code, it->second.data(), it->second.size());
      *code_size = it->second.size();
      return 0;
    }
  }

  hiprtcProgram prog       = nullptr;
  const char* header_src[] = {cinn_hip_device_lib_source_text};
  const char* header_name[] = {"cinn_hip_runtime_source.h"};
  hiprtcResult st = hiprtcCreateProgram(&prog, source, "cinn_hip_module.hip", with_device_lib ? 1 : 0,
                                        with_device_lib ? header_src : nullptr, with_device_lib ? header_name : nullptr);
  if (st != HIPRTC_SUCCESS) {
    if (log) *log = DupString(std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(st));
    return static_cast<int>(st);
  }
  std::vector<const char*> copts;
  for (auto& o : opts) copts.push_back(o.c_str());
  st = hiprtcCompileProgram(prog, static_cast<int>(copts.size()), copts.data());
  size_t log_size = 0;
  hiprtcGetProgramLogSize(prog, &log_size);
  if (log && log_size > 1) {
    std::string l(log_size, '\0');
    hiprtcGetProgramLog(prog, &l[0]);
    *log = DupString(l);
  }
  if (st != HIPRTC_SUCCESS) {
    if (log && !*log) *log = DupString(std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(st));
    hiprtcDestroyProgram(&prog);
    return static_cast<int>(st);
  }
  size_t size = 0;
  st          = hiprtcGetCodeSize(prog, &size);
  if (st == HIPRTC_SUCCESS) {
    *code = static_cast<char*>(malloc(size));
    st    = hiprtcGetCode(prog, *code);
  }
  hiprtcDestroyProgram(&prog);
  if (st != HIPRTC_SUCCESS) {
    free(*code);
    *code = nullptr;
    return static_cast<int>(st);
  }
  *code_size = size;
  {
    std::lock_guard<std::mutex> lock(g_cache_mu);
    g_code_cache[key] = std::string(*code, size);
  }
  return 0;
}

}  // extern "C"
