// hiprtc wrapper: HIP source -> gfx950 code object.  Role of nvrtc::Compiler
// (cinn/backends/nvrtc/nvrtc_util.cc:40-152): fixed option set, device library handed over as an
// in-memory header, compile log returned on failure.  Identical sources are served from an
// in-process cache so a program that is rebuilt does not pay hiprtc twice, and - when
// FLAGS_cinn_hip_code_cache_dir names a directory - from code objects kept there by earlier processes
// (the reference re-parses its device header and recompiles every module on every start).
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
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

// ---- code objects on disk ------------------------------------------------------------------------------------------
// <dir>/<h1><h2>.hsaco = header {magic, key bytes, check hash, code bytes} + code.  h1 / h2 / check are three
// independent 64-bit FNV-1a style hashes over what determines the code object: hiprtc's version, the options, the
// device library text (when included) and the source.  A file whose header does not match is ignored and rewritten.
struct DiskHeader {
  uint64_t magic;
  uint64_t key_bytes;
  uint64_t check;
  uint64_t code_bytes;
};
constexpr uint64_t kDiskMagic = 0x3130304f43484e43ull;  // "CNHCO001"

uint64_t Fnv(const char* data, size_t n, uint64_t h, uint64_t prime) {
  for (size_t i = 0; i < n; ++i) h = (h ^ static_cast<unsigned char>(data[i])) * prime;
  return h;
}

struct DiskKey {
  uint64_t h1, h2, check, bytes;
};

DiskKey MakeDiskKey(const std::string& key, bool with_device_lib) {
  int major = 0, minor = 0;
  hiprtcVersion(&major, &minor);
  std::string version = "hiprtc " + std::to_string(major) + "." + std::to_string(minor) + "\n";
  const uint64_t seeds[3]  = {0xcbf29ce484222325ull, 0x84222325cbf29ce4ull, 0x9e3779b97f4a7c15ull};
  const uint64_t primes[3] = {0x100000001b3ull, 0x1000000016full, 0x10000000233ull};
  uint64_t h[3];
  size_t bytes = version.size() + key.size();
  for (int i = 0; i < 3; ++i) {
    h[i] = Fnv(version.data(), version.size(), seeds[i], primes[i]);
    h[i] = Fnv(key.data(), key.size(), h[i], primes[i]);
    if (with_device_lib) h[i] = Fnv(cinn_hip_device_lib_source_text, strlen(cinn_hip_device_lib_source_text), h[i], primes[i]);
  }
  if (with_device_lib) bytes += strlen(cinn_hip_device_lib_source_text);
  return {h[0], h[1], h[2], bytes};
}

const char* DiskCacheDir() {
  const char* dir = getenv("FLAGS_cinn_hip_code_cache_dir");
  return dir && *dir ? dir : nullptr;
}

std::string DiskPath(const char* dir, const DiskKey& k) {
  char name[64];
  snprintf(name, sizeof(name), "/%016llx%016llx.hsaco", (unsigned long long)k.h1, (unsigned long long)k.h2);
  return std::string(dir) + name;
}

bool DiskLoad(const char* dir, const DiskKey& k, std::string* code) {
  FILE* f = fopen(DiskPath(dir, k).c_str(), "rb");
  if (!f) return false;
  DiskHeader hd{};
  bool ok = fread(&hd, sizeof(hd), 1, f) == 1 && hd.magic == kDiskMagic && hd.key_bytes == k.bytes &&
            hd.check == k.check && hd.code_bytes > 0 && hd.code_bytes < (1ull << 31);
  if (ok) {
    code->resize(hd.code_bytes);
    ok = fread(&(*code)[0], 1, hd.code_bytes, f) == hd.code_bytes && fgetc(f) == EOF;
  }
  fclose(f);
  return ok;
}

// written under a temporary name and renamed, so that a concurrent reader never sees half a file; failures are
// silent (the cache is an optimisation)
void DiskStore(const char* dir, const DiskKey& k, const char* code, size_t size) {
  mkdir(dir, 0777);
  const std::string path = DiskPath(dir, k);
  const std::string tmp  = path + ".tmp." + std::to_string(getpid());
  FILE* f                = fopen(tmp.c_str(), "wb");
  if (!f) return;
  DiskHeader hd{kDiskMagic, k.bytes, k.check, size};
  bool ok = fwrite(&hd, sizeof(hd), 1, f) == 1 && fwrite(code, 1, size, f) == size;
  ok      = (fclose(f) == 0) && ok;
  if (!ok || rename(tmp.c_str(), path.c_str()) != 0) remove(tmp.c_str());
}
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
  const char* cache_dir = DiskCacheDir();
  DiskKey disk_key{};
  if (cache_dir) {
    disk_key = MakeDiskKey(key, with_device_lib != 0);
    std::string image;
    if (DiskLoad(cache_dir, disk_key, &image)) {
      *code = static_cast<char*>(malloc(image.size()));
      memcpy(*code, image.data(), image.size());
      *code_size = image.size();
      std::lock_guard<std::mutex> lock(g_cache_mu);
      g_code_cache[key] = std::move(image);
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
  if (cache_dir) DiskStore(cache_dir, disk_key, *code, size);
  return 0;
}

}  // extern "C"
