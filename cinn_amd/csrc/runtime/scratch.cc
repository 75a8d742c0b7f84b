#include "runtime/scratch.h"

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

struct Buffer {
  void* data{nullptr};
  size_t capacity{0};
};

struct Arena {
  std::mutex mu;
  std::map<std::tuple<int, hipStream_t, int>, Buffer> live;  // (device, stream, kind)
  std::vector<Buffer> retired;
  size_t retired_bytes{0};
};

Arena& TheArena() {
  static Arena* arena = new Arena;  // leaked on purpose: intrinsics may run during static teardown
  return *arena;
}

int CurrentDevice() {
  int device = 0;
  CINN_HIP_CALL(hipGetDevice(&device));
  return device;
}

bool Capturing(hipStream_t stream) {
  if (!stream) return false;  // the null stream cannot be captured
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  CINN_HIP_CALL(hipStreamIsCapturing(stream, &status));
  return status != hipStreamCaptureStatusNone;
}

// caller holds the arena's mutex
void* Ensure(Arena& arena, ScratchKind kind, size_t bytes, hipStream_t stream) {
  Buffer& b = arena.live[{CurrentDevice(), stream, static_cast<int>(kind)}];
  if (bytes <= b.capacity) return b.data;
  CINN_RT_CHECK(!Capturing(stream),
                "library scratch (kind %d) must grow from %zu to %zu bytes while its stream is being captured; run the "
                "same calls once eagerly, or call cinn_hip_scratch_reserve, before the capture",
                static_cast<int>(kind), b.capacity, bytes);
  // at least double, so that the retired buffers of a stream add up to less than its live one
  size_t capacity = bytes > 2 * b.capacity ? bytes : 2 * b.capacity;
  capacity        = (capacity + 255) & ~static_cast<size_t>(255);
  if (b.data) {
    arena.retired.push_back(b);
    arena.retired_bytes += b.capacity;
  }
  CINN_HIP_CALL(hipMalloc(&b.data, capacity));
  b.capacity = capacity;
  return b.data;
}

}  // namespace

void* Scratch(ScratchKind kind, size_t bytes, hipStream_t stream) {
  Arena& arena = TheArena();
  std::lock_guard<std::mutex> lock(arena.mu);
  return Ensure(arena, kind, bytes ? bytes : 1, stream);
}

const void* ZeroPage() {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* pages[kMaxDevices];  // one page per device, allocated and cleared on its first use there
  const int device = CurrentDevice();
  CINN_RT_CHECK(device >= 0 && device < kMaxDevices, "device %d: the library keeps a page of zeros for at most %d devices", device,
                kMaxDevices);
  std::lock_guard<std::mutex> lock(mu);
  if (!pages[device]) {
    CINN_HIP_CALL(hipMalloc(&pages[device], 256));
    CINN_HIP_CALL(hipMemset(pages[device], 0, 256));  // synchronous with respect to the host for device memory
  }
  return pages[device];
}

}  // namespace cinn_hip_kernels

extern "C" {

int cinn_hip_scratch_reserve(void* stream, size_t split_k_bytes, size_t transpose_bytes) {
  using namespace cinn_hip_kernels;
  ZeroPage();  // allocated and cleared on first use, which must not fall into a capture either
  Arena& arena = TheArena();
  std::lock_guard<std::mutex> lock(arena.mu);
  if (split_k_bytes) Ensure(arena, ScratchKind::kSplitK, split_k_bytes, static_cast<hipStream_t>(stream));
  if (transpose_bytes) Ensure(arena, ScratchKind::kTranspose, transpose_bytes, static_cast<hipStream_t>(stream));
  return 0;
}

int cinn_hip_scratch_info(void* stream, size_t* split_k_capacity, size_t* transpose_capacity, size_t* retired_bytes) {
  using namespace cinn_hip_kernels;
  Arena& arena = TheArena();
  std::lock_guard<std::mutex> lock(arena.mu);
  auto capacity = [&](ScratchKind kind) -> size_t {
    auto it = arena.live.find({CurrentDevice(), static_cast<hipStream_t>(stream), static_cast<int>(kind)});
    return it == arena.live.end() ? 0 : it->second.capacity;
  };
  if (split_k_capacity) *split_k_capacity = capacity(ScratchKind::kSplitK);
  if (transpose_capacity) *transpose_capacity = capacity(ScratchKind::kTranspose);
  if (retired_bytes) *retired_bytes = arena.retired_bytes;
  return 0;
}

int cinn_hip_scratch_release_stream(void* stream) {
  using namespace cinn_hip_kernels;
  Arena& arena = TheArena();
  std::lock_guard<std::mutex> lock(arena.mu);
  const int device = CurrentDevice();
  for (int kind = 0; kind < kScratchKinds; ++kind) {
    auto it = arena.live.find({device, static_cast<hipStream_t>(stream), kind});
    if (it == arena.live.end()) continue;
    if (it->second.data) {  // a graph captured on the stream may still hold the address: retire, do not free
      arena.retired.push_back(it->second);
      arena.retired_bytes += it->second.capacity;
    }
    arena.live.erase(it);
  }
  return 0;
}

int cinn_hip_scratch_release_retired(void) {
  using namespace cinn_hip_kernels;
  Arena& arena = TheArena();
  std::lock_guard<std::mutex> lock(arena.mu);
  int status = 0;
  for (auto& b : arena.retired) {
    hipError_t e = hipFree(b.data);
    if (e != hipSuccess && status == 0) status = static_cast<int>(e);
  }
  arena.retired.clear();
  arena.retired_bytes = 0;
  return status;
}

}  // extern "C"
