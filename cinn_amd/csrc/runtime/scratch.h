// Device scratch owned by the library: what a kernel needs beyond its inputs and outputs (partial sums of a split
// reduction, a transposed copy of an operand, a page of zeros).
//
// One buffer per (device, stream, kind): launches on one stream run in order and may share it, launches on different
// streams may overlap and must not.  A stream's buffers outlive the stream unless its owner calls
// cinn_hip_scratch_release_stream before destroying it; a later stream that the runtime gives the same handle value
// would otherwise inherit them (harmless - they are only scratch - but never returned).  A buffer that has become too small is RETIRED, never freed: a captured graph
// (Program::ExecuteGraph) keeps the addresses its kernel nodes were recorded with, and replays them long after a
// later call on the same stream has asked for more.  Retired buffers stay allocated until
// cinn_hip_scratch_release_retired() - which only a caller that knows no graph refers to them may call - or the end
// of the process.  Nothing here waits for the device.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>

namespace cinn_hip_kernels {

enum class ScratchKind : int { kSplitK = 0, kTranspose = 1 };
constexpr int kScratchKinds = 2;

// At least `bytes` of device memory for launches on `stream`, 256-byte aligned.  Grows by retiring (see above).  While
// `stream` is being captured nothing can be allocated: a request beyond the current capacity aborts with a message
// that says to reserve first (one eager execution of the same calls, or cinn_hip_scratch_reserve).
void* Scratch(ScratchKind kind, size_t bytes, hipStream_t stream);

// 256 bytes of zeros in the current device's memory, allocated and cleared once per device (what masked-out 16-byte
// chunks are read from)
const void* ZeroPage();

}  // namespace cinn_hip_kernels
