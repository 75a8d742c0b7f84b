"""How fast do direct-to-LDS loads land when every CU pulls at once?  A measurement behind the convolution kernels that
keep their input patch in LDS (conv_patch_mfma.hip), runnable on its own:
    python bench_lds_fetch.py
A kernel compiled through the library's own hiprtc entry points does nothing but issue the loads of one block of the
64 -> 64 3x3 layer at batch 32 (224 blocks of 512 threads, one per CU): 64 KiB of filter that every block wants (the
same addresses for all) and 72 KiB of its own band of a cold input (launches rotate over 21 input sets, 270 MB), 1 KiB
per load instruction (`global_load_lds_dwordx4`, 16 bytes per lane), every wavefront its share in one burst.  Each
wavefront then waits for its loads one by one (`s_waitcnt vmcnt(n)`, loads complete in issue order) and stores the
100 MHz counter after each.  Reported per mode (filter + patch, patch only, filter only; and the same loads into
registers with `global_load_dwordx4` instead of into LDS): microseconds per launch, when
the first load of every wavefront of a block has landed, the interval between consecutive loads of a wavefront (eight
wavefronts: 8 KiB per CU and interval) and the rate that interval means per CU and over the 224 CUs."""
import ctypes
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SOURCE = r"""
#define VMCNT(n) ((((n) & 15) | (((n) >> 4) << 14)) | 0x0F70)
__device__ __forceinline__ void AsyncCopy16(const void* src, unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr_uniform), "v"(src) : "memory");
}
__device__ __forceinline__ void WaitN(int n) {
  switch (n) {
#define C(k) case k: __builtin_amdgcn_s_waitcnt(VMCNT(k)); break;
    C(0) C(1) C(2) C(3) C(4) C(5) C(6) C(7) C(8) C(9) C(10) C(11) C(12) C(13) C(14) C(15) C(16) C(17) C(18) C(19) C(20)
#undef C
    default: __builtin_amdgcn_s_waitcnt(VMCNT(0)); break;
  }
}
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 LoadToRegisters(const void* src) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(src) : "memory");
  return v;
}
// mode 0: filter and patch, 1: patch only, 2: filter only; 4 + mode: the same loads into registers instead of LDS.  stamps: 32 words per wavefront - block start, number of
// loads, the time after each load has landed
extern "C" __global__ void __launch_bounds__(512) lds_fetch_probe(const char* x, const char* w, long long* stamps, int mode) {
  __shared__ __attribute__((aligned(1024))) char lds[160 * 1024];
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)lds);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int img = blockIdx.x / 7, band = blockIdx.x % 7;
  const long long t0 = __builtin_amdgcn_s_memrealtime();
  int issued = 0;
  const bool to_registers = mode >= 4;
  mode &= 3;
  u32x4 regs[17];
  const int first_row = band * 8 - 1 < 0 ? 0 : band * 8 - 1;
  const char* src = x + ((long long)img * 56 * 56 + (long long)first_row * 56) * 128;
  if (to_registers) {
    if (mode != 1)
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        regs[t] = LoadToRegisters(w + (t * 8 + wave) * 1024 + lane * 16);
        ++issued;
      }
    if (mode != 2)
#pragma unroll
      for (int i = 0; i < 9; ++i) {
        regs[8 + i] = LoadToRegisters(src + (wave + 8 * i) * 1024 + lane * 16);
        ++issued;
      }
  } else {
    if (mode != 1)
      for (int t = 0; t < 8; ++t) {
        AsyncCopy16(w + (t * 8 + wave) * 1024 + lane * 16, lds_addr + 96 * 1024 + (t * 8 + wave) * 1024);
        ++issued;
      }
    if (mode != 2)
      for (int q = wave; q < 72; q += 8) {
        AsyncCopy16(src + q * 1024 + lane * 16, lds_addr + q * 1024);
        ++issued;
      }
  }
  long long* out = stamps + ((long long)blockIdx.x * 8 + wave) * 32;
  long long t[24];
  int n = 0;
  for (int k = issued - 1; k >= 0; --k) {
    WaitN(k);
    t[n++] = __builtin_amdgcn_s_memrealtime();
  }
  if (to_registers) {  // keep the loads alive
    unsigned sum = 0;
#pragma unroll
    for (int i = 0; i < 17; ++i) asm volatile("" : "+v"(regs[i]));
#pragma unroll
    for (int i = 0; i < 17; ++i) sum += regs[i][0];
    if (sum == 0x12345678u) out[31] = sum;
  }
  if (lane == 0) {
    out[0] = t0;
    out[1] = n;
    for (int i = 0; i < n; ++i) out[2 + i] = t[i];
  }
}
"""


def measure(launches=200, sets=21):
    from cinn_amd import _lib, runtime
    lib = _lib.load()
    lib.cinn_call_cuda_kernel.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int] + [ctypes.c_int] * 6 + [ctypes.c_void_p]
    module = runtime.Module(runtime.rtc_compile(SOURCE, with_device_lib=False))
    fn = module.get_function("lds_fetch_probe")
    blocks = 224
    x_elems = 32 * 56 * 56 * 64 + (1 << 19)  # fp16 elements, with room behind the last band
    xs = [runtime.DeviceBuffer.from_numpy(np.ones(x_elems, np.float16)) for _ in range(sets)]
    ws = [runtime.DeviceBuffer.from_numpy(np.ones(64 * 1024, np.float16)) for _ in range(sets)]
    stamps = runtime.DeviceBuffer((blocks * 8, 32), "int64")
    stream = runtime.Stream()
    out = {}
    for mode, name in ((0, "filter_and_patch"), (1, "patch_only"), (2, "filter_only"),
                       (4, "filter_and_patch_to_registers"), (5, "patch_only_to_registers"), (6, "filter_only_to_registers")):
        pods = []
        for i in range(sets):
            arr = (runtime.cinn_pod_value_t * 4)()
            for j, b in enumerate((xs[i], ws[i], stamps)):
                lib.cinn_hip_pod_from_buffer(ctypes.byref(arr[j]), ctypes.byref(b.buffer))
            lib.cinn_hip_pod_from_int32(ctypes.byref(arr[3]), ctypes.c_int32(mode))
            pods.append(arr)

        def launch(i):
            lib.cinn_call_cuda_kernel(fn, pods[i % sets], 4, blocks, 1, 1, 512, 1, 1, stream.handle)

        for i in range(launches):
            launch(i)
        stream.synchronize()
        s, e = runtime.Event(), runtime.Event()
        s.record(stream)
        for i in range(launches):
            launch(i)
        e.record(stream)
        e.synchronize()
        t = stamps.numpy().reshape(blocks, 8, 32)
        n = int(t[0, 0, 1])
        start = t[:, :, 0].min(axis=1)                                   # a block's first wavefront
        landed = (t[:, :, 2:2 + n].max(axis=1) - start[:, None]) / 100.0  # load i of every wavefront of the block, us
        med = np.median(landed, axis=0)
        interval = float(np.median(np.diff(med))) if n > 1 else 0.0
        per_cu = 8 * 1024 / (interval * 1e-6) / 1e9 if interval > 0 else 0.0
        out[name] = dict(us_per_launch=round(s.elapsed_ms(e) * 1e3 / launches, 2), loads_per_wavefront=n,
                         first_load_landed_us=round(float(med[0]), 2), last_load_landed_us=round(float(med[-1]), 2),
                         last_load_landed_us_slowest_block=round(float(landed[:, -1].max()), 2),
                         interval_between_loads_us=round(interval, 3), GB_per_s_per_CU=round(per_cu, 1),
                         TB_per_s_over_224_CUs=round(per_cu * blocks / 1e3, 2))
    return out


if __name__ == "__main__":
    print(json.dumps(measure()))
