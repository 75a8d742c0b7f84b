// Host stubs beyond the pre-compiled trampolines: 4096 slots are taken first, every further stub is a generated
// thunk; all of them must call their own closure with the arguments they were given, and released ones are reused.
#include <cstdint>
#include <algorithm>
#include <cstdio>
#include <vector>

#include "backends/host_stub.h"

using cinn::backends::HostStubPool;

int main() {
  auto& pool      = HostStubPool::Global();
  const int total = HostStubPool::kSlots + 700;
  const int before = pool.in_use();
  std::vector<long> hits(total, 0);
  std::vector<lower_func_ptr_g> fns;
  for (int i = 0; i < total; ++i) {
    fns.push_back(pool.Acquire([i, &hits](void* args, int32_t n, void* stream) {
      hits[i] += n + static_cast<long>(reinterpret_cast<intptr_t>(args)) + 2 * static_cast<long>(reinterpret_cast<intptr_t>(stream));
    }));
  }
  int failures = 0;
  if (pool.in_use() != HostStubPool::kSlots) { std::printf("FAILED: %d slots in use\n", pool.in_use()); ++failures; }
  if (pool.thunks_in_use() != total - (HostStubPool::kSlots - before)) {
    std::printf("FAILED: %d thunks in use\n", pool.thunks_in_use());
    ++failures;
  }
  for (int i = 0; i < total; ++i) fns[i](reinterpret_cast<void*>(static_cast<intptr_t>(i)), 7, reinterpret_cast<void*>(static_cast<intptr_t>(3)));
  for (int i = 0; i < total; ++i)
    if (hits[i] != 7 + i + 6) { std::printf("FAILED: stub %d saw %ld\n", i, hits[i]); ++failures; break; }
  // every function pointer is distinct
  std::vector<lower_func_ptr_g> sorted = fns;
  std::sort(sorted.begin(), sorted.end());
  if (std::adjacent_find(sorted.begin(), sorted.end()) != sorted.end()) { std::printf("FAILED: two stubs share an address\n"); ++failures; }
  // release the thunks and take them again: the freed code slots are reused, the new closures are the ones called
  const int thunks = pool.thunks_in_use();
  for (int i = HostStubPool::kSlots - before; i < total; ++i) pool.Release(fns[i]);
  if (pool.thunks_in_use() != 0) { std::printf("FAILED: thunks left after release\n"); ++failures; }
  long again = 0;
  std::vector<lower_func_ptr_g> second;
  for (int i = 0; i < thunks; ++i) second.push_back(pool.Acquire([&again](void*, int32_t n, void*) { again += n; }));
  for (auto fn : second) fn(nullptr, 2, nullptr);
  if (again != 2L * thunks) { std::printf("FAILED: reused thunks saw %ld\n", again); ++failures; }
  for (auto fn : second) pool.Release(fn);
  for (int i = 0; i < HostStubPool::kSlots - before; ++i) pool.Release(fns[i]);
  if (pool.in_use() != before || pool.thunks_in_use() != 0) { std::printf("FAILED: pool not back to its start\n"); ++failures; }
  if (failures) return 1;
  std::printf("ok\n");
  return 0;
}
