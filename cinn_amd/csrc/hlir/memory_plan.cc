#include "hlir/memory_plan.h"

#include <algorithm>
#include <iterator>
#include <map>

namespace cinn {
namespace hlir {
namespace framework {

size_t PlanMemorySlots(std::vector<MemorySlot>* slots) {
  size_t persistent_bytes = 0;
  int instructions        = 0;
  for (auto& s : *slots) {
    if (s.persistent) {
      s.offset = persistent_bytes;
      persistent_bytes += s.bytes;
    } else {
      instructions = std::max(instructions, s.last + 1);
    }
  }
  std::vector<std::vector<MemorySlot*>> starts(instructions + 1), ends(instructions + 2);
  for (auto& s : *slots)
    if (!s.persistent) {
      starts[s.def].push_back(&s);
      ends[s.last + 1].push_back(&s);
    }
  std::map<size_t, size_t> holes;  // offset -> bytes inside the transient region, coalesced
  size_t peak = 0;                 // size of the transient region: the highest end ever used
  auto release = [&](size_t offset, size_t bytes) {
    auto next = holes.lower_bound(offset);
    if (next != holes.begin()) {
      auto prev = std::prev(next);
      if (prev->first + prev->second == offset) {
        offset = prev->first;
        bytes += prev->second;
        holes.erase(prev);
      }
    }
    if (next != holes.end() && offset + bytes == next->first) {
      bytes += next->second;
      holes.erase(next);
    }
    holes[offset] = bytes;
  };
  for (int i = 0; i < instructions; ++i) {
    for (MemorySlot* s : ends[i]) release(s->offset, s->bytes);
    std::stable_sort(starts[i].begin(), starts[i].end(), [](const MemorySlot* a, const MemorySlot* b) { return a->bytes > b->bytes; });
    for (MemorySlot* s : starts[i]) {
      bool found = false;
      for (auto it = holes.begin(); it != holes.end(); ++it) {
        if (it->second < s->bytes) continue;
        const size_t off = it->first, len = it->second;
        holes.erase(it);
        s->offset = off;
        if (len > s->bytes) holes[off + s->bytes] = len - s->bytes;
        found = true;
        break;
      }
      if (found) continue;
      // grow the region: a hole that touches its end is extended, otherwise the slot goes behind everything
      size_t at = peak;
      if (!holes.empty()) {
        auto tail = std::prev(holes.end());
        if (tail->first + tail->second == peak) {
          at = tail->first;
          holes.erase(tail);
        }
      }
      s->offset = at;
      peak      = at + s->bytes;
    }
  }
  for (auto& s : *slots)
    if (!s.persistent) s.offset += persistent_bytes;
  return persistent_bytes + peak;
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
