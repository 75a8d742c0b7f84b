// Placement of a program's tensors in one allocation (csrc/hlir/memory_plan.h): on random lifetimes no two slots that
// are alive at the same time may share a byte, persistent slots share with nobody, the allocation is never larger than
// the sum of the slots and never smaller than the largest set of slots alive at once; plus hand-made cases with known
// optimal sizes.
#include <algorithm>
#include <cstdio>
#include <random>
#include <vector>

#include "hlir/memory_plan.h"

using cinn::hlir::framework::MemorySlot;
using cinn::hlir::framework::PlanMemorySlots;

static int failures = 0;
#define EXPECT(cond)                                                \
  do {                                                              \
    if (!(cond)) {                                                  \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      ++failures;                                                   \
    }                                                               \
  } while (0)

static MemorySlot Slot(size_t bytes, int def, int last, bool persistent = false) {
  MemorySlot s;
  s.bytes = bytes, s.def = def, s.last = last, s.persistent = persistent;
  return s;
}

static bool AliveTogether(const MemorySlot& a, const MemorySlot& b) {
  if (a.persistent || b.persistent) return true;
  return a.def <= b.last && b.def <= a.last;  // closed ranges: an output never takes an input's bytes
}

static void CheckPlan(const std::vector<MemorySlot>& slots, size_t total) {
  size_t sum = 0;
  for (auto& s : slots) {
    sum += s.bytes;
    EXPECT(s.offset + s.bytes <= total);
  }
  EXPECT(total <= sum);
  for (size_t i = 0; i < slots.size(); ++i)
    for (size_t j = i + 1; j < slots.size(); ++j)
      if (AliveTogether(slots[i], slots[j])) {
        const bool apart = slots[i].offset + slots[i].bytes <= slots[j].offset || slots[j].offset + slots[j].bytes <= slots[i].offset;
        if (!apart) {
          std::printf("FAILED: slots %zu [%d,%d] and %zu [%d,%d] overlap in memory\n", i, slots[i].def, slots[i].last, j, slots[j].def,
                      slots[j].last);
          ++failures;
          return;
        }
      }
  // lower bound: the most bytes alive at one instruction
  int n = 0;
  for (auto& s : slots)
    if (!s.persistent) n = std::max(n, s.last + 1);
  size_t persistent = 0, most = 0;
  for (auto& s : slots)
    if (s.persistent) persistent += s.bytes;
  for (int i = 0; i < n; ++i) {
    size_t alive = 0;
    for (auto& s : slots)
      if (!s.persistent && s.def <= i && i <= s.last) alive += s.bytes;
    most = std::max(most, alive);
  }
  EXPECT(total >= persistent + most);
}

int main() {
  {  // a chain a -> b -> c -> d of equal sizes ping-pongs between two slices
    std::vector<MemorySlot> s = {Slot(1024, 0, 1), Slot(1024, 1, 2), Slot(1024, 2, 3), Slot(1024, 3, 4)};
    const size_t total        = PlanMemorySlots(&s);
    EXPECT(total == 2048);
    EXPECT(s[0].offset == s[2].offset && s[1].offset == s[3].offset && s[0].offset != s[1].offset);
    CheckPlan(s, total);
  }
  {  // a residual block: x lives across the three layers of the main branch
    std::vector<MemorySlot> s = {Slot(4096, 0, 4), Slot(1024, 1, 2), Slot(1024, 2, 3), Slot(4096, 3, 4), Slot(4096, 4, 5)};
    const size_t total        = PlanMemorySlots(&s);
    CheckPlan(s, total);
    EXPECT(total <= 4096 * 3 + 2048);
  }
  {  // persistent slots come first and are never shared; a slot nobody reads lives for its own instruction only
    std::vector<MemorySlot> s = {Slot(512, 0, 0, true), Slot(256, 0, 0), Slot(256, 1, 1), Slot(768, 0, 9, true)};
    const size_t total        = PlanMemorySlots(&s);
    EXPECT(s[0].offset == 0 && s[3].offset == 512 && s[1].offset == 1280 && s[2].offset == 1280 && total == 1536);
    CheckPlan(s, total);
  }
  {  // nothing to place
    std::vector<MemorySlot> s;
    EXPECT(PlanMemorySlots(&s) == 0);
  }
  std::mt19937 rng(12345);
  for (int round = 0; round < 300; ++round) {
    const int instructions = 1 + rng() % 60;
    const int count        = 1 + rng() % 80;
    std::vector<MemorySlot> s;
    for (int i = 0; i < count; ++i) {
      const int def  = rng() % instructions;
      const int last = def + (rng() % 4 == 0 ? rng() % (instructions - def) : std::min<int>(instructions - 1 - def, rng() % 3));
      s.push_back(Slot(256 * (1 + rng() % 64), def, last, rng() % 10 == 0));
    }
    const size_t total = PlanMemorySlots(&s);
    CheckPlan(s, total);
    if (failures) break;
  }
  if (failures) return 1;
  std::printf("ok\n");
  return 0;
}
