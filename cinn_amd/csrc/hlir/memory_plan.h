// Placement of a compiled program's tensors inside one device allocation.
//
// The reference gives every tensor a buffer of its own (cinn/hlir/framework/memory.cc:43-53, tensor.h:64-82,
// buffer.cc).  Here a program's instructions run in program order on one stream, so a value that run instruction
// `def` produces and run instruction `last` reads for the last time needs its bytes only in between: two values whose
// [def, last] ranges do not intersect may share them.  Kernels declare their operands __restrict__, hence the ranges
// are closed: an output never takes the bytes of an input of the same instruction.
#pragma once
#include <cstddef>
#include <vector>

namespace cinn {
namespace hlir {
namespace framework {

struct MemorySlot {
  size_t bytes{0};       // a multiple of the alignment the caller wants
  bool persistent{false};  // keeps bytes of its own for the whole life of the program
  int def{0}, last{0};   // run-instruction indices, def <= last; ignored for persistent slots
  size_t offset{0};      // result: byte offset inside the allocation
};

// Fills `offset` of every slot and returns the size of the allocation.  Persistent slots come first, one after the
// other in the order given; transient ones follow in a region that is walked in instruction order: a slot is freed
// after instruction `last`, a new one takes the lowest hole that fits (first fit, holes coalesced, larger slots of
// one instruction first) and the region grows when none does.
size_t PlanMemorySlots(std::vector<MemorySlot>* slots);

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
