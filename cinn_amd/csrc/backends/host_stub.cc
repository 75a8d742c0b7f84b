#include "backends/host_stub.h"

#include <sys/mman.h>

#include <array>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

namespace cinn {
namespace backends {

// ---------------------------------------------------------------------------------------------------
// extern API registry
// ---------------------------------------------------------------------------------------------------
namespace {

int I(const BakedArg& a) { return static_cast<int>(a.i); }
float F(const BakedArg& a) { return static_cast<float>(a.f); }
bool B(const BakedArg& a) { return a.i != 0; }

// Argument lists below follow the call the lowering builds: (kernel_args, kernel_args_num, <constants...>,
// kernel_stream).  Index 0/1 and the last entry are the pass-through arguments.
void InvokeHipKernel(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_hip_kernel(a[0].p, args, n, I(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), stream);
}
void InvokeCublas(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cublas(args, n, B(a[2]), B(a[3]), B(a[4]), F(a[5]), F(a[6]), I(a[7]), I(a[8]), I(a[9]), I(a[10]), I(a[11]),
                   I(a[12]), I(a[13]), I(a[14]), stream);
}
void InvokeConv2dForward(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cudnn_conv2d_forward(args, n, I(a[2]), F(a[3]), F(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                                 I(a[10]), I(a[11]), I(a[12]), I(a[13]), I(a[14]), I(a[15]), I(a[16]), I(a[17]),
                                 I(a[18]), I(a[19]), I(a[20]), I(a[21]), I(a[22]), I(a[23]), stream);
}
void InvokeConv2dBnRelu(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_hip_conv2d_bn_relu(args, n, I(a[2]), I(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                               I(a[10]), I(a[11]), I(a[12]), I(a[13]), I(a[14]), I(a[15]), I(a[16]), I(a[17]),
                               I(a[18]), I(a[19]), I(a[20]), I(a[21]), I(a[22]), stream);
}
void InvokeConv2dBnReluChain(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_hip_conv2d_bn_relu_chain(args, n, I(a[2]), I(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), stream);
}
void InvokeConv2dPairChain(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_hip_conv2d_pair_chain(args, n, I(a[2]), I(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]), stream);
}
void InvokeConv2dPointwisePair(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_hip_conv2d_pointwise_pair(args, n, I(a[2]), I(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]), I(a[10]),
                                      I(a[11]), I(a[12]), stream);
}
void InvokePool2dForward(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cudnn_pool2d_forward(args, n, I(a[2]), I(a[3]), F(a[4]), F(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                                 I(a[10]), I(a[11]), I(a[12]), I(a[13]), I(a[14]), I(a[15]), I(a[16]), I(a[17]),
                                 I(a[18]), I(a[19]), stream);
}
void InvokeSoftmaxForward(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cudnn_softmax_forward(args, n, I(a[2]), I(a[3]), F(a[4]), F(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                                  I(a[10]), I(a[11]), I(a[12]), I(a[13]), stream);
}
void InvokeArgsort(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_hip_argsort(args, n, I(a[2]), I(a[3]), I(a[4]), I(a[5]), I(a[6]), stream);
}
void InvokeBatchedCublas(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_batched_cublas(args, n, I(a[2]), B(a[3]), B(a[4]), B(a[5]), F(a[6]), F(a[7]), I(a[8]), I(a[9]), I(a[10]),
                           I(a[11]), I(a[12]), I(a[13]), I(a[14]), I(a[15]), stream);
}
// the two convolution gradients share the forward call's argument list (format, alpha, beta, 19 extents)
template <decltype(&cinn_call_cudnn_conv2d_backward_data) Fn>
void InvokeConv2dBackward(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  Fn(args, n, I(a[2]), F(a[3]), F(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]), I(a[10]), I(a[11]), I(a[12]),
     I(a[13]), I(a[14]), I(a[15]), I(a[16]), I(a[17]), I(a[18]), I(a[19]), I(a[20]), I(a[21]), I(a[22]), I(a[23]), stream);
}
void InvokePool2dBackward(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cudnn_pool2d_backward(args, n, I(a[2]), I(a[3]), F(a[4]), F(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                                  I(a[10]), I(a[11]), I(a[12]), I(a[13]), I(a[14]), I(a[15]), I(a[16]), I(a[17]),
                                  I(a[18]), I(a[19]), stream);
}
void InvokeSoftmaxBackward(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cudnn_softmax_backward(args, n, I(a[2]), I(a[3]), F(a[4]), F(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                                   I(a[10]), I(a[11]), I(a[12]), I(a[13]), stream);
}
void InvokeMemset(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cuda_memset(args, n, I(a[2]), static_cast<size_t>(a[3].i), stream);
}
void InvokeMemcpy(const std::vector<BakedArg>& a, void* args, int32_t n, void* stream) {
  cinn_call_cuda_memcpy(args, n, static_cast<size_t>(a[2].i), stream);
}

}  // namespace

ExternApiRegistry::ExternApiRegistry() {
  // kernel launch: (kernel_fn, kernel_args, kernel_args_num, gx, gy, gz, bx, by, bz, kernel_stream)
  Register("cinn_call_hip_kernel", InvokeHipKernel, 10);
  Register("cinn_call_cuda_kernel", InvokeHipKernel, 10);
  Register("cinn_call_cublas", InvokeCublas, 16);
  Register("cinn_call_cudnn_conv2d_forward", InvokeConv2dForward, 25);
  Register("cinn_call_hip_conv2d_bn_relu", InvokeConv2dBnRelu, 24);
  // (kernel_args, kernel_args_num, relu bits, n, h, w, input_c, middle_c, output_c, kernel_stream)
  Register("cinn_call_hip_conv2d_bn_relu_chain", InvokeConv2dBnReluChain, 10);
  // (kernel_args, kernel_args_num, relu, n, h, w, c, second h, w, c, second stride h, w, output_c, kernel_stream)
  Register("cinn_call_hip_conv2d_pointwise_pair", InvokeConv2dPointwisePair, 14);
  // (kernel_args, kernel_args_num, relu bits, n, h, w, input_c, second_c, middle_c, output_c, kernel_stream)
  Register("cinn_call_hip_conv2d_pair_chain", InvokeConv2dPairChain, 11);
  Register("cinn_call_cudnn_pool2d_forward", InvokePool2dForward, 21);
  Register("cinn_call_cudnn_softmax_forward", InvokeSoftmaxForward, 15);
  // (kernel_args, kernel_args_num, outer, size, inner, is_ascend, outputs, kernel_stream)
  Register("cinn_call_hip_argsort", InvokeArgsort, 8);
  // (kernel_args, kernel_args_num, opside, trans_a, trans_b, trans_o, alpha, beta, a1..a4, b1..b4, kernel_stream)
  Register("cinn_call_batched_cublas", InvokeBatchedCublas, 17);
  Register("cinn_call_cudnn_conv2d_backward_data", InvokeConv2dBackward<&cinn_call_cudnn_conv2d_backward_data>, 25);
  Register("cinn_call_cudnn_conv2d_backward_filter", InvokeConv2dBackward<&cinn_call_cudnn_conv2d_backward_filter>, 25);
  Register("cinn_call_cudnn_pool2d_backward", InvokePool2dBackward, 21);
  Register("cinn_call_cudnn_softmax_backward", InvokeSoftmaxBackward, 15);
  Register("cinn_call_cuda_memset", InvokeMemset, 5);
  Register("cinn_call_cuda_memcpy", InvokeMemcpy, 4);
}

ExternApiRegistry& ExternApiRegistry::Global() {
  static ExternApiRegistry r;
  return r;
}
void ExternApiRegistry::Register(const std::string& name, ApiInvoker invoker, size_t num_call_args) {
  table_[name] = Entry{invoker, num_call_args};
}
ApiInvoker ExternApiRegistry::Find(const std::string& name, size_t* num_call_args) const {
  auto it = table_.find(name);
  if (it == table_.end()) return nullptr;
  if (num_call_args) *num_call_args = it->second.num_call_args;
  return it->second.invoker;
}
std::vector<std::string> ExternApiRegistry::Names() const {
  std::vector<std::string> out;
  for (auto& kv : table_) out.push_back(kv.first);
  return out;
}

// ---------------------------------------------------------------------------------------------------
// trampoline pool
// ---------------------------------------------------------------------------------------------------
namespace {
struct PoolState {
  std::mutex mu;
  std::array<HostStubPool::Closure, HostStubPool::kSlots> closures;
  std::array<bool, HostStubPool::kSlots> used{};
  int in_use{0};
  int next_hint{0};
};
PoolState& State() {
  static PoolState* s = new PoolState;  // intentionally leaked: stubs may run during static teardown
  return *s;
}

template <int Slot>
void Trampoline(void* args, int32_t num_args, void* stream) {
  State().closures[Slot](args, num_args, stream);
}
template <int... Slots>
constexpr std::array<lower_func_ptr_g, sizeof...(Slots)> MakeTable(std::integer_sequence<int, Slots...>) {
  return {{&Trampoline<Slots>...}};
}
const std::array<lower_func_ptr_g, HostStubPool::kSlots>& Table() {
  static const auto table = MakeTable(std::make_integer_sequence<int, HostStubPool::kSlots>{});
  return table;
}
}  // namespace

// ---- stubs beyond the pre-compiled slots: generated thunks ---------------------------------------------------------
namespace {
#if defined(__x86_64__)
void ThunkDispatch(void* args, int32_t num_args, void* stream, HostStubPool::Closure* closure) {
  (*closure)(args, num_args, stream);
}

// A thunk is position-independent code that never changes once written:
//   mov rcx, [rip + d0]   ; its closure, from the thunk's slot in a data region that follows the code region
//   mov rax, [rip + d1]   ; &ThunkDispatch, same slot
//   jmp rax               ; the stub's own three arguments stay in rdi, esi, rdx
// A region's code is generated in full while it is mapped read + write, then made read + execute for good; only the
// data slots (never executable) are written afterwards.  No page is ever writable and executable at once, and no
// page's protection changes while a stub on it may be running.
constexpr size_t kThunkBytes  = 32;
constexpr size_t kThunkRegion = 1 << 16;                       // code bytes per region, and data bytes after them
constexpr size_t kThunksPerRegion = kThunkRegion / kThunkBytes;
struct ThunkSlot {
  HostStubPool::Closure* closure;
  void (*dispatch)(void*, int32_t, void*, HostStubPool::Closure*);
};
static_assert(sizeof(ThunkSlot) * kThunksPerRegion <= kThunkRegion, "the data region holds one slot per thunk");

struct ThunkState {
  std::vector<unsigned char*> regions;
  size_t used_in_last{kThunksPerRegion};
  std::vector<unsigned char*> free_list;
  std::map<lower_func_ptr_g, HostStubPool::Closure*> live;
};
ThunkState& Thunks() {
  static ThunkState* s = new ThunkState;  // leaked like the pool: stubs may run during static teardown
  return *s;
}

ThunkSlot* SlotOf(unsigned char* code) {
  const uintptr_t addr   = reinterpret_cast<uintptr_t>(code);
  const uintptr_t region = addr & ~static_cast<uintptr_t>(kThunkRegion - 1);  // regions are aligned to their size
  return reinterpret_cast<ThunkSlot*>(region + kThunkRegion) + (addr - region) / kThunkBytes;
}

// a new region with all its thunks written; null when the system refuses the mapping or the protection change
unsigned char* NewThunkRegion() {
  // twice the span, so that an aligned code + data pair lies inside whatever address comes back
  const size_t span = 4 * kThunkRegion;
  void* raw = mmap(nullptr, span, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
  if (raw == MAP_FAILED) return nullptr;
  const uintptr_t base = (reinterpret_cast<uintptr_t>(raw) + kThunkRegion - 1) & ~static_cast<uintptr_t>(kThunkRegion - 1);
  auto* code = reinterpret_cast<unsigned char*>(base);
  // give back what lies before and behind the pair
  if (base > reinterpret_cast<uintptr_t>(raw)) munmap(raw, base - reinterpret_cast<uintptr_t>(raw));
  const uintptr_t end = reinterpret_cast<uintptr_t>(raw) + span;
  if (end > base + 2 * kThunkRegion) munmap(reinterpret_cast<void*>(base + 2 * kThunkRegion), end - (base + 2 * kThunkRegion));
  for (size_t i = 0; i < kThunksPerRegion; ++i) {
    unsigned char* t   = code + i * kThunkBytes;
    const uintptr_t slot = base + kThunkRegion + i * sizeof(ThunkSlot);
    const int32_t d0 = static_cast<int32_t>(slot - (reinterpret_cast<uintptr_t>(t) + 7));
    const int32_t d1 = static_cast<int32_t>(slot + 8 - (reinterpret_cast<uintptr_t>(t) + 14));
    unsigned char bytes[16] = {0x48, 0x8B, 0x0D, 0, 0, 0, 0, 0x48, 0x8B, 0x05, 0, 0, 0, 0, 0xFF, 0xE0};
    std::memcpy(bytes + 3, &d0, 4);
    std::memcpy(bytes + 10, &d1, 4);
    std::memcpy(t, bytes, sizeof(bytes));
    std::memset(t + sizeof(bytes), 0xCC, kThunkBytes - sizeof(bytes));  // int3 padding
  }
  if (mprotect(code, kThunkRegion, PROT_READ | PROT_EXEC) != 0) {
    munmap(code, 2 * kThunkRegion);
    return nullptr;
  }
  __builtin___clear_cache(reinterpret_cast<char*>(code), reinterpret_cast<char*>(code) + kThunkRegion);
  return code;
}

// caller holds the pool's mutex; null when the system does not hand out executable memory
lower_func_ptr_g NewThunk(HostStubPool::Closure closure) {
  auto& t = Thunks();
  unsigned char* code = nullptr;
  if (!t.free_list.empty()) {
    code = t.free_list.back();
    t.free_list.pop_back();
  } else {
    if (t.used_in_last >= kThunksPerRegion) {
      unsigned char* region = NewThunkRegion();
      if (!region) return nullptr;
      t.regions.push_back(region);
      t.used_in_last = 0;
    }
    code = t.regions.back() + t.used_in_last * kThunkBytes;
    ++t.used_in_last;
  }
  auto* owned     = new HostStubPool::Closure(std::move(closure));
  ThunkSlot* slot = SlotOf(code);
  slot->closure   = owned;
  slot->dispatch  = &ThunkDispatch;
  auto fn    = reinterpret_cast<lower_func_ptr_g>(code);
  t.live[fn] = owned;
  return fn;
}

bool ReleaseThunk(lower_func_ptr_g fn) {
  auto& t = Thunks();
  auto it = t.live.find(fn);
  if (it == t.live.end()) return false;
  delete it->second;
  t.live.erase(it);
  t.free_list.push_back(reinterpret_cast<unsigned char*>(fn));
  return true;
}
#else
lower_func_ptr_g NewThunk(HostStubPool::Closure) { return nullptr; }
bool ReleaseThunk(lower_func_ptr_g) { return false; }
#endif
}  // namespace

HostStubPool& HostStubPool::Global() {
  static HostStubPool pool;
  return pool;
}

lower_func_ptr_g HostStubPool::Acquire(Closure closure) {
  auto& s = State();
  std::lock_guard<std::mutex> lock(s.mu);
  if (s.in_use >= kSlots) {
    lower_func_ptr_g fn = NewThunk(std::move(closure));
    CINN_CHECK(fn) << "all " << kSlots << " pre-compiled host stub slots are in use and no executable memory could be "
                   << "mapped for more; release compiled programs";
    return fn;
  }
  for (int probe = 0; probe < kSlots; ++probe) {
    int slot = (s.next_hint + probe) % kSlots;
    if (!s.used[slot]) {
      s.used[slot]     = true;
      s.closures[slot] = std::move(closure);
      s.next_hint      = slot + 1;
      ++s.in_use;
      return Table()[slot];
    }
  }
  CINN_CHECK(false) << "host stub pool is inconsistent";
  return nullptr;
}

void HostStubPool::Release(lower_func_ptr_g fn) {
  auto& s = State();
  std::lock_guard<std::mutex> lock(s.mu);
  const auto& table = Table();
  for (int slot = 0; slot < kSlots; ++slot) {
    if (table[slot] == fn) {
      if (s.used[slot]) {
        s.used[slot]     = false;
        s.closures[slot] = nullptr;
        --s.in_use;
      }
      return;
    }
  }
  ReleaseThunk(fn);
}

int HostStubPool::in_use() const {
  auto& s = State();
  std::lock_guard<std::mutex> lock(s.mu);
  return s.in_use;
}

int HostStubPool::thunks_in_use() const {
  auto& s = State();
  std::lock_guard<std::mutex> lock(s.mu);
#if defined(__x86_64__)
  return static_cast<int>(Thunks().live.size());
#else
  return 0;
#endif
}

// ---------------------------------------------------------------------------------------------------
// host function -> closure
// ---------------------------------------------------------------------------------------------------
HostStubPool::Closure LowerHostFunction(const ir::LoweredFunc& func, const std::map<std::string, void*>& kernel_symbols) {
  CINN_CHECK(!func.is_device) << func.name << " is a device function";
  auto* call = func.body.As<ir::Call>();
  CINN_CHECK(call) << "the body of host function " << func.name << " must be one intrinsic call";
  size_t expected = 0;
  ApiInvoker invoker = ExternApiRegistry::Global().Find(call->name, &expected);
  CINN_CHECK(invoker) << "host function " << func.name << " calls unknown runtime intrinsic " << call->name;
  CINN_CHECK_EQ(call->args.size(), expected) << "wrong number of arguments in the call of " << call->name;

  std::vector<BakedArg> baked;
  for (auto& a : call->args) {
    BakedArg b;
    if (auto* v = a.As<ir::Var>()) {
      if (v->name == "kernel_args") {
        b.kind = BakedArg::Kind::kArgs;
      } else if (v->name == "kernel_args_num") {
        b.kind = BakedArg::Kind::kNumArgs;
      } else if (v->name == "kernel_stream") {
        b.kind = BakedArg::Kind::kStream;
      } else {
        auto it = kernel_symbols.find(v->name);
        CINN_CHECK(it != kernel_symbols.end()) << "unresolved symbol " << v->name << " in host function " << func.name;
        b.kind = BakedArg::Kind::kHandle;
        b.p    = it->second;
      }
    } else if (auto* i = a.As<ir::IntImm>()) {
      b.kind = BakedArg::Kind::kInt;
      b.i    = i->value;
    } else if (auto* u = a.As<ir::UIntImm>()) {
      b.kind = u->type.is_bool() ? BakedArg::Kind::kBool : BakedArg::Kind::kInt;
      b.i    = static_cast<int64_t>(u->value);
    } else if (auto* f = a.As<ir::FloatImm>()) {
      b.kind = BakedArg::Kind::kFloat;
      b.f    = f->value;
    } else {
      CINN_CHECK(false) << "argument of " << call->name << " in " << func.name << " is not a constant: " << ir::ToString(a);
    }
    baked.push_back(b);
  }
  return [invoker, baked](void* args, int32_t num_args, void* stream) { invoker(baked, args, num_args, stream); };
}

}  // namespace backends
}  // namespace cinn
