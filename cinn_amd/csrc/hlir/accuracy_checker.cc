#include "hlir/accuracy_checker.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <mutex>
#include <sstream>
#include <vector>

namespace cinn {
namespace hlir {
namespace framework {

namespace {

float HalfBitsToFloat(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  uint32_t exp        = (h >> 10) & 0x1fu;
  uint32_t man        = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      // subnormal: normalise
      int shift = 0;
      while (!(man & 0x400u)) {
        man <<= 1;
        ++shift;
      }
      man &= 0x3ffu;
      bits = sign | ((113u - shift) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

float BFloatBitsToFloat(uint16_t b) {
  uint32_t bits = static_cast<uint32_t>(b) << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

// the tensor's elements as doubles (every supported type fits: int64 values beyond 2^53 lose their low bits in the
// printout only)
std::vector<double> ToDoubles(const std::vector<char>& raw, const common::Type& t, int64_t numel) {
  std::vector<double> v(static_cast<size_t>(numel));
  const char* p = raw.data();
  for (int64_t i = 0; i < numel; ++i) {
    if (t.is_float(32)) {
      float f;
      std::memcpy(&f, p + 4 * i, 4);
      v[i] = f;
    } else if (t.is_float(64)) {
      std::memcpy(&v[i], p + 8 * i, 8);
    } else if (t.is_float16() || t.is_bfloat16()) {
      uint16_t h;
      std::memcpy(&h, p + 2 * i, 2);
      v[i] = t.is_float16() ? HalfBitsToFloat(h) : BFloatBitsToFloat(h);
    } else if (t.is_int(32)) {
      int32_t x;
      std::memcpy(&x, p + 4 * i, 4);
      v[i] = x;
    } else if (t.is_int(64)) {
      int64_t x;
      std::memcpy(&x, p + 8 * i, 8);
      v[i] = static_cast<double>(x);
    } else if (t.bytes() == 1) {
      v[i] = t.is_bool() ? static_cast<double>(p[i] != 0) : static_cast<double>(static_cast<signed char>(p[i]));
    } else if (t.bytes() == 2) {
      int16_t x;
      std::memcpy(&x, p + 2 * i, 2);
      v[i] = x;
    } else {
      v[i] = 0.0;
    }
  }
  return v;
}

bool FlagIsTrue(const std::string& s) { return s == "1" || s == "true" || s == "True" || s == "TRUE"; }
bool FlagIsFalse(const std::string& s) { return s.empty() || s == "0" || s == "false" || s == "False" || s == "FALSE"; }

}  // namespace

std::string DescribeTensor(const Tensor& tensor, const std::string& name, int print_num) {
  const int64_t numel = tensor->numel();
  std::ostringstream ss;
  ss << "name=" << name << ", dtype=" << common::Type2Str(tensor->type()) << ", shape={";
  for (size_t i = 0; i < tensor->shape().size(); ++i) ss << (i ? ", " : "") << tensor->shape()[i];
  ss << "}, data=[";
  if (!tensor->data() || numel == 0) {
    ss << "], not allocated";
    return ss.str();
  }
  std::vector<char> raw(tensor->bytes());
  tensor->CopyToHost(raw.data(), raw.size());
  std::vector<double> v = ToDoubles(raw, tensor->type(), numel);
  bool has_nan = false, has_inf = false, all_zero = true, all_one = true;
  for (double x : v) {
    if (std::isnan(x)) has_nan = true;
    if (std::isinf(x)) has_inf = true;
    if (x != 0.0) all_zero = false;
    if (x != 1.0) all_one = false;
  }
  ss.precision(std::numeric_limits<float>::max_digits10);
  const int64_t n = print_num < 0 ? numel : print_num;
  if (numel <= 2 * n) {
    for (int64_t i = 0; i < numel; ++i) ss << (i ? ", " : "") << v[i];
  } else {
    for (int64_t i = 0; i < n; ++i) ss << (i ? ", " : "") << v[i];
    ss << ", ... , ";
    for (int64_t i = numel - n; i < numel; ++i) ss << v[i] << (i + 1 < numel ? ", " : "");
  }
  ss << "], " << (has_nan ? "NaN" : has_inf ? "Inf" : all_zero ? "Zero" : all_one ? "One" : "OK");
  return ss.str();
}

SelfCheckSink& SelfCheckSink::Get() {
  static SelfCheckSink sink;
  return sink;
}

SelfCheckSink::SelfCheckSink() {
  const char* flag = getenv("FLAGS_cinn_self_check_accuracy");
  std::string value = flag ? flag : "";
  if (FlagIsFalse(value)) return;
  enabled_ = true;
  if (const char* n = getenv("FLAGS_cinn_self_check_accuracy_num")) print_num_ = atoi(n);
  if (!FlagIsTrue(value)) {
    file_ = fopen(value.c_str(), "w");
    if (!file_) fprintf(stderr, "cinn: cannot open \"%s\", the self-check reports go to stderr\n", value.c_str());
  }
}

SelfCheckSink::~SelfCheckSink() {
  if (file_) fclose(static_cast<FILE*>(file_));
}

void SelfCheckSink::Write(const std::string& text) {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  FILE* out = file_ ? static_cast<FILE*>(file_) : stderr;
  fputs(text.c_str(), out);
  fputc('\n', out);
  fflush(out);
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
