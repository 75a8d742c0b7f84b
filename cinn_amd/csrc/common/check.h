// Error handling for the host-side compiler code: failed checks throw cinn::Error, which the C API
// boundary turns into a status code plus message.  (The runtime intrinsics keep the reference's
// abort-on-error convention instead; see runtime/hip_check.h.)
#pragma once
#include <sstream>
#include <stdexcept>
#include <string>

namespace cinn {

class Error : public std::runtime_error {
 public:
  explicit Error(const std::string& msg) : std::runtime_error(msg) {}
};

namespace detail {
class CheckFailStream {
 public:
  CheckFailStream(const char* file, int line, const char* cond) { ss_ << file << ":" << line << " check failed: " << cond << " "; }
  template <typename T>
  CheckFailStream& operator<<(const T& v) {
    ss_ << v;
    return *this;
  }
  [[noreturn]] ~CheckFailStream() noexcept(false) { throw Error(ss_.str()); }

 private:
  std::ostringstream ss_;
};
}  // namespace detail
}  // namespace cinn

#define CINN_CHECK(cond) \
  if (!(cond)) ::cinn::detail::CheckFailStream(__FILE__, __LINE__, #cond)
#define CINN_CHECK_EQ(a, b) CINN_CHECK((a) == (b)) << "(" << (a) << " vs " << (b) << ") "
#define CINN_CHECK_NE(a, b) CINN_CHECK((a) != (b)) << "(" << (a) << " vs " << (b) << ") "
#define CINN_CHECK_LT(a, b) CINN_CHECK((a) < (b)) << "(" << (a) << " vs " << (b) << ") "
#define CINN_CHECK_LE(a, b) CINN_CHECK((a) <= (b)) << "(" << (a) << " vs " << (b) << ") "
#define CINN_CHECK_GT(a, b) CINN_CHECK((a) > (b)) << "(" << (a) << " vs " << (b) << ") "
#define CINN_CHECK_GE(a, b) CINN_CHECK((a) >= (b)) << "(" << (a) << " vs " << (b) << ") "
#define CINN_NOT_IMPLEMENTED(what) ::cinn::detail::CheckFailStream(__FILE__, __LINE__, "not implemented") << what
