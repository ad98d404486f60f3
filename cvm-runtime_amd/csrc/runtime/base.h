// Error reporting and small shared types of the host-side graph runtime.
//
// Two exception classes carry the reference's status-code contract
// (include/cvm/errors.h:15-36, include/utils/logging.h:301-338):
//   VERIFY(...) failures -> std::logic_error   -> ERROR_LOGIC (1)
//   CHECK(...)/FATAL     -> std::runtime_error -> ERROR_RUNTIME (2)
#ifndef CVM_RT_BASE_H_
#define CVM_RT_BASE_H_

#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace cvmrt {

typedef std::vector<int64_t> Shape;

inline int64_t shape_size(const Shape& s) {
  int64_t n = 1;
  for (int64_t v : s) n *= v;
  return n;
}

inline std::string shape_str(const Shape& s) {
  std::ostringstream os;
  os << "(";
  for (size_t i = 0; i < s.size(); ++i) os << (i ? ", " : "") << s[i];
  os << ")";
  return os.str();
}

// Collects a message with operator<< and throws E when it goes out of scope.
template <typename E>
class Thrower {
 public:
  Thrower(const char* file, int line, const char* cond) {
    os_ << file << ":" << line << ": ";
    if (cond) os_ << "Check failed: " << cond << " ";
  }
  [[noreturn]] ~Thrower() noexcept(false) { throw E(os_.str()); }
  template <typename T>
  Thrower& operator<<(const T& v) {
    os_ << v;
    return *this;
  }

 private:
  std::ostringstream os_;
};

struct Voidify {
  template <typename E>
  void operator&(const Thrower<E>&) {}
};

}  // namespace cvmrt

#define CVM_VERIFY(cond) \
  (cond) ? (void)0 : ::cvmrt::Voidify() & ::cvmrt::Thrower<std::logic_error>(__FILE__, __LINE__, #cond)
#define CVM_CHECK(cond) \
  (cond) ? (void)0 : ::cvmrt::Voidify() & ::cvmrt::Thrower<std::runtime_error>(__FILE__, __LINE__, #cond)
#define CVM_FATAL() ::cvmrt::Voidify() & ::cvmrt::Thrower<std::runtime_error>(__FILE__, __LINE__, nullptr)

#endif
