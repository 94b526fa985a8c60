// Error reporting of the front end: a failed C-ABI call becomes thrust::system_error, a
// failed allocation thrust::system::detail::bad_alloc (a std::bad_alloc), as in the
// reference (thrust/system/cuda/detail/util.h:181-241, malloc_and_free.h:65-69).
#pragma once
#include <new>
#include <stdexcept>
#include <string>

#include <thrust/detail/config.h>
#include <thrust_amd.h>

namespace thrust {
namespace system {

class system_error : public std::runtime_error {
 public:
  system_error(int status, const std::string& what)
      : std::runtime_error(what + ": " + thrust_amd_error_string(status)), status_(status) {}
  int code() const { return status_; }

 private:
  int status_;
};

namespace detail {
class bad_alloc : public std::bad_alloc {
 public:
  explicit bad_alloc(const std::string& w) : what_(std::string("std::bad_alloc: ") + w) {}
  const char* what() const noexcept override { return what_.c_str(); }

 private:
  std::string what_;
};
}  // namespace detail

namespace hip {
namespace detail {
inline void throw_on_error(int status, const char* what) {
  if (status != 0) throw thrust::system::system_error(status, what);
}
}  // namespace detail
}  // namespace hip

}  // namespace system
using system::system_error;
}  // namespace thrust
