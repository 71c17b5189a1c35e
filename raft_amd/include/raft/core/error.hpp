// Exceptions and precondition macros of the reduction path.
// Follows the reference's contract (core/error.hpp:86-188,328-347): a base
// raft::exception, raft::logic_error thrown by RAFT_EXPECTS / RAFT_FAIL with the
// message "RAFT failure at file=<f> line=<n>: <reason>", and a device-runtime
// error type for launch failures (here HIP instead of CUDA).
#pragma once

#include <cstdarg>
#include <cstdio>
#include <exception>
#include <string>
#include <vector>

namespace raft {

class exception : public std::exception {
 public:
  exception() noexcept = default;
  explicit exception(std::string msg) noexcept : msg_(std::move(msg)) {}
  char const* what() const noexcept override { return msg_.c_str(); }

 private:
  std::string msg_;
};

struct logic_error : public raft::exception {
  explicit logic_error(char const* m) : raft::exception(m) {}
  explicit logic_error(std::string const& m) : raft::exception(m) {}
};

// Raised when the device runtime or the reduction library reports a failure
// (the reference's raft::cuda_error, util/cuda_rt_essentials.hpp:25-67).
struct hip_error : public raft::exception {
  explicit hip_error(char const* m) : raft::exception(m) {}
  explicit hip_error(std::string const& m) : raft::exception(m) {}
};
using cuda_error = hip_error;

namespace detail {
inline std::string format_failure(char const* prefix, char const* file, int line, char const* fmt, ...)
{
  std::va_list a1, a2;
  va_start(a1, fmt);
  va_copy(a2, a1);
  const int n_reason = std::vsnprintf(nullptr, 0, fmt, a1);
  va_end(a1);
  std::string reason(n_reason > 0 ? (size_t)n_reason : 0, '\0');
  if (n_reason > 0) std::vsnprintf(reason.data(), reason.size() + 1, fmt, a2);
  va_end(a2);
  return std::string(prefix) + "file=" + file + " line=" + std::to_string(line) + ": " + reason;
}
}  // namespace detail
}  // namespace raft

#define RAFT_EXPECTS(cond, fmt, ...)                                                       \
  do {                                                                                     \
    if (!(cond)) {                                                                         \
      throw raft::logic_error(raft::detail::format_failure(                                \
        "RAFT failure at ", __FILE__, __LINE__, fmt, ##__VA_ARGS__));                      \
    }                                                                                      \
  } while (0)

#define RAFT_FAIL(fmt, ...)                                                                \
  do {                                                                                     \
    throw raft::logic_error(raft::detail::format_failure(                                  \
      "RAFT failure at ", __FILE__, __LINE__, fmt, ##__VA_ARGS__));                        \
  } while (0)

#define THROW(fmt, ...)                                                                    \
  do {                                                                                     \
    throw raft::exception(raft::detail::format_failure(                                    \
      "exception occurred! ", __FILE__, __LINE__, fmt, ##__VA_ARGS__));                    \
  } while (0)

// core/error.hpp:297-300 in the reference: a failed check raises raft::exception
#define ASSERT(check, fmt, ...)              \
  do {                                       \
    if (!(check)) THROW(fmt, ##__VA_ARGS__); \
  } while (0)

#define RAFT_HIP_TRY(call)                                                                 \
  do {                                                                                     \
    hipError_t const raft_status_ = (call);                                                \
    if (raft_status_ != hipSuccess) {                                                      \
      (void)hipGetLastError();                                                             \
      throw raft::hip_error(raft::detail::format_failure(                                  \
        "HIP error encountered at: ", __FILE__, __LINE__, "call='%s', Reason=%s:%s", #call,\
        hipGetErrorName(raft_status_), hipGetErrorString(raft_status_)));                  \
    }                                                                                      \
  } while (0)
