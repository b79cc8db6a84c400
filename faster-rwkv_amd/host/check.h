// Error reporting of the host layer.  Same surface as the reference's check.h
// (FRException, RV_CHECK, RV_UNIMPLEMENTED: /root/reference check.h:11-48) so that
// operator code written against it compiles unchanged; FRHIP_CHECK turns a non-zero
// C-ABI status into an FRException carrying frhip_error_string().
#pragma once

#include <sstream>
#include <stdexcept>
#include <string>

struct FRException : public std::runtime_error {
  FRException() : std::runtime_error("") {}
  explicit FRException(std::string m) : std::runtime_error(""), msg(std::move(m)) {}
  const char *what() const noexcept override { return msg.c_str(); }
  template <typename T> FRException &operator<<(const T &v) {
    std::ostringstream os;
    os << v;
    msg += os.str();
    return *this;
  }
  std::string msg;
};

namespace rwkv::detail {
inline std::string where(const char *what, const char *file, int line) {
  return std::string(what) + " at " + file + ":" + std::to_string(line) + "\n  > Error msg: ";
}
}  // namespace rwkv::detail

// Usage: RV_CHECK(cond) << "context";   -- throws only when cond is false.
#define RV_CHECK(...)                          \
  while (!static_cast<bool>(__VA_ARGS__))      \
  throw FRException(::rwkv::detail::where("Check \"" #__VA_ARGS__ "\" failed", __FILE__, __LINE__))

#define RV_UNIMPLEMENTED() throw FRException(::rwkv::detail::where("Unimplemented", __FILE__, __LINE__))

#define FRHIP_CHECK(call)                                                                      \
  do {                                                                                         \
    int _st = (call);                                                                          \
    if (_st != 0)                                                                              \
      throw FRException(::rwkv::detail::where(#call " failed", __FILE__, __LINE__))            \
          << "status " << _st << ": " << frhip_error_string();                                 \
  } while (0)

#define FR_DISALLOW_COPY_AND_MOVE(Class)     \
  Class(const Class &) = delete;             \
  Class &operator=(const Class &) = delete;  \
  Class(Class &&) = delete;                  \
  Class &operator=(Class &&) = delete
