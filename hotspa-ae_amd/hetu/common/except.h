// Error convention of the host layer: stream-style macros that THROW subclasses
// of hetu::hetu_exception (same names as hetu/common/except.h:10-90 of the
// reference).  No error codes are returned from the hetu:: API.
#pragma once

#include <exception>
#include <sstream>
#include <string>

namespace hetu {

class hetu_exception : public std::exception {
 public:
  explicit hetu_exception(const std::string& msg, const char* file, int line) {
    std::ostringstream ss;
    ss << " (" << file << ":" << line << ") " << msg;
    _msg = ss.str();
  }
  explicit hetu_exception(const std::string& msg) : _msg(msg) {}
  const char* what() const noexcept override { return _msg.c_str(); }

 protected:
  std::string _msg;
};

#define HT_DECLARE_EXCEPTION(Name)                                              \
  class Name : public hetu_exception {                                          \
   public:                                                                      \
    using hetu_exception::hetu_exception;                                       \
  }

HT_DECLARE_EXCEPTION(assertion_error);
HT_DECLARE_EXCEPTION(bad_alloc);
HT_DECLARE_EXCEPTION(not_implemented);
HT_DECLARE_EXCEPTION(value_error);
HT_DECLARE_EXCEPTION(timeout_error);
HT_DECLARE_EXCEPTION(type_error);
HT_DECLARE_EXCEPTION(runtime_error);

namespace detail {
// Collects a message with operator<< and throws E when the full expression ends.
template <typename E>
class Thrower {
 public:
  Thrower(const char* file, int line, const char* prefix) : _file(file), _line(line) { _ss << prefix; }
  Thrower(const Thrower&) = delete;
  [[noreturn]] ~Thrower() noexcept(false) { throw E(_ss.str(), _file, _line); }
  template <typename V>
  Thrower& operator<<(const V& v) {
    _ss << v;
    return *this;
  }

 private:
  std::ostringstream _ss;
  const char* _file;
  int _line;
};
} // namespace detail

} // namespace hetu

#define __HT_THROW(Exc, prefix) ::hetu::detail::Thrower<Exc>(__FILE__, __LINE__, prefix)

#define HT_ASSERT(cond)                                                         \
  if (!(cond)) __HT_THROW(::hetu::assertion_error, "Assertion " #cond " failed: ")
#define HT_ASSERT_LT(x, y) HT_ASSERT((x) < (y))
#define HT_ASSERT_GT(x, y) HT_ASSERT((x) > (y))
#define HT_ASSERT_LE(x, y) HT_ASSERT((x) <= (y))
#define HT_ASSERT_GE(x, y) HT_ASSERT((x) >= (y))
#define HT_ASSERT_EQ(x, y) HT_ASSERT((x) == (y))
#define HT_ASSERT_NE(x, y) HT_ASSERT((x) != (y))
#define HT_BAD_ALLOC __HT_THROW(::hetu::bad_alloc, "Bad alloc: ")
#define HT_BAD_ALLOC_IF(cond) if (cond) HT_BAD_ALLOC
#define HT_NOT_IMPLEMENTED __HT_THROW(::hetu::not_implemented, "Not implemented: ")
#define HT_NOT_IMPLEMENTED_IF(cond) if (cond) HT_NOT_IMPLEMENTED
#define HT_VALUE_ERROR __HT_THROW(::hetu::value_error, "Value error: ")
#define HT_VALUE_ERROR_IF(cond) if (cond) HT_VALUE_ERROR
#define HT_TYPE_ERROR __HT_THROW(::hetu::type_error, "Type error: ")
#define HT_TYPE_ERROR_IF(cond) if (cond) HT_TYPE_ERROR
#define HT_RUNTIME_ERROR __HT_THROW(::hetu::runtime_error, "Runtime error: ")
#define HT_RUNTIME_ERROR_IF(cond) if (cond) HT_RUNTIME_ERROR
