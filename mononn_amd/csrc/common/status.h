// Error type used inside the host compiler.  The reference aborts the process on every failure
// (LOG(FATAL), e.g. mononn_engine/module/mononn_module.cc:84,163); here failures are exceptions
// that the C-ABI layer turns into return codes plus a thread-local message.
#pragma once
#include <sstream>
#include <stdexcept>
#include <string>

namespace mononn {

enum Code : int {
  kOk = 0,
  kInvalidArgument = 1,
  kParseError = 2,
  kUnsupported = 3,
  kSpecError = 4,
  kCompileError = 5,
  kRuntimeError = 6,
  kResourceExhausted = 7,
  kNotFound = 8,
  kInternal = 9,
};

class Error : public std::runtime_error {
 public:
  Error(Code code, const std::string& msg) : std::runtime_error(msg), code_(code) {}
  Code code() const { return code_; }

 private:
  Code code_;
};

class ErrorStream {
 public:
  explicit ErrorStream(Code c) : code_(c) {}
  template <class T>
  ErrorStream& operator<<(const T& v) {
    os_ << v;
    return *this;
  }
  [[noreturn]] void raise() const { throw Error(code_, os_.str()); }

 private:
  Code code_;
  std::ostringstream os_;
};

struct Raiser {
  [[noreturn]] void operator&(const ErrorStream& s) const { s.raise(); }
};

}  // namespace mononn

#define MONONN_FAIL(code) ::mononn::Raiser() & ::mononn::ErrorStream(::mononn::code)
#define MONONN_CHECK(cond, code) \
  if (cond) {                    \
  } else                         \
    MONONN_FAIL(code) << "[" #cond "] "
