// Shared plumbing of libtvmkv: error propagation across the C ABI and HIP call checking.
#ifndef TVMKV_CSRC_COMMON_H_
#define TVMKV_CSRC_COMMON_H_

#include <hip/hip_runtime_api.h>

#include <sstream>
#include <stdexcept>
#include <string>

#include "../../include/tvmkv.h"

namespace tvmkv {

// Exception used inside the library; converted to (code, thread-local message) at the ABI.
class Error : public std::runtime_error {
 public:
  Error(int code, const std::string& msg) : std::runtime_error(msg), code(code) {}
  int code;
};

void SetLastError(const std::string& msg);

// Stream-style message builder: KV_CHECK(x) << "text" << value;
class Thrower {
 public:
  Thrower(int code, const char* prefix) : code_(code) { os_ << prefix; }
  template <typename T>
  Thrower& operator<<(const T& v) {
    os_ << v;
    return *this;
  }
  [[noreturn]] void Throw() const { throw Error(code_, os_.str()); }

 private:
  int code_;
  std::ostringstream os_;
};

struct ThrowTrigger {
  [[noreturn]] void operator&(const Thrower& t) const { t.Throw(); }
};

}  // namespace tvmkv

// Mirrors the reference's TVM_FFI_ICHECK(cond) << msg: the message is what the caller sees.
#define KV_CHECK(cond) \
  if (cond) {          \
  } else               \
    ::tvmkv::ThrowTrigger() & ::tvmkv::Thrower(TVMKV_EINVAL, "")
#define KV_UNSUPPORTED(cond) \
  if (!(cond)) {             \
  } else                     \
    ::tvmkv::ThrowTrigger() & ::tvmkv::Thrower(TVMKV_EUNSUPPORTED, "")

#define HIP_CHECK(expr)                                                                          \
  do {                                                                                           \
    hipError_t _e = (expr);                                                                      \
    if (_e != hipSuccess) {                                                                      \
      throw ::tvmkv::Error(TVMKV_EDEVICE, std::string(#expr) + ": " + hipGetErrorString(_e));    \
    }                                                                                            \
  } while (0)

// Body wrapper of every extern "C" entry point.
#define KV_API_BEGIN() try {
#define KV_API_END()                               \
  }                                                \
  catch (const ::tvmkv::Error& e) {                \
    ::tvmkv::SetLastError(e.what());               \
    return e.code;                                 \
  }                                                \
  catch (const std::exception& e) {                \
    ::tvmkv::SetLastError(e.what());               \
    return TVMKV_EINVAL;                           \
  }                                                \
  return TVMKV_OK;

#endif  // TVMKV_CSRC_COMMON_H_
