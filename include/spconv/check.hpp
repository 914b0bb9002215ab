// Log-only assertions and HIP call checking, same macro names as the reference's
// libraries/3DSparseConvolution/libspconv/include/spconv/check.hpp:23-57 with the runtime switched to HIP:
// nothing here aborts; failures are sent to the logger and reported through the return value.
#ifndef SCN_SPCONV_CHECK_HPP
#define SCN_SPCONV_CHECK_HPP

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <string>

#include "engine.hpp"

namespace spconv {

inline std::string format(const char* fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  return buf;
}

inline bool check_hip_api_(hipError_t e, const char* call, int line, const char* file) {
  if (e == hipSuccess) return true;
  logger_output(file, line, LoggerLevel::Error, "HIP runtime error %s # %s, code = %s [ %d ]", call, hipGetErrorString(e),
                hipGetErrorName(e), (int)e);
  return false;
}

#define check_hip_api(call) spconv::check_hip_api_(call, #call, __LINE__, __FILE__)
#define check_hip_kernel(...)                                                       \
  do {                                                                              \
    __VA_ARGS__;                                                                    \
    spconv::check_hip_api_(hipPeekAtLastError(), #__VA_ARGS__, __LINE__, __FILE__); \
  } while (0)

#define spconv_assertf(cond, fmt, ...)                                                                        \
  do {                                                                                                        \
    if (!(cond))                                                                                              \
      spconv::logger_output(__FILE__, __LINE__, spconv::LoggerLevel::Error,                                   \
                            "Assert failed. %s in file %s:%d, message: " fmt, #cond, __FILE__, __LINE__, __VA_ARGS__); \
  } while (false)
#define spconv_asserts(cond, s)                                                                               \
  do {                                                                                                        \
    if (!(cond))                                                                                              \
      spconv::logger_output(__FILE__, __LINE__, spconv::LoggerLevel::Error,                                   \
                            "Assert failed. %s in file %s:%d, message: " s, #cond, __FILE__, __LINE__);      \
  } while (false)
#define spconv_assert(cond)                                                                                   \
  do {                                                                                                        \
    if (!(cond))                                                                                              \
      spconv::logger_output(__FILE__, __LINE__, spconv::LoggerLevel::Error, "Assert failed. %s in file %s:%d", #cond, \
                            __FILE__, __LINE__);                                                              \
  } while (false)
#define spconv_logf(level, fmt, ...) spconv::logger_output(__FILE__, __LINE__, level, fmt, __VA_ARGS__);
#define spconv_log(level, msg) spconv::logger_output(__FILE__, __LINE__, level, "%s", msg);

}  // namespace spconv

#endif  // SCN_SPCONV_CHECK_HPP
