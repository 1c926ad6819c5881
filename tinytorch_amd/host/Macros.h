// Assertion / logging conventions of the host layer.
//
// They follow TinyTorch's (reference src/Utils/Macros.h:19-43, src/Utils/Logger.h:29-41): the library is built
// without exceptions; a failed precondition logs "Assertion failed: (...)" through LOGE and then stops the program.
// The stop action is replaceable (setAssertHandler) so that tests can observe a failure instead of dying.
#pragma once

#include <cstdarg>
#include <cstdio>

namespace tinytorch {

using LogFunc = void (*)(int level, const char* msg);  // level: 0 info, 1 debug, 2 warning, 3 error
void setLogFunc(LogFunc fn);
void logMessage(int level, const char* file, int line, const char* fmt, ...) __attribute__((format(printf, 4, 5)));

using AssertHandler = void (*)(const char* expr, const char* file, int line);
// nullptr restores the default (trap).  Returns the previous handler.
AssertHandler setAssertHandler(AssertHandler h);
void assertFailed(const char* expr, const char* file, int line);

}  // namespace tinytorch

#define LOGI(...) ::tinytorch::logMessage(0, __FILE__, __LINE__, __VA_ARGS__)
#define LOGD(...) ::tinytorch::logMessage(1, __FILE__, __LINE__, __VA_ARGS__)
#define LOGW(...) ::tinytorch::logMessage(2, __FILE__, __LINE__, __VA_ARGS__)
#define LOGE(...) ::tinytorch::logMessage(3, __FILE__, __LINE__, __VA_ARGS__)

#define ASSERT(expr)                                                   \
  do {                                                                 \
    if (!(expr)) {                                                     \
      LOGE("Assertion failed: (%s)", #expr);                           \
      ::tinytorch::assertFailed(#expr, __FILE__, __LINE__);            \
    }                                                                  \
  } while (0)

#define NOT_IMPLEMENTED() ASSERT(!"Not implemented")

// Runs `func` once during static initialisation of every translation unit that sees the macro; registration
// functions are idempotent (reference src/Utils/Macros.h:53-57).
namespace tinytorch {
struct StaticCaller {
  explicit StaticCaller(void (*func)()) { func(); }
};
}  // namespace tinytorch
#define STATIC_CALL(func) static ::tinytorch::StaticCaller _static_caller_##func(func);

// HIP runtime failure: print and abort, as the reference does for its device runtime (src/Utils/CUDAUtils.h:36-44).
#define HIP_CHECK(call)                                                                              \
  do {                                                                                               \
    hipError_t _e = (call);                                                                          \
    if (_e != hipSuccess) {                                                                          \
      std::fprintf(stderr, "HIP error %d (%s) at %s:%d\n", (int)_e, hipGetErrorString(_e), __FILE__, \
                   __LINE__);                                                                        \
      std::abort();                                                                                  \
    }                                                                                                \
  } while (0)
