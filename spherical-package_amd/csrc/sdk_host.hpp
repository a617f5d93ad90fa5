// Host-side helpers shared by the C-ABI translation units: error reporting,
// argument checks and launch checks.  gfx950 only; no other backend.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "sdk_mapped_ops.h"

namespace sdk {

// Thread-local message returned by sdk_last_error(); defined in api_common.hip.
void set_error(const char* fmt, ...);

inline int fail(sdk_status st, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  set_error("%s", buf);
  return st;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Number of interpolation points a sample consumes in the map: 1 for the
// unweighted layout (P == 0), P otherwise.
inline int pts(int P) { return P == 0 ? 1 : P; }

// Kernel launch as an expression (usable inside the dispatch macros below).
template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t stream,
                   Args... args) {
  kernel<<<grid, block, 0, stream>>>(args...);
}

}  // namespace sdk

#define SDK_REQUIRE(cond, ...)                                         \
  do {                                                                 \
    if (!(cond)) return sdk::fail(SDK_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

#define SDK_LAUNCH_CHECK(what)                                                         \
  do {                                                                                 \
    hipError_t e__ = hipGetLastError();                                                \
    if (e__ != hipSuccess)                                                             \
      return sdk::fail(SDK_ERR_DEVICE, "%s: %s", what, hipGetErrorString(e__));        \
  } while (0)

// Runs `CALL` with `T` bound to the C type of `dtype`.
#define SDK_DISPATCH_DTYPE(dtype, CALL)                                 \
  do {                                                                  \
    if ((dtype) == SDK_F32) { using T = float; CALL; }                  \
    else if ((dtype) == SDK_F64) { using T = double; CALL; }            \
    else return sdk::fail(SDK_ERR_INVALID_ARGUMENT, "unknown dtype %d", (int)(dtype)); \
  } while (0)

// Runs `CALL` with compile-time `INTERP` (0,1,2; anything else is nearest, as
// the reference's switch default) and `WEIGHTED`.
#define SDK_DISPATCH_INTERP(interp, P, CALL)                                             \
  do {                                                                                   \
    const int i__ = ((interp) == 1 || (interp) == 2) ? (interp) : 0;                     \
    if ((P) == 0) {                                                                      \
      constexpr bool WEIGHTED = false;                                                   \
      if (i__ == 0) { constexpr int INTERP = 0; CALL; }                                  \
      else if (i__ == 1) { constexpr int INTERP = 1; CALL; }                             \
      else { constexpr int INTERP = 2; CALL; }                                           \
    } else {                                                                             \
      constexpr bool WEIGHTED = true;                                                    \
      if (i__ == 0) { constexpr int INTERP = 0; CALL; }                                  \
      else if (i__ == 1) { constexpr int INTERP = 1; CALL; }                             \
      else { constexpr int INTERP = 2; CALL; }                                           \
    }                                                                                    \
  } while (0)
