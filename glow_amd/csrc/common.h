// Shared host-side helpers of the MI355X kernel library: error reporting and
// launch plumbing. Device code lives in requant.h / the *.hip files.
#ifndef GLOW_MI355X_COMMON_H
#define GLOW_MI355X_COMMON_H

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/glow_mi355x.h"

namespace mi355x {

// Records the message returned by mi355x_last_error() on this thread and
// returns `code`, so call sites read `return fail(MI355X_ERR_..., "...")`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Checks the launch that was just issued.
int check_launch(const char *what);

constexpr int kWave = 64;

inline bool shift_ok(int32_t s) { return s >= 0 && s <= 31; }

// SparseLengths scratch (slws.hip). A stream the library knows has a buffer for
// the bag-offset pre-pass of launches with more than 4096 bags; reserving
// allocates (once per device and stream), launches never do.
int slws_reserve_stream(hipStream_t st);
int slws_release_stream(hipStream_t st);
// Looks up, once per device, the address of the fixed scratch array used by
// mi355x_frwq_slws_noalloc on the current device.
int slws_init_device();

} // namespace mi355x

#define MI355X_HIP(expr)                                                       \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess) {                                                    \
      return ::mi355x::fail(e_ == hipErrorOutOfMemory                          \
                                ? MI355X_ERR_OUT_OF_DEVICE_MEMORY              \
                                : MI355X_ERR_RUNTIME,                          \
                            "%s failed: %s", #expr, hipGetErrorString(e_));    \
    }                                                                          \
  } while (0)

#define MI355X_REQUIRE(cond, ...)                                              \
  do {                                                                         \
    if (!(cond))                                                               \
      return ::mi355x::fail(MI355X_ERR_INVALID_ARGUMENT, __VA_ARGS__);         \
  } while (0)

#endif
