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

// Options of the launch being issued on this thread. The entry points with an
// options argument set them for the duration of the call (OptsScope); the ones
// without leave the thread's defaults in place (the legacy setters
// mi355x_gemm_tile_override, mi355x_gemm_requant_hint; the process-wide
// mi355x_slws_set_fused_math). Nothing outlives a call that names its options.
extern thread_local int g_tile_override;   // -1: chosen from the shape
extern thread_local int g_requant_hint;    // MI355X_REQUANT_* flags
extern thread_local int g_slws_math;       // -1: the process default
extern thread_local void *g_workspace;     // device memory a matrix-core launch may use
extern thread_local size_t g_workspace_bytes;

struct OptsScope {
  int rc = MI355X_OK;
  int tile, hint, math;
  void *ws;
  size_t ws_bytes;
  // the struct may end behind slws_math (callers built before the workspace
  // fields existed) or hold all of it
  static constexpr size_t kSizeWithoutWorkspace = offsetof(mi355x_launch_opts, workspace);
  explicit OptsScope(const mi355x_launch_opts *o)
      : tile(g_tile_override), hint(g_requant_hint), math(g_slws_math), ws(g_workspace),
        ws_bytes(g_workspace_bytes) {
    if (!o) return;
    if (o->struct_size != sizeof(mi355x_launch_opts) && o->struct_size != kSizeWithoutWorkspace) {
      rc = fail(MI355X_ERR_INVALID_ARGUMENT, "mi355x_launch_opts: struct_size %u, expected %zu",
                o->struct_size, sizeof(mi355x_launch_opts));
    } else if (o->gemm_tile < -1 || o->gemm_tile > 12) {
      rc = fail(MI355X_ERR_INVALID_ARGUMENT, "gemm_tile %d outside [-1, 12]", o->gemm_tile);
    } else if (o->requant_hint < 0 || o->requant_hint > 3 || o->requant_hint == 2) {
      rc = fail(MI355X_ERR_INVALID_ARGUMENT,
                "requant_hint %d: bit 1 (no pre-shifts) needs bit 0 (24-bit operands)",
                o->requant_hint);
    } else if (o->slws_math < -1 || o->slws_math > MI355X_SLWS_MATH_REGROUPED) {
      rc = fail(MI355X_ERR_INVALID_ARGUMENT, "slws_math %d outside [-1, 2]", o->slws_math);
    } else {
      g_tile_override = o->gemm_tile;
      g_requant_hint = o->requant_hint;
      g_slws_math = o->slws_math;
      const bool has_ws = o->struct_size == sizeof(mi355x_launch_opts);
      g_workspace = has_ws ? o->workspace : nullptr;
      g_workspace_bytes = has_ws && o->workspace ? (size_t)o->workspace_bytes : 0;
    }
  }
  ~OptsScope() {
    g_tile_override = tile;
    g_requant_hint = hint;
    g_slws_math = math;
    g_workspace = ws;
    g_workspace_bytes = ws_bytes;
  }
  OptsScope(const OptsScope &) = delete;
  OptsScope &operator=(const OptsScope &) = delete;
};

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
