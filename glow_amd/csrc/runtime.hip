// Device, memory, stream, event and static-memory-plan entry points of the
// MI355X kernel library. The arena mirrors how Glow lays a compiled function
// out: constants | mutable | activations with RuntimeBundle offsets
// (reference lib/Backend/BackendUtils.cpp:702-730), one HBM allocation per
// function like the reference's OpenCL device manager does with one cl_mem
// (lib/Backends/OpenCL/OpenCLDeviceManager.cpp:391-421).
#include "common.h"

#include <cstring>
#include <new>

namespace mi355x {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    return fail(MI355X_ERR_RUNTIME, "launch of %s failed: %s", what,
                hipGetErrorString(e));
  }
  return MI355X_OK;
}

__global__ void fill_u8_kernel(uint8_t *dst, uint8_t v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = v;
}

// 16 bytes per lane and trip; head and tail bytes one at a time.
__global__ __launch_bounds__(256) void copy_u8_kernel(uint8_t *__restrict__ dst,
                                                      const uint8_t *__restrict__ src,
                                                      size_t n, int vec_ok) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t done = 0;
  if (vec_ok) {
    const size_t nv = n / 16;
    const int4 *s4 = reinterpret_cast<const int4 *>(src);
    int4 *d4 = reinterpret_cast<int4 *>(dst);
    for (size_t i = tid; i < nv; i += stride) d4[i] = s4[i];
    done = nv * 16;
  }
  for (size_t i = done + tid; i < n; i += stride) dst[i] = src[i];
}

// One wavefront that waits `wall_ticks` ticks of the constant-rate device
// clock and reports how many shader-clock cycles went by meanwhile:
// out[0] = shader cycles, out[1] = constant-rate ticks. The wait sleeps between
// polls and ends after max_polls polls at the latest.
__global__ __launch_bounds__(64) void clock_probe_kernel(unsigned long long *out,
                                                         unsigned wall_ticks,
                                                         unsigned max_polls) {
  const unsigned long long w0 = wall_clock64();
  const unsigned long long c0 = clock64();
  unsigned long long w = w0;
  for (unsigned i = 0; i < max_polls && w - w0 < wall_ticks; i++) {
    __builtin_amdgcn_s_sleep(32);
    w = wall_clock64();
  }
  const unsigned long long c1 = clock64();
  if (threadIdx.x == 0) {
    out[0] = c1 - c0;
    out[1] = w - w0;
  }
}

} // namespace mi355x

using namespace mi355x;

// Tensor alignment Glow's allocators use (reference
// include/glow/Support/Memory.h:29); regions are padded to a multiple of it so
// every region base keeps the alignment the offsets were planned for.
static constexpr size_t kTensorAlignment = 64;
// Each region base is aligned to 256 B so 16-byte vector accesses at planned
// offsets stay aligned and regions do not share a cache line.
static constexpr size_t kRegionAlignment = 256;

struct mi355x_arena {
  char *base = nullptr;
  size_t bytes = 0;
  size_t offset[3] = {0, 0, 0};
  size_t size[3] = {0, 0, 0};
};

extern "C" {

const char *mi355x_last_error(void) { return g_err; }

int mi355x_num_devices(int *count) {
  MI355X_REQUIRE(count, "count is NULL");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    *count = 0;
    return fail(MI355X_ERR_DEVICE_NOT_FOUND, "hipGetDeviceCount: %s",
                hipGetErrorString(e));
  }
  *count = n;
  return MI355X_OK;
}

int mi355x_init(int device) {
  int n = 0;
  int rc = mi355x_num_devices(&n);
  if (rc != MI355X_OK) return rc;
  if (device < 0 || device >= n) {
    return fail(MI355X_ERR_DEVICE_NOT_FOUND, "device %d not found (%d present)",
                device, n);
  }
  MI355X_HIP(hipSetDevice(device));
  hipDeviceProp_t p;
  MI355X_HIP(hipGetDeviceProperties(&p, device));
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    return fail(MI355X_ERR_NOT_SUPPORTED,
                "device %d is %s; this library only carries gfx950 code",
                device, p.gcnArchName);
  }
  // per-device set-up of the SparseLengths scratch: the fixed array's address
  // and a buffer for launches on the default stream
  rc = slws_init_device();
  if (rc != MI355X_OK) return rc;
  return slws_reserve_stream(nullptr);
}

int mi355x_device_info(mi355x_info *info) {
  MI355X_REQUIRE(info, "info is NULL");
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  hipDeviceProp_t p;
  MI355X_HIP(hipGetDeviceProperties(&p, dev));
  memset(info, 0, sizeof(*info));
  snprintf(info->name, sizeof(info->name), "%s", p.name);
  snprintf(info->arch, sizeof(info->arch), "%s", p.gcnArchName);
  info->compute_units = p.multiProcessorCount;
  info->clock_khz = p.clockRate;
  info->device = dev;
  info->lds_bytes_per_block = (int32_t)p.sharedMemPerBlock;
  size_t fr = 0, tot = 0;
  MI355X_HIP(hipMemGetInfo(&fr, &tot));
  info->total_memory = tot;
  info->free_memory = fr;
  return MI355X_OK;
}

int mi355x_malloc(void **dptr, size_t bytes) {
  MI355X_REQUIRE(dptr, "dptr is NULL");
  *dptr = nullptr;
  if (bytes == 0) return MI355X_OK;
  MI355X_HIP(hipMalloc(dptr, bytes));
  return MI355X_OK;
}

int mi355x_free(void *dptr) {
  if (dptr) MI355X_HIP(hipFree(dptr));
  return MI355X_OK;
}

int mi355x_host_alloc(void **hptr, size_t bytes) {
  MI355X_REQUIRE(hptr, "hptr is NULL");
  *hptr = nullptr;
  if (bytes == 0) return MI355X_OK;
  MI355X_HIP(hipHostMalloc(hptr, bytes, hipHostMallocDefault));
  return MI355X_OK;
}

int mi355x_host_free(void *hptr) {
  if (hptr) MI355X_HIP(hipHostFree(hptr));
  return MI355X_OK;
}

int mi355x_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL pointer in h2d copy");
  MI355X_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice,
                            as_stream(stream)));
  return MI355X_OK;
}

int mi355x_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL pointer in d2h copy");
  MI355X_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost,
                            as_stream(stream)));
  return MI355X_OK;
}

int mi355x_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL pointer in d2d copy");
  MI355X_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice,
                            as_stream(stream)));
  return MI355X_OK;
}

int mi355x_fill_u8(void *dst, int value, size_t bytes, void *stream) {
  if (bytes == 0) return MI355X_OK;
  MI355X_REQUIRE(dst, "dst is NULL");
  size_t blocks = (bytes + 256 * 16 - 1) / (256 * 16);
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(fill_u8_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     as_stream(stream), (uint8_t *)dst, (uint8_t)value, bytes);
  return check_launch("fill_u8");
}

int mi355x_copy_u8(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL pointer in device copy");
  size_t blocks = (bytes / 16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 256 * 32) blocks = 256 * 32;
  const int vec_ok = ((((uintptr_t)dst) | ((uintptr_t)src)) & 15) == 0;
  hipLaunchKernelGGL(copy_u8_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     as_stream(stream), (uint8_t *)dst, (const uint8_t *)src,
                     bytes, vec_ok);
  return check_launch("copy_u8");
}

int mi355x_shader_clock_probe(uint64_t *out2, uint32_t micros, void *stream) {
  MI355X_REQUIRE(out2, "out2 is NULL");
  MI355X_REQUIRE(micros >= 1 && micros <= 100000, "probe time %u us outside [1, 100000]", micros);
  int dev = 0, khz = 0;
  MI355X_HIP(hipGetDevice(&dev));
  MI355X_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
  MI355X_REQUIRE(khz > 0, "the device reports no constant-rate clock");
  const unsigned ticks = (unsigned)((uint64_t)micros * (uint64_t)khz / 1000);
  // a poll takes well over 100 ns: this many polls outlast the requested time
  const unsigned max_polls = micros * 16 + 1024;
  hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, as_stream(stream),
                     (unsigned long long *)out2, ticks, max_polls);
  return check_launch("clock_probe");
}

int mi355x_wall_clock_khz(int *khz) {
  MI355X_REQUIRE(khz, "khz is NULL");
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  MI355X_HIP(hipDeviceGetAttribute(khz, hipDeviceAttributeWallClockRate, dev));
  return MI355X_OK;
}

int mi355x_stream_create(void **stream) {
  MI355X_REQUIRE(stream, "stream is NULL");
  hipStream_t s;
  // default priority only
  MI355X_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  int rc = slws_reserve_stream(s);
  if (rc != MI355X_OK) {
    (void)hipStreamDestroy(s);
    return rc;
  }
  *stream = s;
  return MI355X_OK;
}

int mi355x_stream_destroy(void *stream) {
  if (stream) {
    // the stream's work is finished before its scratch goes away
    MI355X_HIP(hipStreamSynchronize(as_stream(stream)));
    int rc = slws_release_stream(as_stream(stream));
    if (rc != MI355X_OK) return rc;
    MI355X_HIP(hipStreamDestroy(as_stream(stream)));
  }
  return MI355X_OK;
}

int mi355x_stream_sync(void *stream) {
  MI355X_HIP(hipStreamSynchronize(as_stream(stream)));
  return MI355X_OK;
}

int mi355x_device_sync(void) {
  MI355X_HIP(hipDeviceSynchronize());
  return MI355X_OK;
}

int mi355x_event_create(void **event) {
  MI355X_REQUIRE(event, "event is NULL");
  hipEvent_t e;
  MI355X_HIP(hipEventCreate(&e));
  *event = e;
  return MI355X_OK;
}

int mi355x_event_destroy(void *event) {
  if (event) MI355X_HIP(hipEventDestroy((hipEvent_t)event));
  return MI355X_OK;
}

int mi355x_event_record(void *event, void *stream) {
  MI355X_REQUIRE(event, "event is NULL");
  MI355X_HIP(hipEventRecord((hipEvent_t)event, as_stream(stream)));
  return MI355X_OK;
}

int mi355x_stream_wait_event(void *stream, void *event) {
  MI355X_REQUIRE(event, "event is NULL");
  MI355X_HIP(hipStreamWaitEvent(as_stream(stream), (hipEvent_t)event, 0));
  return MI355X_OK;
}

int mi355x_event_sync(void *event) {
  MI355X_REQUIRE(event, "event is NULL");
  MI355X_HIP(hipEventSynchronize((hipEvent_t)event));
  return MI355X_OK;
}

int mi355x_event_elapsed_ms(void *start, void *stop, float *ms) {
  MI355X_REQUIRE(start && stop && ms, "NULL argument");
  MI355X_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return MI355X_OK;
}

struct mi355x_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

int mi355x_graph_begin_capture(void *stream) {
  MI355X_REQUIRE(stream, "graph capture needs a created stream, not the default one");
  MI355X_HIP(hipStreamBeginCapture(as_stream(stream),
                                   hipStreamCaptureModeThreadLocal));
  return MI355X_OK;
}

int mi355x_graph_end_capture(void *stream, mi355x_graph **graph) {
  MI355X_REQUIRE(stream && graph, "NULL argument");
  *graph = nullptr;
  hipGraph_t g = nullptr;
  MI355X_HIP(hipStreamEndCapture(as_stream(stream), &g));
  hipGraphExec_t e = nullptr;
  hipError_t err = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
  if (err != hipSuccess) {
    (void)hipGraphDestroy(g);
    return fail(MI355X_ERR_RUNTIME, "hipGraphInstantiate: %s",
                hipGetErrorString(err));
  }
  mi355x_graph *out = new (std::nothrow) mi355x_graph();
  if (!out) {
    (void)hipGraphExecDestroy(e);
    (void)hipGraphDestroy(g);
    return fail(MI355X_ERR_RUNTIME, "host allocation failed");
  }
  out->graph = g;
  out->exec = e;
  *graph = out;
  return MI355X_OK;
}

int mi355x_graph_launch(mi355x_graph *graph, void *stream) {
  MI355X_REQUIRE(graph && graph->exec, "graph is NULL");
  MI355X_HIP(hipGraphLaunch(graph->exec, as_stream(stream)));
  return MI355X_OK;
}

int mi355x_graph_destroy(mi355x_graph *graph) {
  if (!graph) return MI355X_OK;
  hipError_t e1 = graph->exec ? hipGraphExecDestroy(graph->exec) : hipSuccess;
  hipError_t e2 = graph->graph ? hipGraphDestroy(graph->graph) : hipSuccess;
  delete graph;
  if (e1 != hipSuccess || e2 != hipSuccess)
    return fail(MI355X_ERR_RUNTIME, "graph destroy: %s",
                hipGetErrorString(e1 != hipSuccess ? e1 : e2));
  return MI355X_OK;
}

static size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int mi355x_arena_create(size_t const_bytes, size_t mutable_bytes,
                        size_t activation_bytes, mi355x_arena **arena) {
  MI355X_REQUIRE(arena, "arena is NULL");
  *arena = nullptr;
  mi355x_arena *a = new (std::nothrow) mi355x_arena();
  if (!a) return fail(MI355X_ERR_RUNTIME, "host allocation failed");
  const size_t sz[3] = {const_bytes, mutable_bytes, activation_bytes};
  size_t off = 0;
  for (int r = 0; r < 3; r++) {
    a->offset[r] = off;
    a->size[r] = sz[r];
    off += round_up(round_up(sz[r], kTensorAlignment), kRegionAlignment);
  }
  a->bytes = off;
  if (off) {
    hipError_t e = hipMalloc((void **)&a->base, off);
    if (e != hipSuccess) {
      delete a;
      return fail(e == hipErrorOutOfMemory ? MI355X_ERR_OUT_OF_DEVICE_MEMORY
                                           : MI355X_ERR_RUNTIME,
                  "arena of %zu bytes: %s", off, hipGetErrorString(e));
    }
  }
  *arena = a;
  return MI355X_OK;
}

int mi355x_arena_destroy(mi355x_arena *arena) {
  if (!arena) return MI355X_OK;
  hipError_t e = arena->base ? hipFree(arena->base) : hipSuccess;
  delete arena;
  if (e != hipSuccess)
    return fail(MI355X_ERR_RUNTIME, "hipFree: %s", hipGetErrorString(e));
  return MI355X_OK;
}

uint64_t mi355x_arena_bytes(const mi355x_arena *arena) {
  return arena ? arena->bytes : 0;
}

static int arena_span(mi355x_arena *a, int region, size_t offset, size_t bytes,
                      char **p) {
  MI355X_REQUIRE(a, "arena is NULL");
  MI355X_REQUIRE(region >= 0 && region < 3, "region %d out of range", region);
  MI355X_REQUIRE(offset <= a->size[region] && bytes <= a->size[region] - offset,
                 "span [%zu, +%zu) outside region %d of %zu bytes", offset,
                 bytes, region, a->size[region]);
  *p = a->base + a->offset[region] + offset;
  return MI355X_OK;
}

int mi355x_arena_ptr(mi355x_arena *arena, int region, size_t offset,
                     void **dptr) {
  MI355X_REQUIRE(dptr, "dptr is NULL");
  *dptr = nullptr;
  char *p = nullptr;
  int rc = arena_span(arena, region, offset, 0, &p);
  if (rc != MI355X_OK) return rc;
  *dptr = p;
  return MI355X_OK;
}

int mi355x_arena_upload(mi355x_arena *arena, int region, size_t offset,
                        const void *host, size_t bytes, void *stream) {
  char *p = nullptr;
  int rc = arena_span(arena, region, offset, bytes, &p);
  if (rc != MI355X_OK) return rc;
  return mi355x_memcpy_h2d(p, host, bytes, stream);
}

int mi355x_arena_download(mi355x_arena *arena, int region, size_t offset,
                          void *host, size_t bytes, void *stream) {
  char *p = nullptr;
  int rc = arena_span(arena, region, offset, bytes, &p);
  if (rc != MI355X_OK) return rc;
  return mi355x_memcpy_d2h(host, p, bytes, stream);
}

} // extern "C"
