// Quantize / Dequantize / RescaleQuantized for int8 tensors: the HBM-bound
// elementwise instructions of the quantized path (reference
// lib/LLVMIRCodeGen/libjit/libjit.cpp:2998-3038). Each lane moves 16 elements
// per trip with 16-byte accesses on the int8 side and 4 x 16 bytes on the
// fp32 side; tensors whose base is not 16-byte aligned, and the last n % 16
// elements, go through the scalar tail.
#include "common.h"

// Every multiply and add below must round on its own (the CPU code this
// reproduces has no fused multiply-add). The pragma covers contraction in the
// front end; the build must also pass -ffp-contract=off (the Makefile does),
// because HIP's default "fast" mode fuses in the back end regardless.
#pragma clang fp contract(off)
#include "requant.h"

namespace mi355x {

constexpr int kEwThreads = 256;
constexpr int kEwPerLane = 16;

// clip((int32)nearbyintf(x / scale + offset)): IEEE division and
// round-half-even, each operation rounded on its own.
__device__ __forceinline__ int32_t quantize_one(float x, float scale,
                                                float offset) {
  float r = rintf(__fadd_rn(__fdiv_rn(x, scale), offset));
  return clip_i8((int32_t)r);
}

__device__ __forceinline__ uint32_t pack4(int32_t a, int32_t b, int32_t c,
                                          int32_t d) {
  return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) |
         ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}

__device__ __forceinline__ int32_t sext8(uint32_t w, int i) {
  return (int32_t)(int8_t)(w >> (8 * i));
}

__global__ __launch_bounds__(kEwThreads) void quantize_i8_kernel(
    int8_t *__restrict__ dst, const float *__restrict__ src, size_t n,
    size_t vec_chunks, float scale, float offset) {
  const size_t t = (size_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (t < vec_chunks) {
    const float4 *s = reinterpret_cast<const float4 *>(src) + t * 4;
    float4 a = s[0], b = s[1], c = s[2], d = s[3];
    uint4 o;
    o.x = pack4(quantize_one(a.x, scale, offset), quantize_one(a.y, scale, offset),
                quantize_one(a.z, scale, offset), quantize_one(a.w, scale, offset));
    o.y = pack4(quantize_one(b.x, scale, offset), quantize_one(b.y, scale, offset),
                quantize_one(b.z, scale, offset), quantize_one(b.w, scale, offset));
    o.z = pack4(quantize_one(c.x, scale, offset), quantize_one(c.y, scale, offset),
                quantize_one(c.z, scale, offset), quantize_one(c.w, scale, offset));
    o.w = pack4(quantize_one(d.x, scale, offset), quantize_one(d.y, scale, offset),
                quantize_one(d.z, scale, offset), quantize_one(d.w, scale, offset));
    reinterpret_cast<uint4 *>(dst)[t] = o;
  }
  // scalar tail: elements [vec_chunks*16, n), one per lane from the front
  const size_t tail0 = vec_chunks * kEwPerLane;
  const size_t stride = (size_t)gridDim.x * kEwThreads;
  for (size_t i = tail0 + t; i < n; i += stride)
    dst[i] = (int8_t)quantize_one(src[i], scale, offset);
}

// A block converts tiles of 256 x 16 elements in four steps; in each step
// consecutive lanes take consecutive groups of 4 elements, so a wavefront reads
// 256 contiguous bytes and writes 1 KiB contiguous.
__global__ __launch_bounds__(kEwThreads) void dequantize_i8_kernel(
    float *__restrict__ dst, const int8_t *__restrict__ src, size_t n,
    size_t vec_chunks, float scale, int32_t offset) {
  constexpr size_t kTile = (size_t)kEwThreads * kEwPerLane;
  const size_t tiles = vec_chunks / kEwThreads;       // whole tiles only
  if (blockIdx.x < tiles) {
    const size_t base = (size_t)blockIdx.x * kTile + (size_t)threadIdx.x * 4;
#pragma unroll
    for (int st = 0; st < kEwPerLane / 4; st++) {
      const size_t e = base + (size_t)st * kEwThreads * 4;
      const uint32_t w = *reinterpret_cast<const uint32_t *>(src + e);
      float4 f;
      f.x = __fmul_rn(scale, (float)(sext8(w, 0) - offset));
      f.y = __fmul_rn(scale, (float)(sext8(w, 1) - offset));
      f.z = __fmul_rn(scale, (float)(sext8(w, 2) - offset));
      f.w = __fmul_rn(scale, (float)(sext8(w, 3) - offset));
      *reinterpret_cast<float4 *>(dst + e) = f;
    }
  }
  // scalar tail: elements [tiles * kTile, n)
  const size_t t = (size_t)blockIdx.x * kEwThreads + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * kEwThreads;
  for (size_t i = tiles * kTile + t; i < n; i += stride)
    dst[i] = __fmul_rn(scale, (float)((int32_t)src[i] - offset));
}

// RescaleQuantized with no pre-shift, a scale below 2^23 and room below the
// post-shift for the offsets: ((q - in_off) * s + rtn) >> post) + out_off
// == (q * s + folded) >> post with folded = rtn - in_off * s + (out_off << post),
// exact in 32 bits under the bound the caller checks (no intermediate leaves
// int32, so (A >> p) + d == (A + (d << p)) >> p). One 24-bit multiply-add, one
// shift and one clamp per value instead of nine instructions: the kernel is
// bound by its instruction stream, not by memory.
__global__ __launch_bounds__(kEwThreads) void rescale_folded_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, size_t n, size_t vec_chunks,
    int32_t folded, int32_t post, int32_t scale) {
  auto one = [=](int32_t q) {
    return med3_i32((int32_t)((uint32_t)__mul24(q, scale) + (uint32_t)folded) >> post, -128, 127);
  };
  const size_t t = (size_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (t < vec_chunks) {
    uint4 q = reinterpret_cast<const uint4 *>(src)[t];
    uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; j++)
      w[j] = pack4(one(sext8(w[j], 0)), one(sext8(w[j], 1)), one(sext8(w[j], 2)),
                   one(sext8(w[j], 3)));
    reinterpret_cast<uint4 *>(dst)[t] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  const size_t tail0 = vec_chunks * kEwPerLane;
  const size_t stride = (size_t)gridDim.x * kEwThreads;
  for (size_t i = tail0 + t; i < n; i += stride) dst[i] = (int8_t)one((int32_t)src[i]);
}

template <bool SMALL>
__global__ __launch_bounds__(kEwThreads) void rescale_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, size_t n,
    size_t vec_chunks, int32_t out_offset, int32_t in_offset, int32_t pre,
    int32_t post, int32_t scale) {
  const size_t t = (size_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (t < vec_chunks) {
    uint4 q = reinterpret_cast<const uint4 *>(src)[t];
    uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int32_t r[4];
#pragma unroll
      for (int b = 0; b < 4; b++)
        r[b] = clip_i8(scale_i32_sel<SMALL>(sext8(w[j], b) - in_offset, pre, post,
                                            scale, out_offset));
      w[j] = pack4(r[0], r[1], r[2], r[3]);
    }
    reinterpret_cast<uint4 *>(dst)[t] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  const size_t tail0 = vec_chunks * kEwPerLane;
  const size_t stride = (size_t)gridDim.x * kEwThreads;
  for (size_t i = tail0 + t; i < n; i += stride)
    dst[i] = (int8_t)clip_i8(scale_i32_sel<SMALL>((int32_t)src[i] - in_offset, pre,
                                                  post, scale, out_offset));
}

// RescaleQuantized of a [rows x cols] tensor written as a slice of a wider one
// (dst rows dst_row_stride bytes apart): V bytes per lane. The host keeps
// rows * cols / V below 2^31, so the index arithmetic is 32-bit.
template <int V>
__global__ __launch_bounds__(kEwThreads) void rescale_rows_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, unsigned total, unsigned per_row,
    long long dst_row_stride, int32_t out_offset, int32_t in_offset, int32_t pre,
    int32_t post, int32_t scale) {
  const unsigned i = blockIdx.x * kEwThreads + threadIdx.x;
  if (i >= total) return;
  const unsigned r = i / per_row;
  const unsigned c = (i - r * per_row) * V;
  const int8_t *s = src + (size_t)i * V;
  int8_t *d = dst + (long long)r * dst_row_stride + c;
  if constexpr (V == 1) {
    d[0] = (int8_t)clip_i8(scale_i32((int32_t)s[0] - in_offset, pre, post, scale, out_offset));
  } else {
    uint32_t w[V / 4];
    if constexpr (V == 16) {
      const uint4 q = *reinterpret_cast<const uint4 *>(s);
      w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w;
    } else {
      w[0] = *reinterpret_cast<const uint32_t *>(s);
    }
#pragma unroll
    for (int j = 0; j < V / 4; j++) {
      int32_t q[4];
#pragma unroll
      for (int b = 0; b < 4; b++)
        q[b] = clip_i8(scale_i32(sext8(w[j], b) - in_offset, pre, post, scale, out_offset));
      w[j] = pack4(q[0], q[1], q[2], q[3]);
    }
    if constexpr (V == 16)
      *reinterpret_cast<uint4 *>(d) = make_uint4(w[0], w[1], w[2], w[3]);
    else
      *reinterpret_cast<uint32_t *>(d) = w[0];
  }
}

// Dequantize followed by Sigmoid (libjit_sigmoid_kernel_f on the dequantized
// value): 1 / (expf(-(scale * (q - offset))) + 1).
__global__ __launch_bounds__(kEwThreads) void dequantize_sigmoid_kernel(
    float *__restrict__ dst, const int8_t *__restrict__ src, size_t n, float scale,
    int32_t offset) {
  const size_t stride = (size_t)gridDim.x * kEwThreads;
  for (size_t i = (size_t)blockIdx.x * kEwThreads + threadIdx.x; i < n; i += stride) {
    const float x = __fmul_rn(scale, (float)((int32_t)src[i] - offset));
    dst[i] = __fdiv_rn(1.0f, __fadd_rn(expf(-x), 1.0f));
  }
}

static bool aligned16(const void *a, const void *b) {
  return (((uintptr_t)a | (uintptr_t)b) & 15) == 0;
}

// Grid covering `vec_chunks` 16-element chunks, and at least one block so the
// tail loop runs.
static unsigned ew_blocks(size_t vec_chunks) {
  size_t b = (vec_chunks + kEwThreads - 1) / kEwThreads;
  return (unsigned)(b ? b : 1);
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

int mi355x_quantize_i8(int8_t *dst, const float *src, size_t n, float scale,
                       int32_t offset, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(n / kEwPerLane / kEwThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = aligned16(dst, src) ? n / kEwPerLane : 0;
  hipLaunchKernelGGL(quantize_i8_kernel, dim3(ew_blocks(chunks)),
                     dim3(kEwThreads), 0, as_stream(stream), dst, src, n,
                     chunks, scale, (float)offset);
  return check_launch("quantize_i8");
}

int mi355x_dequantize_i8(float *dst, const int8_t *src, size_t n, float scale,
                         int32_t offset, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(n / kEwPerLane / kEwThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = aligned16(dst, src) ? n / kEwPerLane : 0;
  hipLaunchKernelGGL(dequantize_i8_kernel, dim3(ew_blocks(chunks)),
                     dim3(kEwThreads), 0, as_stream(stream), dst, src, n,
                     chunks, scale, offset);
  return check_launch("dequantize_i8");
}

int mi355x_rescale_i8(int8_t *dst, const int8_t *src, size_t n,
                      int32_t out_offset, int32_t in_offset, int32_t pre,
                      int32_t post, int32_t scale, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(shift_ok(pre) && shift_ok(post),
                 "pre/post shift outside [0, 31]: %d %d", pre, post);
  MI355X_REQUIRE(n / kEwPerLane / kEwThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = aligned16(dst, src) ? n / kEwPerLane : 0;
  // |q - in_offset| < 2^23 always holds for int8 data when the offset does;
  // with a scale below 2^23 too, the 24-bit multiplier is exact
  const bool small = scale > -(1 << 23) && scale < (1 << 23) &&
                     in_offset > -(1 << 22) && in_offset < (1 << 22);
  // everything folded into one constant: |(q - in_off) * s| + rtn + |out_off << post|
  // stays below 2^31 (q int8, so |q - in_off| < 2^8 + |in_off|)
  const long long mag = (256ll + std::llabs((long long)in_offset)) * std::llabs((long long)scale) +
                        (post > 0 ? (1ll << (post - 1)) : 0) +
                        (std::llabs((long long)out_offset) << post);
  if (small && pre == 0 && mag < (1ll << 31)) {
    const int32_t folded = (int32_t)((post > 0 ? (1ll << (post - 1)) : 0) -
                                     (long long)in_offset * scale +
                                     ((long long)out_offset << post));
    hipLaunchKernelGGL(rescale_folded_i8_kernel, dim3(ew_blocks(chunks)), dim3(kEwThreads), 0,
                       as_stream(stream), dst, src, n, chunks, folded, post, scale);
    return check_launch("rescale_i8");
  }
  if (small)
    hipLaunchKernelGGL(rescale_i8_kernel<true>, dim3(ew_blocks(chunks)),
                       dim3(kEwThreads), 0, as_stream(stream), dst, src, n,
                       chunks, out_offset, in_offset, pre, post, scale);
  else
    hipLaunchKernelGGL(rescale_i8_kernel<false>, dim3(ew_blocks(chunks)),
                       dim3(kEwThreads), 0, as_stream(stream), dst, src, n,
                       chunks, out_offset, in_offset, pre, post, scale);
  return check_launch("rescale_i8");
}

int mi355x_rescale_rows_i8(int8_t *dst, const int8_t *src, size_t rows, size_t cols,
                           size_t dst_row_stride, int32_t out_offset, int32_t in_offset,
                           int32_t pre, int32_t post, int32_t scale, void *stream) {
  if (rows == 0 || cols == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(shift_ok(pre) && shift_ok(post),
                 "pre/post shift outside [0, 31]: %d %d", pre, post);
  MI355X_REQUIRE(dst_row_stride >= cols, "rows of %zu bytes overlap at a stride of %zu", cols,
                 dst_row_stride);
  MI355X_REQUIRE(rows < (1ull << 40) && cols < (1u << 30) && dst_row_stride < (1ull << 40),
                 "tensor too large");
  const uintptr_t both = (uintptr_t)dst | (uintptr_t)src;
  const int v = (cols % 16 == 0 && dst_row_stride % 16 == 0 && (both & 15) == 0)  ? 16
                : (cols % 4 == 0 && dst_row_stride % 4 == 0 && (both & 3) == 0) ? 4
                                                                                  : 1;
  const size_t work = rows * (cols / v);
  MI355X_REQUIRE(work < 0x7fffffffu, "tensor too large");
  const unsigned blocks = (unsigned)((work + kEwThreads - 1) / kEwThreads);
#define MI355X_RESCALE_ROWS(V)                                                                  \
  hipLaunchKernelGGL(rescale_rows_i8_kernel<V>, dim3(blocks), dim3(kEwThreads), 0,              \
                     as_stream(stream), dst, src, (unsigned)work, (unsigned)(cols / V),         \
                     (long long)dst_row_stride, out_offset, in_offset, pre, post, scale)
  if (v == 16) MI355X_RESCALE_ROWS(16);
  else if (v == 4) MI355X_RESCALE_ROWS(4);
  else MI355X_RESCALE_ROWS(1);
#undef MI355X_RESCALE_ROWS
  return check_launch("rescale_rows_i8");
}

int mi355x_dequantize_sigmoid(float *dst, const int8_t *src, size_t n, float scale,
                              int32_t offset, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  size_t blocks = (n + kEwThreads - 1) / kEwThreads;
  if (blocks > 256 * 64) blocks = 256 * 64;
  hipLaunchKernelGGL(dequantize_sigmoid_kernel, dim3((unsigned)blocks), dim3(kEwThreads), 0,
                     as_stream(stream), dst, src, n, scale, offset);
  return check_launch("dequantize_sigmoid");
}

} // extern "C"
