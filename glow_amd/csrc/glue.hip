// The int8 glue operators between the matrix-core kernels of a quantized
// network: ElementAdd (optionally followed by Relu in the same pass), Relu,
// MaxPool, AvgPool on NHWC int8 tensors, and the fp32 SoftMax at the end
// (reference lib/LLVMIRCodeGen/libjit/libjit.cpp:1593-1603, 1851-1858,
// 812-884, 2592-2597, 2812-2880, 3058-3082). All are HBM-bound: 16-byte
// accesses along the channel dimension, integer arithmetic bit-identical to
// the CPU code.
#include "common.h"

#include <hip/hip_fp16.h>

#pragma clang fp contract(off)
#include "requant.h"

namespace mi355x {

constexpr int kGlueThreads = 256;

__device__ __forceinline__ uint32_t pack4b(int32_t a, int32_t b, int32_t c, int32_t d) {
  return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) |
         ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}
__device__ __forceinline__ int32_t sx8(uint32_t w, int i) {
  return (int32_t)(int8_t)(w >> (8 * i));
}

struct AddParams {
  int32_t dest_off, lhs_off, rhs_off;
  int32_t lhs_pre, lhs_post, lhs_scale, rhs_pre, rhs_post, rhs_scale;
  // optional Relu stage applied to the (already clipped) sum
  int32_t relu_dest_off, relu_pre, relu_post, relu_scale;
};

// SMALL: offsets and scales are below 2^23 in magnitude (checked on the host),
// which lets the multiplies run on the 24-bit multiplier.
template <bool RELU, bool SMALL>
__device__ __forceinline__ int32_t add_one(int32_t l, int32_t r, const AddParams &p) {
  const int32_t a = scale_i32_sel<SMALL>(l - p.lhs_off, p.lhs_pre, p.lhs_post, p.lhs_scale, 0);
  const int32_t b = scale_i32_sel<SMALL>(r - p.rhs_off, p.rhs_pre, p.rhs_post, p.rhs_scale, 0);
  int32_t v = clip_i8((int32_t)((uint32_t)a + (uint32_t)b + (uint32_t)p.dest_off));
  if (RELU) {
    // libjit_element_relu_i8 with srcOffset = the sum's offset
    const int32_t so = (int32_t)(int8_t)p.dest_off;
    v = max(v, so);
    v = clip_i8(scale_i32_sel<SMALL>(v - so, p.relu_pre, p.relu_post, p.relu_scale,
                                     p.relu_dest_off));
  }
  return v;
}

template <bool RELU, bool SMALL>
__global__ __launch_bounds__(kGlueThreads) void add_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ lhs,
    const int8_t *__restrict__ rhs, size_t n, size_t vec_chunks, AddParams p) {
  const size_t t = (size_t)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t < vec_chunks) {
    const uint4 a = reinterpret_cast<const uint4 *>(lhs)[t];
    const uint4 b = reinterpret_cast<const uint4 *>(rhs)[t];
    const uint32_t wa[4] = {a.x, a.y, a.z, a.w}, wb[4] = {b.x, b.y, b.z, b.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = pack4b(add_one<RELU, SMALL>(sx8(wa[j], 0), sx8(wb[j], 0), p),
                    add_one<RELU, SMALL>(sx8(wa[j], 1), sx8(wb[j], 1), p),
                    add_one<RELU, SMALL>(sx8(wa[j], 2), sx8(wb[j], 2), p),
                    add_one<RELU, SMALL>(sx8(wa[j], 3), sx8(wb[j], 3), p));
    reinterpret_cast<uint4 *>(dst)[t] = make_uint4(o[0], o[1], o[2], o[3]);
  }
  const size_t stride = (size_t)gridDim.x * kGlueThreads;
  for (size_t i = vec_chunks * 16 + t; i < n; i += stride)
    dst[i] = (int8_t)add_one<RELU, SMALL>(lhs[i], rhs[i], p);
}

__device__ __forceinline__ int32_t relu_one(int32_t v, int32_t so, int32_t doff,
                                            int32_t pre, int32_t post, int32_t scale) {
  v = max(v, so);
  return clip_i8(scale_i32(v - so, pre, post, scale, doff));
}

static bool fits24(int32_t v) { return v > -(1 << 23) && v < (1 << 23); }
// an int8 value minus such an offset still fits 24 bits
static bool off24(int32_t v) { return v > -(1 << 22) && v < (1 << 22); }

__global__ __launch_bounds__(kGlueThreads) void relu_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, size_t n,
    size_t vec_chunks, int32_t so, int32_t doff, int32_t pre, int32_t post,
    int32_t scale) {
  const size_t t = (size_t)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t < vec_chunks) {
    const uint4 a = reinterpret_cast<const uint4 *>(src)[t];
    const uint32_t wa[4] = {a.x, a.y, a.z, a.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = pack4b(relu_one(sx8(wa[j], 0), so, doff, pre, post, scale),
                    relu_one(sx8(wa[j], 1), so, doff, pre, post, scale),
                    relu_one(sx8(wa[j], 2), so, doff, pre, post, scale),
                    relu_one(sx8(wa[j], 3), so, doff, pre, post, scale));
    reinterpret_cast<uint4 *>(dst)[t] = make_uint4(o[0], o[1], o[2], o[3]);
  }
  const size_t stride = (size_t)gridDim.x * kGlueThreads;
  for (size_t i = vec_chunks * 16 + t; i < n; i += stride)
    dst[i] = (int8_t)relu_one(src[i], so, doff, pre, post, scale);
}

// One int8 value -> one int8 value, 16 values per lane; F(v) is the operation.
template <class F>
__device__ __forceinline__ void map_i8(int8_t *__restrict__ dst, const int8_t *__restrict__ src,
                                       size_t n, size_t vec_chunks, F f) {
  const size_t t = (size_t)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t < vec_chunks) {
    const uint4 a = reinterpret_cast<const uint4 *>(src)[t];
    const uint32_t wa[4] = {a.x, a.y, a.z, a.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = pack4b(f(sx8(wa[j], 0)), f(sx8(wa[j], 1)), f(sx8(wa[j], 2)), f(sx8(wa[j], 3)));
    reinterpret_cast<uint4 *>(dst)[t] = make_uint4(o[0], o[1], o[2], o[3]);
  }
  const size_t stride = (size_t)gridDim.x * kGlueThreads;
  for (size_t i = vec_chunks * 16 + t; i < n; i += stride) dst[i] = (int8_t)f((int32_t)src[i]);
}

// libjit_element_clip_i8: clip(scale(min(max(v, lo), hi) - so) + doff)
__global__ __launch_bounds__(kGlueThreads) void clip_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, size_t n, size_t vec_chunks,
    int32_t lo, int32_t hi, int32_t so, int32_t doff, int32_t pre, int32_t post, int32_t scale) {
  map_i8(dst, src, n, vec_chunks, [=](int32_t v) {
    v = min(max(v, lo), hi);
    return clip_i8(scale_i32(v - so, pre, post, scale, doff));
  });
}

// libjit_element_leaky_relu_i8: one rescale for values at or above the input
// offset, another (alpha folded in) below it
__global__ __launch_bounds__(kGlueThreads) void leaky_relu_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, size_t n, size_t vec_chunks,
    int32_t so, int32_t doff, int32_t ppre, int32_t ppost, int32_t pscale, int32_t npre,
    int32_t npost, int32_t nscale) {
  map_i8(dst, src, n, vec_chunks, [=](int32_t v) {
    const bool pos = v >= so;
    return clip_i8(scale_i32(v - so, pos ? ppre : npre, pos ? ppost : npost,
                             pos ? pscale : nscale, doff));
  });
}

// libjit_element_maxsplat_kernel_i8: max(v, value)
__global__ __launch_bounds__(kGlueThreads) void max_splat_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, size_t n, size_t vec_chunks,
    int32_t value) {
  map_i8(dst, src, n, vec_chunks, [=](int32_t v) { return max(v, value); });
}

// libjit_batchedadd_i8 / _i32_i8: dest[n][i] = clip(scale(batch[n][i] - bo) +
// scale(slice[i] - so) + doff). One lane per 4 consecutive elements of a slice
// position (slice_size % 4 == 0) or per element.
template <class ST>
__global__ __launch_bounds__(kGlueThreads) void batched_add_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ batch, const ST *__restrict__ slice,
    size_t total, size_t slice_size, int vec4, int32_t doff, int32_t bo, int32_t so,
    int32_t bpre, int32_t bpost, int32_t bscale, int32_t spre, int32_t spost, int32_t sscale) {
  const size_t stride = (size_t)gridDim.x * kGlueThreads;
  auto one = [=](int32_t b, int32_t s) {
    const int32_t x = scale_i32((int32_t)((uint32_t)b - (uint32_t)bo), bpre, bpost, bscale, 0);
    const int32_t y = scale_i32((int32_t)((uint32_t)s - (uint32_t)so), spre, spost, sscale, 0);
    return clip_i8((int32_t)((uint32_t)x + (uint32_t)y + (uint32_t)doff));
  };
  if (vec4) {
    for (size_t q = (size_t)blockIdx.x * kGlueThreads + threadIdx.x; q < total / 4; q += stride) {
      const size_t i = (q * 4) % slice_size;
      const uint32_t w = reinterpret_cast<const uint32_t *>(batch)[q];
      reinterpret_cast<uint32_t *>(dst)[q] =
          pack4b(one(sx8(w, 0), (int32_t)slice[i]), one(sx8(w, 1), (int32_t)slice[i + 1]),
                 one(sx8(w, 2), (int32_t)slice[i + 2]), one(sx8(w, 3), (int32_t)slice[i + 3]));
    }
  } else {
    for (size_t e = (size_t)blockIdx.x * kGlueThreads + threadIdx.x; e < total; e += stride)
      dst[e] = (int8_t)one((int32_t)batch[e], (int32_t)slice[e % slice_size]);
  }
}

struct PoolGeom {
  int N, IH, IW, C, OH, OW, KH, KW, SH, SW, padT, padL;
};

// window of valid taps of one output position (libjit_defs.h:257-275)
__device__ __forceinline__ void pool_window(int in_min, int in_size, int k, int &lo, int &len) {
  lo = max(0, -in_min);
  const int hi = min(k, in_size - in_min);
  len = max(0, hi - lo);
}

// Walks the valid taps of a pooling window in row-major order without a
// division per tap and without branches (selects only, so that the loads of a
// group stay in one basic block). `off` is the tap's element offset from the
// window's first tap; past the last tap it stays on the last one.
struct TapWalk {
  long long off;
  int fw, wl, left;
  long long col_step, row_step;
  __device__ __forceinline__ TapWalk(int hl, int wl_, int iw, int c)
      : off(0), fw(0), wl(wl_), left(hl * wl_), col_step(c),
        row_step((long long)(iw - wl_ + 1) * c) {}
  __device__ __forceinline__ void step() {
    const bool adv = left > 1;
    const bool wrap = fw + 1 == wl;
    off += adv ? (wrap ? row_step : col_step) : 0;
    fw = adv ? (wrap ? 0 : fw + 1) : fw;
    --left;
  }
};

// One thread per output pixel and group of VEC channels (VEC bytes per load).
// The taps are read U at a time, all loads of a group issued before the first
// is used; a group's slots beyond the window re-read its last tap, which a
// maximum does not see.
template <int VEC, int U>
__global__ __launch_bounds__(kGlueThreads) void max_pool_i8_kernel(
    int8_t *__restrict__ out, const int8_t *__restrict__ in, PoolGeom g,
    int32_t out_offset, long long total) {
  const long long t = (long long)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t >= total) return;
  const int cg = g.C / VEC;
  const int c0 = (int)(t % cg) * VEC;
  long long pix = t / cg;
  const int ow = (int)(pix % g.OW);
  pix /= g.OW;
  const int oh = (int)(pix % g.OH);
  const int n = (int)(pix / g.OH);
  int h0, hl, w0, wl;
  const int ih_min = oh * g.SH - g.padT, iw_min = ow * g.SW - g.padL;
  pool_window(ih_min, g.IH, g.KH, h0, hl);
  pool_window(iw_min, g.IW, g.KW, w0, wl);
  const bool empty = hl == 0 || wl == 0;
  int32_t m[VEC];
#pragma unroll
  for (int i = 0; i < VEC; i++) m[i] = -128;
  if (!empty) {
    const int8_t *base =
        in + (((long long)n * g.IH + (ih_min + h0)) * g.IW + (iw_min + w0)) * g.C + c0;
    TapWalk tw(hl, wl, g.IW, g.C);
    while (tw.left > 0) {
      if constexpr (VEC == 16) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          v[u] = *reinterpret_cast<const uint4 *>(base + tw.off);
          tw.step();
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
          const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
          for (int i = 0; i < 16; i++) m[i] = max(m[i], sx8(w[i >> 2], i & 3));
        }
      } else {
        int32_t v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          v[u] = base[tw.off];
          tw.step();
        }
#pragma unroll
        for (int u = 0; u < U; u++) m[0] = max(m[0], v[u]);
      }
    }
  }
  int8_t *q = out + (((long long)n * g.OH + oh) * g.OW + ow) * g.C + c0;
  if constexpr (VEC == 16) {
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = empty ? pack4b(out_offset, out_offset, out_offset, out_offset)
                   : pack4b(m[4 * j], m[4 * j + 1], m[4 * j + 2], m[4 * j + 3]);
    *reinterpret_cast<uint4 *>(q) = make_uint4(o[0], o[1], o[2], o[3]);
  } else {
    q[0] = (int8_t)(empty ? out_offset : m[0]);
  }
}

// libjit_div_round_i32 (libjit_defs.h:239-244)
__device__ __forceinline__ int32_t div_round_i32(int32_t v, int32_t d) {
  const int32_t rnd = d >> 1;
  return v > 0 ? (v + rnd) / d : (v - rnd) / d;
}

// Taps are read U at a time like the maximum's; here the slots beyond the
// window are left out of the sum.
template <int VEC, int U>
__global__ __launch_bounds__(kGlueThreads) void avg_pool_i8_kernel(
    int8_t *__restrict__ out, const int8_t *__restrict__ in, PoolGeom g,
    int count_include_pads, int32_t out_offset, int32_t in_offset, int32_t pre,
    int32_t post, int32_t scale, long long total) {
  const long long t = (long long)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t >= total) return;
  const int cg = g.C / VEC;
  const int c0 = (int)(t % cg) * VEC;
  long long pix = t / cg;
  const int ow = (int)(pix % g.OW);
  pix /= g.OW;
  const int oh = (int)(pix % g.OH);
  const int n = (int)(pix / g.OH);
  int h0, hl, w0, wl;
  const int ih_min = oh * g.SH - g.padT, iw_min = ow * g.SW - g.padL;
  pool_window(ih_min, g.IH, g.KH, h0, hl);
  pool_window(iw_min, g.IW, g.KW, w0, wl);
  int32_t s[VEC];
#pragma unroll
  for (int i = 0; i < VEC; i++) s[i] = 0;
  if (hl > 0 && wl > 0) {
    const int8_t *base =
        in + (((long long)n * g.IH + (ih_min + h0)) * g.IW + (iw_min + w0)) * g.C + c0;
    TapWalk tw(hl, wl, g.IW, g.C);
    while (tw.left > 0) {
      const int live = tw.left;
      if constexpr (VEC == 4) {
        uint32_t v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          v[u] = *reinterpret_cast<const uint32_t *>(base + tw.off);
          tw.step();
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
          const bool keep = u < live;
#pragma unroll
          for (int i = 0; i < 4; i++) s[i] += keep ? sx8(v[u], i) - in_offset : 0;
        }
      } else {
        int32_t v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          v[u] = base[tw.off];
          tw.step();
        }
#pragma unroll
        for (int u = 0; u < U; u++) s[0] += u < live ? v[u] - in_offset : 0;
      }
    }
  }
  const int32_t area = hl * wl;
  int32_t r[VEC];
#pragma unroll
  for (int i = 0; i < VEC; i++) {
    if (count_include_pads) {
      r[i] = clip_i8(scale_i32(s[i], pre, post, scale, out_offset));
    } else if (area == 0) {
      r[i] = (int32_t)(int8_t)out_offset;
    } else {
      const int32_t v = scale_i32(s[i], pre, post, scale, 0);
      r[i] = clip_i8((int32_t)((uint32_t)div_round_i32(v, area) + (uint32_t)out_offset));
    }
  }
  int8_t *q = out + (((long long)n * g.OH + oh) * g.OW + ow) * g.C + c0;
  if constexpr (VEC == 4)
    *reinterpret_cast<uint32_t *>(q) = pack4b(r[0], r[1], r[2], r[3]);
  else
    q[0] = (int8_t)r[0];
}

__device__ __forceinline__ float block_reduce(float v, float *s, bool is_max) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = is_max ? fmaxf(v, o) : __fadd_rn(v, o);
  }
  __syncthreads();
  if (lane == 0) s[wave] = v;
  __syncthreads();
  float r = s[0];
  for (int w = 1; w < kGlueThreads / 64; w++) r = is_max ? fmaxf(r, s[w]) : __fadd_rn(r, s[w]);
  return r;
}

// One block per row: max, exp and sum, divide (libjit_softmax_f). The sum is
// formed in a different order than the CPU's sequential loop, so results agree
// to fp32 rounding, not bit for bit.
// DEQ: the row is int8 and dequantized on the way in (scale * (q - offset),
// the very float Dequantize writes), which saves the float tensor in between.
template <bool DEQ>
__global__ __launch_bounds__(kGlueThreads) void softmax_f32_kernel(
    float *__restrict__ out, const void *__restrict__ in, int cols, float scale, int32_t offset) {
  __shared__ float s[kGlueThreads / 64];
  const long long row0 = (long long)blockIdx.x * cols;
  auto x = [&](int i) -> float {
    if constexpr (DEQ)
      return __fmul_rn(scale, (float)((int32_t)reinterpret_cast<const int8_t *>(in)[row0 + i] - offset));
    else
      return reinterpret_cast<const float *>(in)[row0 + i];
  };
  float *y = out + row0;
  float m = -INFINITY;
  for (int i = threadIdx.x; i < cols; i += kGlueThreads) m = fmaxf(m, x(i));
  m = block_reduce(m, s, true);
  float sum = 0.0f;
  for (int i = threadIdx.x; i < cols; i += kGlueThreads) {
    const float e = expf(__fsub_rn(x(i), m));
    y[i] = e;
    sum = __fadd_rn(sum, e);
  }
  sum = block_reduce(sum, s, false);
  for (int i = threadIdx.x; i < cols; i += kGlueThreads) y[i] = __fdiv_rn(y[i], sum);
}

// ---- data movement and the small operators of ranking models ----------------

__global__ __launch_bounds__(kGlueThreads) void convert_f16_f32_kernel(
    float *__restrict__ dst, const __half *__restrict__ src, size_t n) {
  const size_t stride = (size_t)gridDim.x * kGlueThreads;
  for (size_t i = (size_t)blockIdx.x * kGlueThreads + threadIdx.x; i < n; i += stride)
    dst[i] = __half2float(src[i]);
}

// dst[r][off + b] = src[r][b]: rows of row_bytes bytes into rows of a wider tensor
__global__ __launch_bounds__(kGlueThreads) void insert_rows_kernel(
    uint8_t *__restrict__ dst, const uint8_t *__restrict__ src, long long rows,
    long long row_bytes, long long dst_stride, long long dst_off, int unit) {
  const long long per_row = row_bytes / unit;
  const long long total = rows * per_row;
  const long long stride = (long long)gridDim.x * kGlueThreads;
  for (long long i = (long long)blockIdx.x * kGlueThreads + threadIdx.x; i < total; i += stride) {
    const long long r = i / per_row, c = (i - r * per_row) * unit;
    const uint8_t *s = src + r * row_bytes + c;
    uint8_t *d = dst + r * dst_stride + dst_off + c;
    if (unit == 16) *reinterpret_cast<uint4 *>(d) = *reinterpret_cast<const uint4 *>(s);
    else if (unit == 4) *reinterpret_cast<uint32_t *>(d) = *reinterpret_cast<const uint32_t *>(s);
    else *d = *s;
  }
}

// dst [B][cols][rows] = src [B][rows][cols]
__global__ __launch_bounds__(kGlueThreads) void batch_transpose_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, long long batch, int rows,
    int cols) {
  const long long per = (long long)rows * cols;
  const long long total = batch * per;
  const long long stride = (long long)gridDim.x * kGlueThreads;
  for (long long i = (long long)blockIdx.x * kGlueThreads + threadIdx.x; i < total; i += stride) {
    const long long b = i / per;
    const int e = (int)(i - b * per);        // index in the destination sample
    const int c = e / rows, r = e - c * rows;
    dst[i] = src[b * per + (long long)r * cols + c];
  }
}

// libjit_gather: dest[sample][i] = data[sample][indices[i]] for slices of
// slice_bytes bytes; an index outside the sample yields zero bytes.
template <typename IDX>
__global__ __launch_bounds__(kGlueThreads) void gather_kernel(
    uint8_t *__restrict__ dst, const uint8_t *__restrict__ data, const IDX *__restrict__ idx,
    long long num_indices, long long slice_bytes, long long samples, long long sample_bytes,
    long long dst_sample_stride) {
  const long long total = samples * num_indices * slice_bytes;
  const long long stride = (long long)gridDim.x * kGlueThreads;
  const long long slices = sample_bytes / slice_bytes;
  for (long long i = (long long)blockIdx.x * kGlueThreads + threadIdx.x; i < total; i += stride) {
    const long long b = i % slice_bytes;
    const long long t = i / slice_bytes;
    const long long k = t % num_indices, smp = t / num_indices;
    const long long sl = (long long)idx[k];
    dst[smp * dst_sample_stride + k * slice_bytes + b] =
        (sl >= 0 && sl < slices) ? data[smp * sample_bytes + sl * slice_bytes + b] : 0;
  }
}

// One workgroup per sample: out[b] = clip(scale(sum_k (L-lo)(R-ro); outP) + oo),
// libjit_matmul_i8 on each [M x K] x [K x N] pair of a batch of small matrices.
__global__ __launch_bounds__(kGlueThreads) void batch_matmul_i8_kernel(
    int8_t *__restrict__ out, const int8_t *__restrict__ lhs, const int8_t *__restrict__ rhs,
    int M, int K, int N, int32_t oo, int32_t lo, int32_t ro, int32_t pre, int32_t post,
    int32_t scale) {
  extern __shared__ int8_t sm[];
  int8_t *sl = sm, *sr = sm + (size_t)M * K;
  const long long b = blockIdx.x;
  const int8_t *L = lhs + b * (long long)M * K, *R = rhs + b * (long long)K * N;
  for (int i = threadIdx.x; i < M * K; i += kGlueThreads) sl[i] = L[i];
  for (int i = threadIdx.x; i < K * N; i += kGlueThreads) sr[i] = R[i];
  __syncthreads();
  int8_t *O = out + b * (long long)M * N;
  for (int e = threadIdx.x; e < M * N; e += kGlueThreads) {
    const int i = e / N, j = e - i * N;
    uint32_t acc = 0;
    for (int k = 0; k < K; k++)
      acc += (uint32_t)(((int32_t)sl[i * K + k] - lo) * ((int32_t)sr[k * N + j] - ro));
    O[e] = (int8_t)clip_i8(scale_i32((int32_t)acc, pre, post, scale, oo));
  }
}

// out[b] = clip(scale(sum_k (L[m][k]-lo)(R[n][k]-ro); outP) + oo) for a batch of
// small matrix pairs with BOTH operands K-contiguous (L [M x K], R [N x K]):
// libjit_matmul_i8 of L and the transpose of R. One wavefront per sample; each
// 32 x 32 block of the result is K/32 matrix-core instructions on raw bytes,
// the offsets enter through the row sums as in the large contraction kernel.
typedef int nt_v4i __attribute__((ext_vector_type(4)));
typedef int nt_v16i __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(kGlueThreads) void batch_matmul_nt_i8_kernel(
    int8_t *__restrict__ out, const int8_t *__restrict__ lhs, const int8_t *__restrict__ rhs,
    long long batch, int M, int K, int N, int32_t oo, int32_t lo, int32_t ro, int32_t pre,
    int32_t post, int32_t scale, const int32_t *__restrict__ dest_of, long long out_stride) {
  // dest_of (optional): where in the sample's output row element (m, n) goes,
  // negative = nowhere; without it the whole matrix is written
  const int lane = threadIdx.x & 63;
  const long long b = (long long)blockIdx.x * (kGlueThreads / 64) + (threadIdx.x >> 6);
  if (b >= batch) return;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int8_t *L = lhs + b * (long long)M * K, *R = rhs + b * (long long)N * K;
  int8_t *O = out + b * out_stride;
  const uint32_t kconst = (uint32_t)K * (uint32_t)lo * (uint32_t)ro;
  for (int tm = 0; tm < M; tm += 32) {
    for (int tn = 0; tn < N; tn += 32) {
      nt_v16i acc;
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = 0;
      int sa = 0, sb = 0;
      const bool a_ok = tm + l32 < M, b_ok = tn + l32 < N;
      const int8_t *ap = L + (long long)(a_ok ? tm + l32 : 0) * K + lhi * 16;
      const int8_t *bp = R + (long long)(b_ok ? tn + l32 : 0) * K + lhi * 16;
      for (int k0 = 0; k0 < K; k0 += 32) {
        // the upper half of the last slice is empty when K % 32 == 16
        const bool k_ok = k0 + lhi * 16 < K;
        nt_v4i a = {0, 0, 0, 0}, bb = {0, 0, 0, 0};
        if (a_ok && k_ok) a = *reinterpret_cast<const nt_v4i *>(ap + k0);
        if (b_ok && k_ok) bb = *reinterpret_cast<const nt_v4i *>(bp + k0);
#pragma unroll
        for (int q = 0; q < 4; q++) {
          sa = __builtin_amdgcn_sdot4(a[q], 0x01010101, sa, false);
          sb = __builtin_amdgcn_sdot4(bb[q], 0x01010101, sb, false);
        }
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bb, acc, 0, 0, 0);
      }
      sa += __shfl_xor(sa, 32, 64);
      sb += __shfl_xor(sb, 32, 64);
      // lane: column tn + l32; register r: row tm + 8*(r/4) + 4*lhi + r%4
      const uint32_t colc = kconst - (uint32_t)lo * (uint32_t)sb;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ml = (r >> 2) * 8 + lhi * 4 + (r & 3);
        const int row_sum = __shfl(sa, ml, 64);
        const uint32_t v = (uint32_t)acc[r] + colc - (uint32_t)ro * (uint32_t)row_sum;
        const int32_t y = clip_i8(scale_i32((int32_t)v, pre, post, scale, oo));
        if (tm + ml < M && b_ok) {
          const int at = (tm + ml) * N + tn + l32;
          const int to = dest_of ? dest_of[at] : at;
          if (to >= 0) O[to] = (int8_t)y;
        }
      }
    }
  }
}

// dst[n][bh][bw][(dh*2+dw)*C + c] = src[n][2bh+dh-padT][2bw+dw-padL][c]; positions
// outside the image and channels from 4C up hold `fill`. One thread per
// destination pixel.
__global__ __launch_bounds__(kGlueThreads) void space_to_depth2_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, int N, int IH, int IW, int C,
    int padT, int padL, int BH, int BW, int Cout, int fill, long long total) {
  const long long t = (long long)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t >= total) return;
  const int bw = (int)(t % BW);
  long long r = t / BW;
  const int bh = (int)(r % BH);
  const int n = (int)(r / BH);
  int8_t *d = dst + t * Cout;
  for (int q = 0; q < 4; q++) {
    const int ih = 2 * bh + (q >> 1) - padT, iw = 2 * bw + (q & 1) - padL;
    const bool in = ih >= 0 && ih < IH && iw >= 0 && iw < IW;
    const int8_t *p = src + (((long long)n * IH + (in ? ih : 0)) * IW + (in ? iw : 0)) * C;
    for (int c = 0; c < C; c++) d[q * C + c] = in ? p[c] : (int8_t)fill;
  }
  for (int c = 4 * C; c < Cout; c++) d[c] = (int8_t)fill;
}

// The same for 16 output channels (the 3-channel image stem): the 16 bytes of a
// block are put together in registers and leave in one store.
template <int C>
__global__ __launch_bounds__(kGlueThreads) void space_to_depth2_c16_i8_kernel(
    uint4 *__restrict__ dst, const int8_t *__restrict__ src, int N, int IH, int IW, int padT,
    int padL, int BH, int BW, int fill, long long total) {
  const long long t = (long long)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t >= total) return;
  const int bw = (int)(t % BW);
  long long r = t / BW;
  const int bh = (int)(r % BH);
  const int n = (int)(r / BH);
  uint8_t b[16];
#pragma unroll
  for (int i = 0; i < 16; i++) b[i] = (uint8_t)fill;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int ih = 2 * bh + (q >> 1) - padT, iw = 2 * bw + (q & 1) - padL;
    if (ih >= 0 && ih < IH && iw >= 0 && iw < IW) {
      const int8_t *p = src + (((long long)n * IH + ih) * IW + iw) * C;
#pragma unroll
      for (int c = 0; c < C; c++) b[q * C + c] = (uint8_t)p[c];
    }
  }
  uint32_t w[4];
#pragma unroll
  for (int j = 0; j < 4; j++)
    w[j] = (uint32_t)b[4 * j] | ((uint32_t)b[4 * j + 1] << 8) | ((uint32_t)b[4 * j + 2] << 16) |
           ((uint32_t)b[4 * j + 3] << 24);
  dst[t] = make_uint4(w[0], w[1], w[2], w[3]);
}

// Quantize (libjit_quantize_kernel: clip(nearbyintf(x / scale + offset)), every
// operation rounded on its own) and space-to-depth in one pass: the float
// image is read once and the int8 image in between is never written. The
// values are those of mi355x_quantize_i8 followed by mi355x_space_to_depth2_i8.
template <int C>
__global__ __launch_bounds__(kGlueThreads) void quantize_space_to_depth2_c16_kernel(
    uint4 *__restrict__ dst, const float *__restrict__ src, int N, int IH, int IW, int padT,
    int padL, int BH, int BW, int fill, float scale, float offset, long long total) {
  const long long t = (long long)blockIdx.x * kGlueThreads + threadIdx.x;
  if (t >= total) return;
  const int bw = (int)(t % BW);
  long long r = t / BW;
  const int bh = (int)(r % BH);
  const int n = (int)(r / BH);
  uint8_t b[16];
#pragma unroll
  for (int i = 0; i < 16; i++) b[i] = (uint8_t)fill;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int ih = 2 * bh + (q >> 1) - padT, iw = 2 * bw + (q & 1) - padL;
    if (ih >= 0 && ih < IH && iw >= 0 && iw < IW) {
      const float *p = src + (((long long)n * IH + ih) * IW + iw) * C;
#pragma unroll
      for (int c = 0; c < C; c++) {
        const float v = rintf(__fadd_rn(__fdiv_rn(p[c], scale), offset));
        b[q * C + c] = (uint8_t)clip_i8((int32_t)v);
      }
    }
  }
  uint32_t w[4];
#pragma unroll
  for (int j = 0; j < 4; j++)
    w[j] = (uint32_t)b[4 * j] | ((uint32_t)b[4 * j + 1] << 8) | ((uint32_t)b[4 * j + 2] << 16) |
           ((uint32_t)b[4 * j + 3] << 24);
  dst[t] = make_uint4(w[0], w[1], w[2], w[3]);
}

// libjit_sigmoid_kernel_f: 1 / (expf(-x) + 1)
__global__ __launch_bounds__(kGlueThreads) void sigmoid_f32_kernel(
    float *__restrict__ dst, const float *__restrict__ src, size_t n) {
  const size_t stride = (size_t)gridDim.x * kGlueThreads;
  for (size_t i = (size_t)blockIdx.x * kGlueThreads + threadIdx.x; i < n; i += stride)
    dst[i] = __fdiv_rn(1.0f, __fadd_rn(expf(-src[i]), 1.0f));
}

static unsigned capped_blocks(size_t work) {
  size_t b = (work + kGlueThreads - 1) / kGlueThreads;
  if (b > 256 * 64) b = 256 * 64;
  return (unsigned)(b ? b : 1);
}

static bool al16(const void *a, const void *b, const void *c) {
  return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) == 0;
}
static unsigned glue_blocks(size_t work) {
  size_t b = (work + kGlueThreads - 1) / kGlueThreads;
  return (unsigned)(b ? b : 1);
}
static bool shifts_ok(int32_t a, int32_t b) { return a >= 0 && a <= 31 && b >= 0 && b <= 31; }

static int pool_geom(PoolGeom &g, size_t N, size_t IH, size_t IW, size_t C, size_t OH,
                     size_t OW, size_t kH, size_t kW, size_t sH, size_t sW, size_t padT,
                     size_t padL) {
  MI355X_REQUIRE(IH > 0 && IW > 0 && C > 0 && kH > 0 && kW > 0 && sH > 0 && sW > 0,
                 "invalid pooling geometry");
  const size_t lim = 1u << 30;
  MI355X_REQUIRE(N < lim && IH < lim && IW < lim && C < lim && OH < lim && OW < lim &&
                     kH < lim && kW < lim && sH < lim && sW < lim && padT < lim && padL < lim,
                 "pooling dimensions too large");
  // every window must start at or before the last input row / column
  MI355X_REQUIRE(OH == 0 || (OH - 1) * sH < IH + padT, "output height inconsistent with input");
  MI355X_REQUIRE(OW == 0 || (OW - 1) * sW < IW + padL, "output width inconsistent with input");
  g = PoolGeom{(int)N, (int)IH, (int)IW, (int)C, (int)OH, (int)OW, (int)kH, (int)kW,
               (int)sH, (int)sW, (int)padT, (int)padL};
  return MI355X_OK;
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

int mi355x_add_i8(int8_t *dst, const int8_t *lhs, const int8_t *rhs, size_t n,
                  int32_t dest_offset, int32_t lhs_offset, int32_t rhs_offset,
                  int32_t lhs_pre, int32_t lhs_post, int32_t lhs_scale, int32_t rhs_pre,
                  int32_t rhs_post, int32_t rhs_scale, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && lhs && rhs, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(lhs_pre, lhs_post) && shifts_ok(rhs_pre, rhs_post),
                 "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(n / 16 / kGlueThreads < 0x7fffffffu, "tensor too large");
  AddParams p{dest_offset, lhs_offset, rhs_offset, lhs_pre, lhs_post, lhs_scale,
              rhs_pre, rhs_post, rhs_scale, 0, 0, 0, 0};
  const size_t chunks = al16(dst, lhs, rhs) ? n / 16 : 0;
  const bool small = fits24(lhs_scale) && fits24(rhs_scale) && off24(lhs_offset) &&
                     off24(rhs_offset);
  if (small)
    hipLaunchKernelGGL((add_i8_kernel<false, true>), dim3(glue_blocks(chunks)),
                       dim3(kGlueThreads), 0, as_stream(stream), dst, lhs, rhs, n, chunks, p);
  else
    hipLaunchKernelGGL((add_i8_kernel<false, false>), dim3(glue_blocks(chunks)),
                       dim3(kGlueThreads), 0, as_stream(stream), dst, lhs, rhs, n, chunks, p);
  return check_launch("add_i8");
}

int mi355x_add_relu_i8(int8_t *dst, const int8_t *lhs, const int8_t *rhs, size_t n,
                       int32_t sum_offset, int32_t lhs_offset, int32_t rhs_offset,
                       int32_t lhs_pre, int32_t lhs_post, int32_t lhs_scale, int32_t rhs_pre,
                       int32_t rhs_post, int32_t rhs_scale, int32_t dest_offset,
                       int32_t dest_pre, int32_t dest_post, int32_t dest_scale, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && lhs && rhs, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(lhs_pre, lhs_post) && shifts_ok(rhs_pre, rhs_post) &&
                     shifts_ok(dest_pre, dest_post),
                 "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(sum_offset >= -128 && sum_offset <= 127 && dest_offset >= -128 &&
                     dest_offset <= 127,
                 "offsets outside the int8 range");
  MI355X_REQUIRE(n / 16 / kGlueThreads < 0x7fffffffu, "tensor too large");
  AddParams p{sum_offset, lhs_offset, rhs_offset, lhs_pre, lhs_post, lhs_scale,
              rhs_pre, rhs_post, rhs_scale, dest_offset, dest_pre, dest_post, dest_scale};
  const size_t chunks = al16(dst, lhs, rhs) ? n / 16 : 0;
  const bool small = fits24(lhs_scale) && fits24(rhs_scale) && fits24(dest_scale) &&
                     off24(lhs_offset) && off24(rhs_offset);
  if (small)
    hipLaunchKernelGGL((add_i8_kernel<true, true>), dim3(glue_blocks(chunks)),
                       dim3(kGlueThreads), 0, as_stream(stream), dst, lhs, rhs, n, chunks, p);
  else
    hipLaunchKernelGGL((add_i8_kernel<true, false>), dim3(glue_blocks(chunks)),
                       dim3(kGlueThreads), 0, as_stream(stream), dst, lhs, rhs, n, chunks, p);
  return check_launch("add_relu_i8");
}

int mi355x_relu_i8(int8_t *dst, const int8_t *src, size_t n, int32_t src_offset,
                   int32_t dest_offset, int32_t dest_pre, int32_t dest_post,
                   int32_t dest_scale, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(dest_pre, dest_post), "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(src_offset >= -128 && src_offset <= 127 && dest_offset >= -128 &&
                     dest_offset <= 127,
                 "offsets outside the int8 range");
  MI355X_REQUIRE(n / 16 / kGlueThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = al16(dst, src, src) ? n / 16 : 0;
  hipLaunchKernelGGL(relu_i8_kernel, dim3(glue_blocks(chunks)), dim3(kGlueThreads), 0,
                     as_stream(stream), dst, src, n, chunks, src_offset, dest_offset, dest_pre,
                     dest_post, dest_scale);
  return check_launch("relu_i8");
}

int mi355x_clip_i8(int8_t *dst, const int8_t *src, size_t n, int32_t clip_min, int32_t clip_max,
                   int32_t src_offset, int32_t dest_offset, int32_t dest_pre, int32_t dest_post,
                   int32_t dest_scale, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(dest_pre, dest_post), "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(src_offset >= -128 && src_offset <= 127 && dest_offset >= -128 &&
                     dest_offset <= 127 && clip_min >= -128 && clip_min <= 127 &&
                     clip_max >= -128 && clip_max <= 127,
                 "offsets or clip bounds outside the int8 range");
  MI355X_REQUIRE(n / 16 / kGlueThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = al16(dst, src, src) ? n / 16 : 0;
  hipLaunchKernelGGL(clip_i8_kernel, dim3(glue_blocks(chunks)), dim3(kGlueThreads), 0,
                     as_stream(stream), dst, src, n, chunks, clip_min, clip_max, src_offset,
                     dest_offset, dest_pre, dest_post, dest_scale);
  return check_launch("clip_i8");
}

int mi355x_leaky_relu_i8(int8_t *dst, const int8_t *src, size_t n, int32_t src_offset,
                         int32_t dest_offset, int32_t pos_pre, int32_t pos_post,
                         int32_t pos_scale, int32_t neg_pre, int32_t neg_post, int32_t neg_scale,
                         void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(pos_pre, pos_post) && shifts_ok(neg_pre, neg_post),
                 "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(src_offset >= -128 && src_offset <= 127 && dest_offset >= -128 &&
                     dest_offset <= 127,
                 "offsets outside the int8 range");
  MI355X_REQUIRE(n / 16 / kGlueThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = al16(dst, src, src) ? n / 16 : 0;
  hipLaunchKernelGGL(leaky_relu_i8_kernel, dim3(glue_blocks(chunks)), dim3(kGlueThreads), 0,
                     as_stream(stream), dst, src, n, chunks, src_offset, dest_offset, pos_pre,
                     pos_post, pos_scale, neg_pre, neg_post, neg_scale);
  return check_launch("leaky_relu_i8");
}

int mi355x_max_splat_i8(int8_t *dst, const int8_t *src, size_t n, int32_t value, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(value >= -128 && value <= 127, "splat value outside the int8 range");
  MI355X_REQUIRE(n / 16 / kGlueThreads < 0x7fffffffu, "tensor too large");
  const size_t chunks = al16(dst, src, src) ? n / 16 : 0;
  hipLaunchKernelGGL(max_splat_i8_kernel, dim3(glue_blocks(chunks)), dim3(kGlueThreads), 0,
                     as_stream(stream), dst, src, n, chunks, value);
  return check_launch("max_splat_i8");
}

int mi355x_batched_add_i8(int8_t *dst, const int8_t *batch, const void *slice, int slice_is_i32,
                          size_t num_slices, size_t slice_size, int32_t dest_offset,
                          int32_t batch_offset, int32_t slice_offset, int32_t batch_pre,
                          int32_t batch_post, int32_t batch_scale, int32_t slice_pre,
                          int32_t slice_post, int32_t slice_scale, void *stream) {
  if (num_slices == 0 || slice_size == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && batch && slice, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(batch_pre, batch_post) && shifts_ok(slice_pre, slice_post),
                 "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(num_slices < (1ull << 40) / slice_size, "tensor too large");
  const size_t total = num_slices * slice_size;
  const int vec4 = slice_size % 4 == 0 && ((((uintptr_t)dst) | ((uintptr_t)batch)) & 3) == 0;
  const size_t work = vec4 ? total / 4 : total;
  const size_t blocks = (work + kGlueThreads - 1) / kGlueThreads;
  const dim3 grid((unsigned)(blocks < 65536 * 4 ? (blocks ? blocks : 1) : 65536 * 4));
  if (slice_is_i32)
    hipLaunchKernelGGL((batched_add_i8_kernel<int32_t>), grid, dim3(kGlueThreads), 0,
                       as_stream(stream), dst, batch, (const int32_t *)slice, total, slice_size,
                       vec4, dest_offset, batch_offset, slice_offset, batch_pre, batch_post,
                       batch_scale, slice_pre, slice_post, slice_scale);
  else
    hipLaunchKernelGGL((batched_add_i8_kernel<int8_t>), grid, dim3(kGlueThreads), 0,
                       as_stream(stream), dst, batch, (const int8_t *)slice, total, slice_size,
                       vec4, dest_offset, batch_offset, slice_offset, batch_pre, batch_post,
                       batch_scale, slice_pre, slice_post, slice_scale);
  return check_launch("batched_add_i8");
}

int mi355x_max_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH, size_t IW, size_t C,
                       size_t OH, size_t OW, size_t kH, size_t kW, size_t sH, size_t sW,
                       size_t padT, size_t padL, int32_t out_offset, void *stream) {
  if (N == 0 || OH == 0 || OW == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in, "NULL tensor");
  PoolGeom g;
  int rc = pool_geom(g, N, IH, IW, C, OH, OW, kH, kW, sH, sW, padT, padL);
  if (rc != MI355X_OK) return rc;
  const bool vec = (C % 16 == 0) && al16(out, in, in);
  const long long total = (long long)N * OH * OW * (vec ? C / 16 : C);
  MI355X_REQUIRE(total / kGlueThreads < 0x7fffffffLL, "tensor too large");
  // taps read per group: the whole window when it has at most 9 taps
  const bool small = kH * kW <= 4, mid = kH * kW <= 9;
#define MI355X_MAX_POOL(VEC, U)                                                              \
  hipLaunchKernelGGL((max_pool_i8_kernel<VEC, U>), dim3(glue_blocks((size_t)total)),          \
                     dim3(kGlueThreads), 0, as_stream(stream), out, in, g, out_offset, total)
  if (vec) {
    if (small) MI355X_MAX_POOL(16, 4);
    else if (mid) MI355X_MAX_POOL(16, 9);
    else MI355X_MAX_POOL(16, 8);
  } else {
    if (small) MI355X_MAX_POOL(1, 4);
    else if (mid) MI355X_MAX_POOL(1, 9);
    else MI355X_MAX_POOL(1, 8);
  }
#undef MI355X_MAX_POOL
  return check_launch("max_pool_i8");
}

int mi355x_avg_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH, size_t IW, size_t C,
                       size_t OH, size_t OW, size_t kH, size_t kW, size_t sH, size_t sW,
                       size_t padT, size_t padL, int count_include_pads, int32_t out_offset,
                       int32_t in_offset, int32_t out_pre, int32_t out_post, int32_t out_scale,
                       void *stream) {
  if (N == 0 || OH == 0 || OW == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(out_pre, out_post), "pre/post shift outside [0, 31]");
  PoolGeom g;
  int rc = pool_geom(g, N, IH, IW, C, OH, OW, kH, kW, sH, sW, padT, padL);
  if (rc != MI355X_OK) return rc;
  const bool vec = (C % 4 == 0) && ((((uintptr_t)out | (uintptr_t)in) & 3) == 0);
  const long long total = (long long)N * OH * OW * (vec ? C / 4 : C);
  MI355X_REQUIRE(total / kGlueThreads < 0x7fffffffLL, "tensor too large");
  const bool small = kH * kW <= 4, mid = kH * kW <= 9;
#define MI355X_AVG_POOL(VEC, U)                                                              \
  hipLaunchKernelGGL((avg_pool_i8_kernel<VEC, U>), dim3(glue_blocks((size_t)total)),          \
                     dim3(kGlueThreads), 0, as_stream(stream), out, in, g, count_include_pads, \
                     out_offset, in_offset, out_pre, out_post, out_scale, total)
  if (vec) {
    if (small) MI355X_AVG_POOL(4, 4);
    else if (mid) MI355X_AVG_POOL(4, 9);
    else MI355X_AVG_POOL(4, 16);
  } else {
    if (small) MI355X_AVG_POOL(1, 4);
    else if (mid) MI355X_AVG_POOL(1, 9);
    else MI355X_AVG_POOL(1, 16);
  }
#undef MI355X_AVG_POOL
  return check_launch("avg_pool_i8");
}

int mi355x_convert_f16_to_f32(float *dst, const void *src, size_t n, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  hipLaunchKernelGGL(convert_f16_f32_kernel, dim3(capped_blocks(n)), dim3(kGlueThreads), 0,
                     as_stream(stream), dst, (const __half *)src, n);
  return check_launch("convert_f16_to_f32");
}

int mi355x_insert_rows(void *dst, const void *src, size_t rows, size_t row_bytes,
                       size_t dst_row_stride, size_t dst_offset, void *stream) {
  if (rows == 0 || row_bytes == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(dst_offset + row_bytes <= dst_row_stride,
                 "slice of %zu bytes at offset %zu does not fit rows of %zu bytes", row_bytes,
                 dst_offset, dst_row_stride);
  MI355X_REQUIRE(rows < (1ull << 40) && dst_row_stride < (1ull << 40), "tensor too large");
  const uintptr_t all = (uintptr_t)dst | (uintptr_t)src | row_bytes | dst_row_stride | dst_offset;
  const int unit = (all % 16 == 0) ? 16 : (all % 4 == 0) ? 4 : 1;
  hipLaunchKernelGGL(insert_rows_kernel, dim3(capped_blocks(rows * (row_bytes / unit))),
                     dim3(kGlueThreads), 0, as_stream(stream), (uint8_t *)dst,
                     (const uint8_t *)src, (long long)rows, (long long)row_bytes,
                     (long long)dst_row_stride, (long long)dst_offset, unit);
  return check_launch("insert_rows");
}

int mi355x_batch_transpose_i8(int8_t *dst, const int8_t *src, size_t batch, size_t rows,
                              size_t cols, void *stream) {
  if (batch == 0 || rows == 0 || cols == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(rows < (1u << 15) && cols < (1u << 15) && batch < (1ull << 32),
                 "matrices too large");
  hipLaunchKernelGGL(batch_transpose_i8_kernel, dim3(capped_blocks(batch * rows * cols)),
                     dim3(kGlueThreads), 0, as_stream(stream), dst, src, (long long)batch,
                     (int)rows, (int)cols);
  return check_launch("batch_transpose_i8");
}

int mi355x_gather_rows(void *dst, const void *data, const void *indices, int idx_is_64,
                       size_t num_indices, size_t slice_bytes, size_t num_samples,
                       size_t sample_bytes, size_t dst_sample_stride, void *stream) {
  if (num_indices == 0 || slice_bytes == 0 || num_samples == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && data && indices, "NULL tensor");
  MI355X_REQUIRE(sample_bytes % slice_bytes == 0, "sample is not a whole number of slices");
  MI355X_REQUIRE(num_indices < (1ull << 32) && slice_bytes < (1ull << 32) &&
                     num_samples < (1ull << 32) && sample_bytes < (1ull << 40) &&
                     dst_sample_stride < (1ull << 40),
                 "tensor too large");
  MI355X_REQUIRE(dst_sample_stride >= num_indices * slice_bytes,
                 "gathered samples of %zu bytes overlap at a stride of %zu",
                 num_indices * slice_bytes, dst_sample_stride);
  const size_t total = num_samples * num_indices * slice_bytes;
  if (idx_is_64)
    hipLaunchKernelGGL(gather_kernel<long long>, dim3(capped_blocks(total)), dim3(kGlueThreads), 0,
                       as_stream(stream), (uint8_t *)dst, (const uint8_t *)data,
                       (const long long *)indices, (long long)num_indices, (long long)slice_bytes,
                       (long long)num_samples, (long long)sample_bytes,
                       (long long)dst_sample_stride);
  else
    hipLaunchKernelGGL(gather_kernel<int>, dim3(capped_blocks(total)), dim3(kGlueThreads), 0,
                       as_stream(stream), (uint8_t *)dst, (const uint8_t *)data,
                       (const int *)indices, (long long)num_indices, (long long)slice_bytes,
                       (long long)num_samples, (long long)sample_bytes,
                       (long long)dst_sample_stride);
  return check_launch("gather");
}

int mi355x_gather(void *dst, const void *data, const void *indices, int idx_is_64,
                  size_t num_indices, size_t slice_bytes, size_t num_samples,
                  size_t sample_bytes, void *stream) {
  return mi355x_gather_rows(dst, data, indices, idx_is_64, num_indices, slice_bytes, num_samples,
                            sample_bytes, num_indices * slice_bytes, stream);
}

int mi355x_batch_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs, size_t batch,
                           size_t M, size_t K, size_t N, int32_t out_offset, int32_t lhs_offset,
                           int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                           int32_t out_scale, void *stream) {
  if (batch == 0 || M == 0 || N == 0) return MI355X_OK;
  MI355X_REQUIRE(out && lhs && rhs, "NULL tensor");
  MI355X_REQUIRE(shifts_ok(out_pre, out_post), "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(batch < 0x7fffffffu, "batch too large");
  const size_t lds = (M + N) * K;
  MI355X_REQUIRE(lds <= 64 * 1024 && M * N < (1u << 24),
                 "matrices of %zu x %zu x %zu do not fit the small-matrix kernel (use "
                 "mi355x_matmul_i8 per sample)", M, K, N);
  hipLaunchKernelGGL(batch_matmul_i8_kernel, dim3((unsigned)batch), dim3(kGlueThreads), lds,
                     as_stream(stream), out, lhs, rhs, (int)M, (int)K, (int)N, out_offset,
                     lhs_offset, rhs_offset, out_pre, out_post, out_scale);
  return check_launch("batch_matmul_i8");
}

int mi355x_batch_matmul_nt_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_nk, size_t batch,
                              size_t M, size_t K, size_t N, int32_t out_offset,
                              int32_t lhs_offset, int32_t rhs_offset, int32_t out_pre,
                              int32_t out_post, int32_t out_scale, void *stream) {
  return mi355x_batch_matmul_nt_select_i8(out, lhs, rhs_nk, batch, M, K, N, out_offset, lhs_offset,
                                          rhs_offset, out_pre, out_post, out_scale, nullptr, M * N,
                                          stream);
}

int mi355x_batch_matmul_nt_select_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_nk,
                                     size_t batch, size_t M, size_t K, size_t N,
                                     int32_t out_offset, int32_t lhs_offset, int32_t rhs_offset,
                                     int32_t out_pre, int32_t out_post, int32_t out_scale,
                                     const int32_t *dest_of, size_t out_sample_stride,
                                     void *stream) {
  if (batch == 0 || M == 0 || N == 0) return MI355X_OK;
  MI355X_REQUIRE(out && lhs && rhs_nk, "NULL tensor");
  MI355X_REQUIRE(out_sample_stride < (1ull << 40), "output stride too large");
  MI355X_REQUIRE(dest_of || out_sample_stride >= M * N, "output samples overlap");
  MI355X_REQUIRE(shift_ok(out_pre) && shift_ok(out_post), "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(K > 0 && K % 16 == 0 && K < (1u << 20) && M < (1u << 15) && N < (1u << 15),
                 "needs K %% 16 == 0 and matrices below 32768 rows (K = %zu)", K);
  MI355X_REQUIRE((((uintptr_t)lhs | (uintptr_t)rhs_nk) & 15) == 0, "operands must be 16-byte aligned");
  MI355X_REQUIRE(batch < (1ull << 31), "batch too large");
  const size_t per_block = kGlueThreads / 64;
  hipLaunchKernelGGL(batch_matmul_nt_i8_kernel, dim3((unsigned)((batch + per_block - 1) / per_block)),
                     dim3(kGlueThreads), 0, as_stream(stream), out, lhs, rhs_nk, (long long)batch,
                     (int)M, (int)K, (int)N, out_offset, lhs_offset, rhs_offset, out_pre, out_post,
                     out_scale, dest_of, (long long)out_sample_stride);
  return check_launch("batch_matmul_nt_i8");
}

int mi355x_space_to_depth2_i8(int8_t *dst, const int8_t *src, size_t N, size_t IH, size_t IW,
                              size_t C, size_t padT, size_t padL, size_t BH, size_t BW,
                              size_t Cout, int32_t fill, void *stream) {
  if (N == 0 || BH == 0 || BW == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(C > 0 && Cout >= 4 * C && Cout < 4096, "needs 4*C <= Cout < 4096");
  const size_t lim = 1u << 30;
  MI355X_REQUIRE(N < lim && IH < lim && IW < lim && BH < lim && BW < lim && padT < lim && padL < lim,
                 "dimensions too large");
  MI355X_REQUIRE(fill >= -128 && fill <= 127, "fill outside the int8 range");
  const long long total = (long long)N * BH * BW;
  MI355X_REQUIRE(total / kGlueThreads < 0x7fffffffLL, "tensor too large");
  if (Cout == 16 && (C == 3 || C == 4) && (((uintptr_t)dst) & 15) == 0) {
    auto kern = C == 3 ? space_to_depth2_c16_i8_kernel<3> : space_to_depth2_c16_i8_kernel<4>;
    hipLaunchKernelGGL(kern, dim3(glue_blocks((size_t)total)), dim3(kGlueThreads), 0,
                       as_stream(stream), (uint4 *)dst, src, (int)N, (int)IH, (int)IW, (int)padT,
                       (int)padL, (int)BH, (int)BW, fill, total);
    return check_launch("space_to_depth2_i8");
  }
  hipLaunchKernelGGL(space_to_depth2_i8_kernel, dim3(glue_blocks((size_t)total)),
                     dim3(kGlueThreads), 0, as_stream(stream), dst, src, (int)N, (int)IH, (int)IW,
                     (int)C, (int)padT, (int)padL, (int)BH, (int)BW, (int)Cout, fill, total);
  return check_launch("space_to_depth2_i8");
}

int mi355x_quantize_space_to_depth2_i8(int8_t *dst, const float *src, size_t N, size_t IH,
                                       size_t IW, size_t C, size_t padT, size_t padL, size_t BH,
                                       size_t BW, size_t Cout, int32_t fill, float scale,
                                       int32_t offset, void *stream) {
  if (N == 0 || BH == 0 || BW == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE((C == 3 || C == 4) && Cout == 16, "3 or 4 channels into 16 only");
  MI355X_REQUIRE((((uintptr_t)dst) & 15) == 0 && (((uintptr_t)src) & 3) == 0, "unaligned tensor");
  const size_t lim = 1u << 30;
  MI355X_REQUIRE(N < lim && IH < lim && IW < lim && BH < lim && BW < lim && padT < lim && padL < lim,
                 "dimensions too large");
  MI355X_REQUIRE(fill >= -128 && fill <= 127, "fill outside the int8 range");
  const long long total = (long long)N * BH * BW;
  MI355X_REQUIRE(total / kGlueThreads < 0x7fffffffLL, "tensor too large");
  auto kern = C == 3 ? quantize_space_to_depth2_c16_kernel<3> : quantize_space_to_depth2_c16_kernel<4>;
  hipLaunchKernelGGL(kern, dim3(glue_blocks((size_t)total)), dim3(kGlueThreads), 0,
                     as_stream(stream), (uint4 *)dst, src, (int)N, (int)IH, (int)IW, (int)padT,
                     (int)padL, (int)BH, (int)BW, fill, scale, (float)offset, total);
  return check_launch("quantize_space_to_depth2_i8");
}

int mi355x_sigmoid_f32(float *dst, const float *src, size_t n, void *stream) {
  if (n == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  hipLaunchKernelGGL(sigmoid_f32_kernel, dim3(capped_blocks(n)), dim3(kGlueThreads), 0,
                     as_stream(stream), dst, src, n);
  return check_launch("sigmoid_f32");
}

int mi355x_softmax_f32(float *out, const float *in, size_t rows, size_t cols, void *stream) {
  if (rows == 0 || cols == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in, "NULL tensor");
  MI355X_REQUIRE(rows < 0x7fffffffu && cols < 0x7fffffffu, "tensor too large");
  hipLaunchKernelGGL(softmax_f32_kernel<false>, dim3((unsigned)rows), dim3(kGlueThreads), 0,
                     as_stream(stream), out, (const void *)in, (int)cols, 1.0f, 0);
  return check_launch("softmax_f32");
}

int mi355x_dequantize_softmax(float *out, const int8_t *in, size_t rows, size_t cols, float scale,
                              int32_t offset, void *stream) {
  if (rows == 0 || cols == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in, "NULL tensor");
  MI355X_REQUIRE(rows < 0x7fffffffu && cols < 0x7fffffffu, "tensor too large");
  hipLaunchKernelGGL(softmax_f32_kernel<true>, dim3((unsigned)rows), dim3(kGlueThreads), 0,
                     as_stream(stream), out, (const void *)in, (int)cols, scale, offset);
  return check_launch("dequantize_softmax");
}

} // extern "C"
