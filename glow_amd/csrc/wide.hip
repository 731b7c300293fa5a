// The rest of the CPU backend's quantized kernel set, off the hot path but part
// of the same operator family: Quantize / Dequantize / RescaleQuantized for
// int16 and int32 tensors (reference
// lib/LLVMIRCodeGen/libjit/libjit.cpp:3004-3056), Transpose of up to six
// dimensions (libjit.cpp:565-653, 3162-3184) and the channelwise quantized 3-D
// convolution (lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:244-349, 564-596).
// They are plain HBM-bound kernels: coalesced stores, one output element (or
// four) per lane, no staging.
#include "common.h"

// Every multiply and add below must round on its own (the CPU code this
// reproduces has no fused multiply-add).
#pragma clang fp contract(off)
#include "requant.h"

namespace mi355x {

constexpr int kWideThreads = 256;

__device__ __forceinline__ int32_t clip_i16(int32_t v) {
  return min(max(v, -32768), 32767);
}

// libjit_scale<int64_t>: the arithmetic runs in 64 bits, the result is
// truncated to 32.
__device__ __forceinline__ int32_t scale_i64(int64_t in, int32_t pre, int32_t post,
                                             int32_t scale, int32_t offset) {
  const int64_t rtn = post > 0 ? (int64_t)(1 << (post - 1)) : 0;
  const int64_t v = ((((in >> pre) * (int64_t)scale) + rtn) >> post) + (int64_t)offset;
  return (int32_t)(uint32_t)(uint64_t)v;
}

template <class T>
__global__ __launch_bounds__(kWideThreads) void quantize_wide_kernel(T *__restrict__ dst,
                                                                    const float *__restrict__ src,
                                                                    size_t n, float scale,
                                                                    float offset) {
  const size_t stride = (size_t)gridDim.x * kWideThreads;
  for (size_t i = (size_t)blockIdx.x * kWideThreads + threadIdx.x; i < n; i += stride) {
    // the conversion saturates where the CPU's is undefined (|v| >= 2^31)
    const int32_t v = (int32_t)rintf(__fadd_rn(__fdiv_rn(src[i], scale), offset));
    dst[i] = sizeof(T) == 2 ? (T)clip_i16(v) : (T)v;
  }
}

template <class T>
__global__ __launch_bounds__(kWideThreads) void dequantize_wide_kernel(float *__restrict__ dst,
                                                                      const T *__restrict__ src,
                                                                      size_t n, float scale,
                                                                      int32_t offset) {
  const size_t stride = (size_t)gridDim.x * kWideThreads;
  for (size_t i = (size_t)blockIdx.x * kWideThreads + threadIdx.x; i < n; i += stride)
    dst[i] = __fmul_rn(scale, (float)(int32_t)((uint32_t)(int32_t)src[i] - (uint32_t)offset));
}

template <class T>
__global__ __launch_bounds__(kWideThreads) void rescale_wide_kernel(T *__restrict__ dst,
                                                                   const T *__restrict__ src,
                                                                   size_t n, int32_t out_offset,
                                                                   int32_t in_offset, int32_t pre,
                                                                   int32_t post, int32_t scale) {
  const size_t stride = (size_t)gridDim.x * kWideThreads;
  for (size_t i = (size_t)blockIdx.x * kWideThreads + threadIdx.x; i < n; i += stride) {
    // in - in_offset is 32-bit arithmetic, then widened
    const int32_t d = (int32_t)((uint32_t)(int32_t)src[i] - (uint32_t)in_offset);
    const int32_t s = scale_i64((int64_t)d, pre, post, scale, out_offset);
    dst[i] = sizeof(T) == 2 ? (T)clip_i16(s) : (T)s;
  }
}

static unsigned wide_grid(size_t n) {
  const size_t blocks = (n + kWideThreads - 1) / kWideThreads;
  return (unsigned)(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

// ---- Transpose ----------------------------------------------------------------

struct TransposePlan {
  unsigned long long odim[6];     // output extents
  unsigned long long istride[6];  // input stride (elements) of the source dimension of output dim d
  int nd;
};

template <class T>
__global__ __launch_bounds__(kWideThreads) void transpose_nd_kernel(T *__restrict__ dst,
                                                                   const T *__restrict__ src,
                                                                   size_t total, TransposePlan p) {
  const size_t stride = (size_t)gridDim.x * kWideThreads;
  for (size_t o = (size_t)blockIdx.x * kWideThreads + threadIdx.x; o < total; o += stride) {
    size_t rest = o, from = 0;
#pragma unroll
    for (int d = 5; d >= 0; d--) {
      if (d < p.nd) {
        const size_t c = rest % p.odim[d];
        rest /= p.odim[d];
        from += c * p.istride[d];
      }
    }
    dst[o] = src[from];
  }
}

// ---- 3-D channelwise quantized convolution --------------------------------------

struct Conv3dArgs {
  int8_t *out;
  const int8_t *in, *filter;
  const void *bias;
  int bias_is_i8;
  mi355x_conv3d_geom g;
  int32_t out_offset, in_offset;
  const int32_t *f_off, *b_off, *b_pre, *b_post, *b_scale, *o_pre, *o_post, *o_scale;
  int32_t act, a0, a1, a2;
};

// One output element per lane, output channels fastest: the lanes of a wave
// read the same input bytes (one request) and neighbouring filter rows.
__global__ __launch_bounds__(kWideThreads) void cwq_conv3d_kernel(Conv3dArgs a, size_t total) {
  const mi355x_conv3d_geom &g = a.g;
  const int icg = g.IC / g.group, ocg = g.OC / g.group;
  const size_t stride = (size_t)gridDim.x * kWideThreads;
  for (size_t o = (size_t)blockIdx.x * kWideThreads + threadIdx.x; o < total; o += stride) {
    size_t rest = o;
    const int d = (int)(rest % (size_t)g.OC); rest /= (size_t)g.OC;
    const int ay = (int)(rest % (size_t)g.OW); rest /= (size_t)g.OW;
    const int ax = (int)(rest % (size_t)g.OH); rest /= (size_t)g.OH;
    const int at = (int)(rest % (size_t)g.OT); rest /= (size_t)g.OT;
    const size_t n = rest;
    const int grp = d / ocg;
    const int32_t f_off = a.f_off[d];
    const int32_t b = a.bias_is_i8 ? (int32_t) reinterpret_cast<const int8_t *>(a.bias)[d]
                                   : reinterpret_cast<const int32_t *>(a.bias)[d];
    uint32_t sum = (uint32_t)scale_i32((int32_t)((uint32_t)b - (uint32_t)a.b_off[d]), a.b_pre[d],
                                       a.b_post[d], a.b_scale[d], 0);
    const int8_t *frow = a.filter + (size_t)d * g.KT * g.KH * g.KW * icg;
    for (int ft = 0; ft < g.KT; ft++) {
      const int it = at * g.strideT + ft - g.padN;
      if (it < 0 || it >= g.IT) continue;
      for (int fx = 0; fx < g.KH; fx++) {
        const int ih = ax * g.strideH + fx - g.padT;
        if (ih < 0 || ih >= g.IH) continue;
        for (int fy = 0; fy < g.KW; fy++) {
          const int iw = ay * g.strideW + fy - g.padL;
          if (iw < 0 || iw >= g.IW) continue;
          const int8_t *ip = a.in + ((((n * g.IT + it) * g.IH + ih) * g.IW + iw) * (size_t)g.IC +
                                     (size_t)grp * icg);
          const int8_t *fp = frow + (((size_t)ft * g.KH + fx) * g.KW + fy) * icg;
          for (int c = 0; c < icg; c++)
            sum += (uint32_t)((int32_t)fp[c] - f_off) * (uint32_t)((int32_t)ip[c] - a.in_offset);
        }
      }
    }
    int32_t v = scale_i32((int32_t)sum, a.o_pre[d], a.o_post[d], a.o_scale[d], a.out_offset);
    v = activation_i32(v, a.out_offset, a.act, a.a0, a.a1, a.a2);
    a.out[o] = (int8_t)clip_i8(v);
  }
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

#define MI355X_WIDE_ENTRY(NAME, T)                                                            \
  int mi355x_quantize_##NAME(T *dst, const float *src, size_t n, float scale, int32_t offset, \
                             void *stream) {                                                  \
    if (n == 0) return MI355X_OK;                                                             \
    MI355X_REQUIRE(dst && src, "NULL tensor");                                                \
    hipLaunchKernelGGL(quantize_wide_kernel<T>, dim3(wide_grid(n)), dim3(kWideThreads), 0,    \
                       as_stream(stream), dst, src, n, scale, (float)offset);                 \
    return check_launch("quantize_" #NAME);                                                   \
  }                                                                                           \
  int mi355x_dequantize_##NAME(float *dst, const T *src, size_t n, float scale,               \
                               int32_t offset, void *stream) {                                \
    if (n == 0) return MI355X_OK;                                                             \
    MI355X_REQUIRE(dst && src, "NULL tensor");                                                \
    hipLaunchKernelGGL(dequantize_wide_kernel<T>, dim3(wide_grid(n)), dim3(kWideThreads), 0,  \
                       as_stream(stream), dst, src, n, scale, offset);                        \
    return check_launch("dequantize_" #NAME);                                                 \
  }                                                                                           \
  int mi355x_rescale_##NAME(T *dst, const T *src, size_t n, int32_t out_offset,               \
                            int32_t in_offset, int32_t pre, int32_t post, int32_t scale,      \
                            void *stream) {                                                   \
    if (n == 0) return MI355X_OK;                                                             \
    MI355X_REQUIRE(dst && src, "NULL tensor");                                                \
    MI355X_REQUIRE(shift_ok(pre) && shift_ok(post), "shift outside [0, 31]");                 \
    hipLaunchKernelGGL(rescale_wide_kernel<T>, dim3(wide_grid(n)), dim3(kWideThreads), 0,     \
                       as_stream(stream), dst, src, n, out_offset, in_offset, pre, post,      \
                       scale);                                                                \
    return check_launch("rescale_" #NAME);                                                    \
  }

MI355X_WIDE_ENTRY(i16, int16_t)
MI355X_WIDE_ENTRY(i32, int32_t)
#undef MI355X_WIDE_ENTRY

int mi355x_transpose_nd(void *dst, const void *src, const size_t *in_dims, const size_t *shuffle,
                        size_t num_dims, size_t elem_size, void *stream) {
  MI355X_REQUIRE(num_dims >= 1 && num_dims <= 6, "%zu dimensions: 1 to 6 are supported", num_dims);
  MI355X_REQUIRE(in_dims && shuffle, "NULL dims or shuffle");
  MI355X_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4 || elem_size == 8,
                 "element size %zu", elem_size);
  size_t istride[6], total = 1;
  unsigned seen = 0;
  for (size_t d = num_dims; d-- > 0;) {
    istride[d] = total;
    total *= in_dims[d];
  }
  TransposePlan p{};
  p.nd = (int)num_dims;
  for (size_t d = 0; d < num_dims; d++) {
    MI355X_REQUIRE(shuffle[d] < num_dims && !(seen & (1u << shuffle[d])),
                   "shuffle is not a permutation");
    seen |= 1u << shuffle[d];
    p.odim[d] = in_dims[shuffle[d]];
    p.istride[d] = istride[shuffle[d]];
  }
  if (total == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  hipStream_t st = as_stream(stream);
  const dim3 grid(wide_grid(total)), block(kWideThreads);
  switch (elem_size) {
  case 1:
    hipLaunchKernelGGL(transpose_nd_kernel<uint8_t>, grid, block, 0, st, (uint8_t *)dst,
                       (const uint8_t *)src, total, p);
    break;
  case 2:
    hipLaunchKernelGGL(transpose_nd_kernel<uint16_t>, grid, block, 0, st, (uint16_t *)dst,
                       (const uint16_t *)src, total, p);
    break;
  case 4:
    hipLaunchKernelGGL(transpose_nd_kernel<uint32_t>, grid, block, 0, st, (uint32_t *)dst,
                       (const uint32_t *)src, total, p);
    break;
  default:
    hipLaunchKernelGGL(transpose_nd_kernel<uint64_t>, grid, block, 0, st, (uint64_t *)dst,
                       (const uint64_t *)src, total, p);
    break;
  }
  return check_launch("transpose_nd");
}

int mi355x_cwq_conv3d_i8(int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
                         int bias_is_i8, const mi355x_conv3d_geom *g, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type, const int32_t *act_args,
                         void *stream) {
  MI355X_REQUIRE(g, "geometry is NULL");
  MI355X_REQUIRE(g->N >= 0 && g->IT > 0 && g->IH > 0 && g->IW > 0 && g->IC > 0 && g->OC > 0 &&
                     g->KT > 0 && g->KH > 0 && g->KW > 0 && g->strideT > 0 && g->strideH > 0 &&
                     g->strideW > 0 && g->padN >= 0 && g->padT >= 0 && g->padL >= 0 &&
                     g->group > 0 && g->IC % g->group == 0 && g->OC % g->group == 0 &&
                     g->OT >= 0 && g->OH >= 0 && g->OW >= 0,
                 "malformed 3-D convolution geometry");
  // every tap the output extents ask for must start inside the padded input
  MI355X_REQUIRE((g->OT == 0 || (long long)(g->OT - 1) * g->strideT - g->padN < g->IT) &&
                     (g->OH == 0 || (long long)(g->OH - 1) * g->strideH - g->padT < g->IH) &&
                     (g->OW == 0 || (long long)(g->OW - 1) * g->strideW - g->padL < g->IW),
                 "output extents do not fit the input");
  MI355X_REQUIRE(act_type == MI355X_ACT_NONE || act_type == MI355X_ACT_RELU ||
                     act_type == MI355X_ACT_CLIP || act_type == MI355X_ACT_LEAKY_RELU,
                 "fused activation %d is not defined for quantized convolutions", act_type);
  MI355X_REQUIRE(act_type == MI355X_ACT_NONE || act_type == MI355X_ACT_RELU || act_args,
                 "act_args is NULL");
  const size_t total = (size_t)g->N * g->OT * g->OH * g->OW * g->OC;
  if (total == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in && filter && bias && filter_offsets && bias_offsets && bias_pre &&
                     bias_post && bias_scale && out_pre && out_post && out_scale,
                 "NULL tensor");
  Conv3dArgs a;
  a.out = out; a.in = in; a.filter = filter; a.bias = bias; a.bias_is_i8 = bias_is_i8;
  a.g = *g;
  a.out_offset = out_offset; a.in_offset = in_offset;
  a.f_off = filter_offsets; a.b_off = bias_offsets; a.b_pre = bias_pre; a.b_post = bias_post;
  a.b_scale = bias_scale; a.o_pre = out_pre; a.o_post = out_post; a.o_scale = out_scale;
  a.act = act_type;
  a.a0 = act_args ? act_args[0] : 0;
  a.a1 = act_args ? act_args[1] : 0;
  a.a2 = act_args ? act_args[2] : 0;
  if (act_type == MI355X_ACT_LEAKY_RELU)
    MI355X_REQUIRE(shift_ok(a.a0) && shift_ok(a.a1), "LeakyRelu shift outside [0, 31]");
  hipLaunchKernelGGL(cwq_conv3d_kernel, dim3(wide_grid(total)), dim3(kWideThreads), 0,
                     as_stream(stream), a, total);
  return check_launch("cwq_conv3d_i8");
}

} // extern "C"
