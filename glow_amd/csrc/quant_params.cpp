// Host-side quantization parameter math the backend needs at compile time:
// the float -> {pre, post, scale} conversion behind every integer rescale,
// range -> (scale, zero point) selection, and the rowwise / fused-rowwise
// weight packers. Results must equal what Glow's own code produces, since the
// kernels only reproduce the CPU backend bit for bit when they are fed the
// same integers (reference lib/Quantization/Base/Base.cpp:234-565,
// include/glow/Quantization/Base/Base.h:323-678).
#include "common.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>

namespace {

struct Range {
  int64_t lo, hi;
};

// Base.cpp:361-403. Int32 is deliberately narrowed to 30 bits there.
bool quantized_range(int qty, Range &r) {
  switch (qty) {
  case MI355X_QTY_INT8: r = {-128, 127}; return true;
  case MI355X_QTY_UINT8: r = {0, 255}; return true;
  case MI355X_QTY_INT16: r = {-32768, 32767}; return true;
  case MI355X_QTY_INT32:
    r = {(int64_t)std::numeric_limits<int32_t>::min() >> 2,
         (int64_t)std::numeric_limits<int32_t>::max() >> 2};
    return true;
  default: return false;
  }
}

// IEEE binary32 -> binary16 bits with round-to-nearest-even (the behaviour of
// fp16_ieee_from_fp32_value, which glow::float16 wraps).
uint16_t to_half_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, sizeof(x));
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) return sign | 0x7e00u;          // NaN
  if (x >= 0x477ff000u) return sign | 0x7c00u;         // overflow -> inf
  if (x < 0x38800000u) {                               // below 2^-14: subnormal
    // value * 2^24 rounded to an integer with RNE, done in double (exact)
    float a;
    std::memcpy(&a, &x, sizeof(a));
    const double scaled = (double)a * 16777216.0;
    const double r = std::nearbyint(scaled);
    return sign | (uint16_t)r;
  }
  const uint32_t mant = x & 0x7fffffu;
  const uint32_t exp = (x >> 23) - 112u;               // rebias 127 -> 15
  uint32_t h = (exp << 10) | (mant >> 13);
  const uint32_t rest = mant & 0x1fffu;
  if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) h++;
  return sign | (uint16_t)h;
}

void row_min_max(const float *r, size_t cols, float &mn, float &mx) {
  mn = mx = r[0];
  for (size_t j = 1; j < cols; j++) {
    mn = std::min(mn, r[j]);
    mx = std::max(mx, r[j]);
  }
}

// quantization::quantize<int8_t> (Base.h:323-329)
int8_t quantize_to_i8(float x, float scale, int32_t offset) {
  const float r = x / scale + (float)offset;
  const int64_t q = (int64_t)std::nearbyintf(r);
  return (int8_t)std::max<int64_t>(-128, std::min<int64_t>(127, q));
}

} // namespace

extern "C" {

void mi355x_quantize_scale_offset_32to8(float scale, int32_t offset,
                                        int32_t out[4]) {
  out[3] = offset;
  // Powers of two become a pure shift (or a pure integer multiply).
  int e = 0;
  if (std::fabs(std::frexp(scale, &e)) == 0.5f) {
    const int exp2 = std::ilogb(scale);
    out[0] = 0;
    if (exp2 > 0) {
      out[1] = 0;
      out[2] = (int32_t)scale;
    } else {
      out[1] = -exp2;
      out[2] = 1;
    }
    return;
  }
  // Grow the multiplier by doubling (exact in fp32): first through the
  // post-shift, at least to 0.5 and up to 15 bits while it stays below 256,
  // then through the pre-shift for up to half as many bits while below 255.
  int post = 0, pre = 0;
  while (scale < 0.5f || (scale < 256.0f && post < 15)) {
    scale *= 2.0f;
    post++;
  }
  while (scale < 255.0f && pre < post / 2) {
    scale *= 2.0f;
    pre++;
  }
  out[0] = pre;
  out[1] = post;
  out[2] = (int32_t)std::round(scale);
}

int mi355x_choose_quantization_params(float min, float max, int schema,
                                      int qty, float *scale, int32_t *offset) {
  MI355X_REQUIRE(scale && offset, "NULL output");
  MI355X_REQUIRE(min <= max, "min must not be bigger than max");
  MI355X_REQUIRE(schema >= 0 && schema <= 3, "unknown schema %d", schema);
  Range q;
  MI355X_REQUIRE(quantized_range(qty, q), "unknown quantized type %d", qty);

  // zero must be representable
  min = std::min(min, 0.f);
  max = std::max(max, 0.f);
  if (schema == MI355X_SCHEMA_SYMMETRIC_WITH_UNSIGNED && !(min >= 0.f))
    schema = MI355X_SCHEMA_SYMMETRIC;
  const bool symmetric = schema == MI355X_SCHEMA_SYMMETRIC ||
                         schema == MI355X_SCHEMA_SYMMETRIC_POWER2;
  if (symmetric) {
    // widen the end that saturates later so that real 0 maps to quantized 0
    const double rmin = min / (double)q.lo;
    const double rmax = max / (double)q.hi;
    if (rmin > rmax) max = (float)(rmin * q.hi);
    else min = (float)(rmax * q.lo);
  }
  min = std::max(min, std::numeric_limits<float>::lowest());
  max = std::min(max, std::numeric_limits<float>::max());

  double s = ((double)max - min) / ((double)q.hi - q.lo);
  if (s == 0) s = 0.1;

  // zero point from whichever end has the smaller rounding error
  const double zp_lo = q.lo - min / s, zp_hi = q.hi - max / s;
  const double err_lo = std::abs((double)q.lo) + std::abs(min / s);
  const double err_hi = std::abs((double)q.hi) + std::abs(max / s);
  double zp = err_lo < err_hi ? zp_lo : zp_hi;
  if (std::abs(max + min) <= std::numeric_limits<float>::epsilon()) zp = 0;

  int32_t nudged;
  if (zp < q.lo) nudged = (int32_t)q.lo;
  else if (zp > q.hi) nudged = (int32_t)q.hi;
  else nudged = (int32_t)std::round(zp);

  if (schema == MI355X_SCHEMA_SYMMETRIC_POWER2)
    s = std::exp2(std::ceil(std::log2(s)));
  *scale = (float)s;
  *offset = nudged;
  return MI355X_OK;
}

size_t mi355x_fused_row_bytes(size_t cols, int kind) {
  const bool four = kind == MI355X_FUSED_U4_F16 || kind == MI355X_FUSED_U4_F32;
  const bool half = kind == MI355X_FUSED_U8_F16 || kind == MI355X_FUSED_U4_F16;
  return (four ? cols / 2 : cols) + (half ? 4 : 8);
}

int mi355x_fused_rowwise_quantize_host(const float *in, size_t rows,
                                       size_t cols, int kind, uint8_t *out) {
  MI355X_REQUIRE(kind >= 0 && kind <= 3, "unknown fused kind %d", kind);
  if (rows == 0) return MI355X_OK;
  MI355X_REQUIRE(in && out && cols > 0, "NULL or empty tensor");
  const bool four = kind == MI355X_FUSED_U4_F16 || kind == MI355X_FUSED_U4_F32;
  const bool half = kind == MI355X_FUSED_U8_F16 || kind == MI355X_FUSED_U4_F16;
  MI355X_REQUIRE(!four || cols % 2 == 0,
                 "4-bit fused rows need an even number of columns");
  const size_t row_bytes = mi355x_fused_row_bytes(cols, kind);
  const size_t data_bytes = four ? cols / 2 : cols;
  const float levels = four ? 15.0f : 255.0f;
  for (size_t i = 0; i < rows; i++) {
    const float *r = in + i * cols;
    uint8_t *o = out + i * row_bytes;
    float mn, mx;
    row_min_max(r, cols, mn, mx);
    // a (nearly) constant row keeps scale 1 so the division stays defined
    const float scale = (mx - mn) < 1e-10f
                            ? 1.0f
                            : (float)(((double)mx - (double)mn) / levels);
    if (four) std::memset(o, 0, data_bytes);
    for (size_t j = 0; j < cols; j++) {
      const float code = std::round((r[j] - mn) / scale);
      if (four) {
        const int v = std::max(0, std::min((int)code, 15));
        o[j / 2] |= (uint8_t)((j & 1) ? v << 4 : v);
      } else {
        o[j] = (uint8_t)(uint16_t)code;
      }
    }
    uint8_t *tail = o + data_bytes;
    if (half) {
      const uint16_t hs = to_half_bits(scale), ho = to_half_bits(mn);
      std::memcpy(tail, &hs, 2);
      std::memcpy(tail + 2, &ho, 2);
    } else {
      std::memcpy(tail, &scale, 4);
      std::memcpy(tail + 4, &mn, 4);
    }
  }
  return MI355X_OK;
}

int mi355x_specialize_bias_weights_qparams(float *bias_scale, int32_t *bias_offset,
                                           float input_scale, float *weights_scale,
                                           int bias_is_i32, int bias_is_zero) {
  MI355X_REQUIRE(bias_scale && bias_offset && weights_scale, "NULL argument");
  // an int32 bias always gets offset 0: its range makes that free
  if (bias_is_i32) *bias_offset = 0;
  const float product = input_scale * *weights_scale;
  if (product >= *bias_scale || bias_is_zero) {
    // the bias can take the accumulator's own scale without saturating
    *bias_scale = product;
  } else if (bias_is_i32) {
    // otherwise the weights scale gives way, and the product is formed again
    // so that it equals the bias scale exactly
    *weights_scale = *bias_scale / input_scale;
    *bias_scale = input_scale * *weights_scale;
  }
  return MI355X_OK;
}

int mi355x_specialize_bias_qparams(float *bias_scale, int32_t *bias_offset, float input_scale,
                                   float weights_scale, int bias_is_i32, int bias_is_zero) {
  MI355X_REQUIRE(bias_scale && bias_offset, "NULL argument");
  if (bias_is_i32) *bias_offset = 0;
  const float product = input_scale * weights_scale;
  // the accumulator's scale is taken only when it does not make the bias saturate
  if (product >= *bias_scale || bias_is_zero) *bias_scale = product;
  return MI355X_OK;
}

int mi355x_channelwise_quantize_conv_host(const float *filter, const float *bias,
                                          size_t channels, size_t per_channel,
                                          float input_scale, int schema, int8_t *filter_q,
                                          int32_t *bias_q, float *filter_scales,
                                          int32_t *filter_offsets, float *bias_scales,
                                          int32_t *bias_offsets) {
  if (channels == 0) return MI355X_OK;
  MI355X_REQUIRE(filter && bias && filter_q && bias_q && filter_scales && filter_offsets &&
                     bias_scales && bias_offsets && per_channel > 0,
                 "NULL or empty tensor");
  for (size_t c = 0; c < channels; c++) {
    const float *f = filter + c * per_channel;
    // filter parameters of the channel from its own range
    float mn, mx;
    row_min_max(f, per_channel, mn, mx);
    int rc = mi355x_choose_quantization_params(mn, mx, schema, MI355X_QTY_INT8,
                                               &filter_scales[c], &filter_offsets[c]);
    if (rc != MI355X_OK) return rc;
    // bias parameters from the one value the channel has, as an int32 tensor
    rc = mi355x_choose_quantization_params(bias[c], bias[c], schema, MI355X_QTY_INT32,
                                           &bias_scales[c], &bias_offsets[c]);
    if (rc != MI355X_OK) return rc;
    // then both are made to agree: bias scale == input scale * filter scale
    rc = mi355x_specialize_bias_weights_qparams(&bias_scales[c], &bias_offsets[c], input_scale,
                                                &filter_scales[c], 1, bias[c] == 0.0f);
    if (rc != MI355X_OK) return rc;
    for (size_t j = 0; j < per_channel; j++)
      filter_q[c * per_channel + j] = quantize_to_i8(f[j], filter_scales[c], filter_offsets[c]);
    const float r = bias[c] / bias_scales[c] + (float)bias_offsets[c];
    double v = (double)nearbyintf(r);
    if (v > 2147483647.0) v = 2147483647.0;
    if (v < -2147483648.0) v = -2147483648.0;
    bias_q[c] = (int32_t)v;
  }
  return MI355X_OK;
}

int mi355x_gemm_requant_hint_host(size_t K, size_t N, int32_t in_offset, int32_t out_offset,
                                  const int32_t *w_offsets, const void *bias, int bias_is_i8,
                                  const int32_t *bias_offsets, int32_t bias_offset,
                                  const int32_t *bias_pre, const int32_t *bias_post,
                                  const int32_t *bias_scale, const int32_t *out_pre,
                                  const int32_t *out_post, const int32_t *out_scale,
                                  int *flags) {
  MI355X_REQUIRE(flags, "flags is NULL");
  *flags = 0;
  MI355X_REQUIRE(out_pre && out_post && out_scale, "NULL output parameter vector");
  MI355X_REQUIRE(!bias || (bias_pre && bias_post && bias_scale), "NULL bias parameter vector");
  if (N == 0) return MI355X_OK;
  const int64_t k = (int64_t)K;
  const int64_t aoff = in_offset < 0 ? -(int64_t)in_offset : in_offset;
  const int64_t ooff = out_offset < 0 ? -(int64_t)out_offset : out_offset;
  bool ok = true, no_pre = true;
  for (size_t n = 0; n < N && ok; n++) {
    const int32_t pre = out_pre[n], post = out_post[n];
    if (pre < 0 || pre > 31 || post < 0 || post > 31) return MI355X_OK; // no hint for such a launch
    int64_t woff = w_offsets ? w_offsets[n] : 0;
    if (woff < 0) woff = -woff;
    int64_t scaled_bias = 0;
    if (bias) {
      const int32_t b = bias_is_i8 ? (int32_t) reinterpret_cast<const int8_t *>(bias)[n]
                                   : reinterpret_cast<const int32_t *>(bias)[n];
      const int32_t bo = bias_offsets ? bias_offsets[n] : bias_offset;
      const int32_t bp = bias_pre[n], bq = bias_post[n];
      if (bp < 0 || bp > 31 || bq < 0 || bq > 31) return MI355X_OK;
      // libjit_scale with 32-bit wrap-around, as the kernel computes it
      const uint32_t in = (uint32_t)b - (uint32_t)bo;
      const uint32_t rtn = bq > 0 ? (1u << (bq - 1)) : 0u;
      const uint32_t m = (uint32_t)((int32_t)in >> bp) * (uint32_t)bias_scale[n] + rtn;
      scaled_bias = (int64_t)((int32_t)m >> bq);
      if (scaled_bias < 0) scaled_bias = -scaled_bias;
    }
    // the largest magnitude the kernel can meet in front of the output multiply:
    // sum A*B over raw bytes, the two row-sum corrections, the column constant
    const int64_t bound = k * 128 * 128 + woff * k * 128 + k * aoff * woff + aoff * k * 128 +
                          scaled_bias;
    const int64_t x = (bound >> pre) + 1;
    int64_t sc = out_scale[n];
    if (sc < 0) sc = -sc;
    ok = ok && x < (1 << 23) && sc < (1 << 23) &&
         x * sc + ((int64_t)1 << post) * (ooff + 2) < ((int64_t)1 << 31);
    no_pre = no_pre && pre == 0;
  }
  if (ok) *flags = MI355X_REQUANT_ACC24 | (no_pre ? MI355X_REQUANT_NO_PRE_SHIFT : 0);
  return MI355X_OK;
}

int mi355x_rowwise_quantize_i8_host(const float *in, size_t rows, size_t cols,
                                    int schema, int8_t *out, float *scales,
                                    int32_t *offsets) {
  if (rows == 0) return MI355X_OK;
  MI355X_REQUIRE(in && out && scales && offsets && cols > 0,
                 "NULL or empty tensor");
  for (size_t i = 0; i < rows; i++) {
    const float *r = in + i * cols;
    float mn, mx;
    row_min_max(r, cols, mn, mx);
    int rc = mi355x_choose_quantization_params(mn, mx, schema, MI355X_QTY_INT8,
                                               &scales[i], &offsets[i]);
    if (rc != MI355X_OK) return rc;
    for (size_t j = 0; j < cols; j++)
      out[i * cols + j] = quantize_to_i8(r[j], scales[i], offsets[i]);
  }
  return MI355X_OK;
}

} // extern "C"
