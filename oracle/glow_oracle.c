/*
 * CPU restatement of Glow's quantized-inference arithmetic. TEST
 * INFRASTRUCTURE ONLY: the checker for the HIP kernels and the timed CPU
 * baseline. See glow_oracle.h for what pins each function.
 *
 * Build: gcc -std=c11 -O2 -fno-fast-math -ffp-contract=off (see Makefile).
 */
#include "glow_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* scalar helpers                                                           */
/* ------------------------------------------------------------------------ */

/* Arithmetic right shift of a signed value, spelled out so the behaviour does
 * not rest on the implementation-defined >> of a negative int. */
static inline int32_t asr32(int32_t v, int32_t s) {
  uint32_t u = (uint32_t)v;
  s &= 31;
  if (s == 0) return v;
  uint32_t r = u >> s;
  if (v < 0) r |= ~(0xFFFFFFFFu >> s);
  return (int32_t)r;
}

/* libjit_defs.h:158-173. ((((in >> pre) * scale) + rtn) >> post) + offset in
 * 32-bit wrapping arithmetic; rtn = 1 << (post-1) when post > 0. */
int32_t go_scale_i32(int32_t input, int32_t pre, int32_t post, int32_t scale,
                     int32_t offset) {
  uint32_t rtn = (post > 0) ? (1u << ((post - 1) & 31)) : 0u;
  uint32_t m = (uint32_t)asr32(input, pre) * (uint32_t)scale + rtn;
  return (int32_t)((uint32_t)asr32((int32_t)m, post) + (uint32_t)offset);
}

/* libjit_defs.h:147-148 */
int8_t go_clip_i8(int32_t v) {
  return (int8_t)(v < -128 ? -128 : (v > 127 ? 127 : v));
}

/* libjit_defs.h:206-233 */
int32_t go_activation_i32(int32_t input, int32_t offset, int32_t actType,
                          const int32_t *actArgs) {
  switch (actType) {
  case 0:
    return input;
  case 1:
    return input > offset ? input : offset;
  case 2: {
    int32_t v = input > actArgs[0] ? input : actArgs[0];
    return v < actArgs[1] ? v : actArgs[1];
  }
  case 3:
  case 4:
    return input; /* fused tanh / sigmoid are rejected for quantized types */
  default:
    if (input >= offset) return input;
    return go_scale_i32((int32_t)((uint32_t)input - (uint32_t)offset),
                        actArgs[0], actArgs[1], actArgs[2], offset);
  }
}

/* IEEE binary32 -> binary16, round to nearest even, with subnormals, inf and
 * NaN (what fp16_ieee_from_fp32_value computes; Float16.h:38). */
uint16_t go_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7FFFFFFFu;
  if (absx >= 0x7F800000u) { /* inf / NaN */
    return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? 0x0200u : 0));
  }
  if (absx >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7C00u);
  }
  if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (tie goes to even 0) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t m = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  uint32_t shift;
  uint32_t half;
  if (e < -14) { /* subnormal half: value = m * 2^(e-23), unit 2^-24 */
    shift = (uint32_t)(-1 - e); /* 13 + (-14 - e) */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  shift = 13;
  half = 1u << 12;
  uint32_t q = m >> shift; /* 11 bits incl. hidden */
  uint32_t rem = m & 0x1FFFu;
  uint32_t he = (uint32_t)(e + 15);
  uint32_t out = (he << 10) + (q & 0x3FFu);
  if (rem > half || (rem == half && (q & 1u))) out++; /* carry ripples */
  return (uint16_t)(sign | out);
}

float go_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu;
  uint32_t m = h & 0x3FFu;
  uint32_t x;
  if (e == 0) {
    if (m == 0) {
      x = sign;
    } else { /* subnormal */
      float v = (float)m * 5.9604644775390625e-8f; /* 2^-24 */
      memcpy(&x, &v, 4);
      x |= sign;
    }
  } else if (e == 31) {
    x = sign | 0x7F800000u | (m << 13);
  } else {
    x = sign | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

/* ------------------------------------------------------------------------ */
/* host-side parameter derivation                                           */
/* ------------------------------------------------------------------------ */

/* Base.cpp:793-799 */
static int is_float_pow2(float v) {
  int e;
  return fabsf(frexpf(v, &e)) == 0.5f;
}

/* Base.cpp:234-359 */
void go_quantize_scale_offset_32to8(float scale, int32_t offset,
                                    int32_t out[4]) {
  int pre = 0, post = 0;
  if (is_float_pow2(scale)) {
    int e = ilogbf(scale);
    if (e > 0) {
      out[0] = 0; out[1] = 0; out[2] = (int32_t)scale; out[3] = offset;
    } else {
      out[0] = 0; out[1] = -e; out[2] = 1; out[3] = offset;
    }
    return;
  }
  while (scale < 0.5 || (scale < 256 && post < 15)) {
    scale *= 2;
    post++;
  }
  while (scale < 255 && pre < (post / 2)) {
    scale *= 2;
    pre++;
  }
  out[0] = pre;
  out[1] = post;
  out[2] = (int32_t)roundf(scale);
  out[3] = offset;
}

/* Base.cpp:361-403 */
static void quantized_range(int qty, int64_t *qmin, int64_t *qmax) {
  switch (qty) {
  case 8: *qmin = -128; *qmax = 127; break;
  case 108: *qmin = 0; *qmax = 255; break;
  case 16: *qmin = -32768; *qmax = 32767; break;
  default: /* Int32QTy: restricted to int30 */
    *qmin = (int64_t)INT32_MIN >> 2;
    *qmax = (int64_t)INT32_MAX >> 2;
    break;
  }
}

/* Base.cpp:433-565, Calibration::None */
void go_choose_qparams(float min, float max, int schema, int qty,
                       float *scaleOut, int32_t *offsetOut) {
  int64_t qmin, qmax;
  quantized_range(qty, &qmin, &qmax);
  if (min > 0.f) min = 0.f;
  if (max < 0.f) max = 0.f;
  if (schema == GO_SYMMETRIC_WITH_UNSIGNED) {
    if (!(min >= 0.f)) schema = GO_SYMMETRIC;
  }
  if (schema == GO_SYMMETRIC || schema == GO_SYMMETRIC_POW2) {
    double rmin = min / (double)qmin;
    double rmax = max / (double)qmax;
    if (rmin > rmax) {
      max = (float)(rmin * qmax);
    } else {
      min = (float)(rmax * qmin);
    }
  }
  if (min < -3.402823466e+38f) min = -3.402823466e+38f;
  if (max > 3.402823466e+38f) max = 3.402823466e+38f;

  double scale = ((double)max - min) / ((double)qmax - qmin);
  if (scale == 0) scale = 0.1;

  double zpMin = qmin - min / scale;
  double zpMax = qmax - max / scale;
  double zpMinErr = fabs((double)qmin) + fabs(min / scale);
  double zpMaxErr = fabs((double)qmax) + fabs(max / scale);
  double zp = zpMinErr < zpMaxErr ? zpMin : zpMax;

  float diff = fabsf(max + min);
  if (diff <= 1.1920928955078125e-07f) zp = 0;

  int32_t nudged;
  if (zp < qmin) {
    nudged = (int32_t)qmin;
  } else if (zp > qmax) {
    nudged = (int32_t)qmax;
  } else {
    nudged = (int32_t)round(zp);
  }
  if (schema == GO_SYMMETRIC_POW2) {
    scale = exp2(ceil(log2(scale)));
  }
  *scaleOut = (float)scale;
  *offsetOut = nudged;
}

/* Base.cpp:594-629 */
void go_specialize_bias_weights_qparams(float *biasScale, int32_t *biasOffset,
                                        float inputScale, float *weightsScale,
                                        int biasIsI32, int biasZero) {
  if (biasIsI32) *biasOffset = 0;
  float ws = *weightsScale;
  float bs = *biasScale;
  if (inputScale * ws >= bs || biasZero) {
    bs = inputScale * ws;
  } else if (biasIsI32) {
    ws = bs / inputScale;
    bs = inputScale * ws;
  }
  *biasScale = bs;
  *weightsScale = ws;
}

/* Base.cpp:567-592 (specializeBiasQuantizationParams): the weights keep their
 * scale; the bias takes inputScale * weightsScale unless that is smaller than
 * the scale its own range asks for (and the bias is not all zero). */
void go_specialize_bias_qparams(float *biasScale, int32_t *biasOffset, float inputScale,
                                float weightsScale, int biasIsI32, int biasZero) {
  int32_t off = *biasOffset;
  if (biasIsI32) off = 0;
  float bs = *biasScale;
  if (inputScale * weightsScale >= bs || biasZero) bs = inputScale * weightsScale;
  *biasScale = bs;
  *biasOffset = off;
}

/* Base.h:323-329: clip<int64, DestTy>((int64)nearbyintf(x/scale + offset)) */
static int64_t quantize_value_i64(float x, float scale, int32_t offset) {
  float r = x / scale + (float)offset;
  return (int64_t)nearbyintf(r);
}

int8_t go_quantize_value_i8(float x, float scale, int32_t offset) {
  int64_t q = quantize_value_i64(x, scale, offset);
  return (int8_t)(q < -128 ? -128 : (q > 127 ? 127 : q));
}

int32_t go_quantize_value_i32(float x, float scale, int32_t offset) {
  int64_t q = quantize_value_i64(x, scale, offset);
  return (int32_t)(q < INT32_MIN ? INT32_MIN : (q > INT32_MAX ? INT32_MAX : q));
}

/* Base.h:522-557, int32-offset branch (FC weights) */
void go_rowwise_quantize_i8(const float *in, size_t rows, size_t cols,
                            int schema, int8_t *out, float *scales,
                            int32_t *offsets) {
  for (size_t i = 0; i < rows; i++) {
    const float *r = in + i * cols;
    float mn = r[0], mx = r[0];
    for (size_t j = 1; j < cols; j++) {
      if (r[j] < mn) mn = r[j];
      if (r[j] > mx) mx = r[j];
    }
    float s;
    int32_t o;
    go_choose_qparams(mn, mx, schema, 8, &s, &o);
    for (size_t j = 0; j < cols; j++) {
      out[i * cols + j] = go_quantize_value_i8(r[j], s, o);
    }
    scales[i] = s;
    offsets[i] = o;
  }
}

/* Graph.cpp:3576-3700 (createChannelwiseQuantizedConv with a float filter and a
 * float bias, no parameters given, int8 filter / int32 bias), in the order of
 * the reference: all filter parameters (getTensorQuantizationParams over
 * dimension 0, Base.cpp:632-691), all bias parameters (each channel's bias is a
 * one-element group, so min == max == bias[c]; Int32QTy), the specialisation
 * loop (Base.cpp:594-629), then quantizeTensor of the filter and of the bias
 * (Base.cpp:707-760 with quantize<T>, Base.h:323-329). */
void go_channelwise_quantize_conv(const float *filter, const float *bias, size_t channels,
                                  size_t perChannel, float inputScale, int schema,
                                  int8_t *filterQ, int32_t *biasQ, float *filterScales,
                                  int32_t *filterOffsets, float *biasScales,
                                  int32_t *biasOffsets) {
  for (size_t c = 0; c < channels; c++) {
    float lo = FLT_MAX, hi = -FLT_MAX;
    for (size_t j = 0; j < perChannel; j++) {
      const float v = filter[c * perChannel + j];
      if (v < lo) lo = v;
      if (v > hi) hi = v;
    }
    go_choose_qparams(lo, hi, schema, 8, &filterScales[c], &filterOffsets[c]);
  }
  for (size_t c = 0; c < channels; c++)
    go_choose_qparams(bias[c], bias[c], schema, 32, &biasScales[c], &biasOffsets[c]);
  for (size_t c = 0; c < channels; c++)
    go_specialize_bias_weights_qparams(&biasScales[c], &biasOffsets[c], inputScale,
                                       &filterScales[c], 1, bias[c] == 0.f);
  for (size_t c = 0; c < channels; c++)
    for (size_t j = 0; j < perChannel; j++)
      filterQ[c * perChannel + j] =
          go_quantize_value_i8(filter[c * perChannel + j], filterScales[c], filterOffsets[c]);
  for (size_t c = 0; c < channels; c++)
    biasQ[c] = go_quantize_value_i32(bias[c], biasScales[c], biasOffsets[c]);
}

size_t go_fused_row_bytes(size_t cols, int kind) {
  size_t so = (kind == GO_U8_F32 || kind == GO_U4_F32) ? 8 : 4;
  size_t data = (kind == GO_U8_F32 || kind == GO_U8_F16) ? cols : cols / 2;
  return data + so;
}

/* Base.h:598-678. 8-bit: q = (uint8)(uint16)round((x-offset)/scale)
 * (Base.h:361-370); 4-bit: clamp(round(.),0,15), even column -> low nibble
 * (Base.h:374-379, 663-669). Scale/offset stored after the data as T. */
void go_fused_rowwise_quantize(const float *in, size_t rows, size_t cols,
                               int kind, uint8_t *out) {
  const int is4 = (kind == GO_U4_F16 || kind == GO_U4_F32);
  const int isF16 = (kind == GO_U8_F16 || kind == GO_U4_F16);
  const size_t rowBytes = go_fused_row_bytes(cols, kind);
  const float range = is4 ? 15.0f : 255.0f;
  for (size_t i = 0; i < rows; i++) {
    const float *r = in + i * cols;
    uint8_t *o = out + i * rowBytes;
    float mn = r[0], mx = r[0];
    for (size_t j = 1; j < cols; j++) {
      if (r[j] < mn) mn = r[j];
      if (r[j] > mx) mx = r[j];
    }
    const float scale = ((mx - mn) < 1e-10f)
                            ? 1.0f
                            : (float)(((double)mx - (double)mn) / range);
    const float offset = mn;
    for (size_t j = 0; j < cols; j++) {
      float q = roundf((r[j] - offset) / scale);
      if (!is4) {
        o[j] = (uint8_t)(uint16_t)q;
      } else {
        int v = (int)q;
        if (v > 15) v = 15;
        if (v < 0) v = 0;
        if ((j & 1) == 0) {
          o[j / 2] = (uint8_t)v;
        } else {
          o[j / 2] |= (uint8_t)(v << 4);
        }
      }
    }
    uint8_t *so = o + rowBytes - (isF16 ? 4 : 8);
    if (isF16) {
      uint16_t hs = go_f32_to_f16(scale), ho = go_f32_to_f16(offset);
      memcpy(so, &hs, 2);
      memcpy(so + 2, &ho, 2);
    } else {
      memcpy(so, &scale, 4);
      memcpy(so + 4, &offset, 4);
    }
  }
}

/* ------------------------------------------------------------------------ */
/* elementwise                                                              */
/* ------------------------------------------------------------------------ */

/* libjit.cpp:2998-3002: clip((int32)nearbyintf(in/scale + offset)).
 * The reference's float -> int32 conversion is undefined for |v| >= 2^31 (on
 * x86 it happens to yield INT32_MIN for either sign). Beyond that range this
 * restatement saturates before the clip, which is what Glow's host-side
 * quantization::quantize does through int64 (Base.h:323-329); inside the
 * range the two agree. */
void go_quantize_i8(int8_t *dst, const float *src, size_t n, float scale,
                    int32_t offset) {
  for (size_t i = 0; i < n; i++) {
    float r = nearbyintf(src[i] / scale + (float)offset);
    int32_t v;
    if (r >= 2147483648.0f) v = INT32_MAX;
    else if (r <= -2147483648.0f) v = INT32_MIN;
    else v = (int32_t)r;
    dst[i] = go_clip_i8(v);
  }
}

/* libjit.cpp:3016-3019: scale * (in - offset) */
void go_dequantize_i8(float *dst, const int8_t *src, size_t n, float scale,
                      int32_t offset) {
  for (size_t i = 0; i < n; i++) {
    dst[i] = scale * (float)((int32_t)src[i] - offset);
  }
}

/* libjit.cpp:3031-3038 */
void go_rescale_i8(int8_t *dst, const int8_t *src, size_t n, int32_t outOffset,
                   int32_t inOffset, int32_t pre, int32_t post,
                   int32_t scale) {
  for (size_t i = 0; i < n; i++) {
    int32_t s = go_scale_i32((int32_t)src[i] - inOffset, pre, post, scale,
                             outOffset);
    dst[i] = go_clip_i8(s);
  }
}

/* libjit_defs.h:151-153 */
static inline int16_t clip_i16(int32_t v) {
  return (int16_t)(v < -32768 ? -32768 : (v > 32767 ? 32767 : v));
}

/* libjit_defs.h:158-173 instantiated as libjit_scale<int64_t> (DestTy stays
 * int32_t): the arithmetic runs in 64 bits and the result is truncated. */
static inline int32_t scale_i64(int64_t input, int32_t pre, int32_t post, int32_t scale,
                                int32_t offset) {
  const int64_t rtn = (post > 0) ? (int64_t)(1 << (post - 1)) : 0;
  const int64_t v = ((((input >> pre) * (int64_t)scale) + rtn) >> post) + (int64_t)offset;
  return (int32_t)(uint32_t)(uint64_t)v;
}

static inline int32_t round_to_i32(float r) {
  /* saturating where the reference's conversion is undefined (see go_quantize_i8) */
  if (r >= 2147483648.0f) return INT32_MAX;
  if (r <= -2147483648.0f) return INT32_MIN;
  return (int32_t)r;
}

/* libjit.cpp:3004-3008 */
void go_quantize_i16(int16_t *dst, const float *src, size_t n, float scale, int32_t offset) {
  for (size_t i = 0; i < n; i++)
    dst[i] = clip_i16(round_to_i32(nearbyintf(src[i] / scale + (float)offset)));
}

/* libjit.cpp:3010-3014 (no clip) */
void go_quantize_i32(int32_t *dst, const float *src, size_t n, float scale, int32_t offset) {
  for (size_t i = 0; i < n; i++)
    dst[i] = round_to_i32(nearbyintf(src[i] / scale + (float)offset));
}

/* libjit.cpp:3021-3024 */
void go_dequantize_i16(float *dst, const int16_t *src, size_t n, float scale, int32_t offset) {
  for (size_t i = 0; i < n; i++) dst[i] = scale * (float)((int32_t)src[i] - offset);
}

/* libjit.cpp:3026-3029: the subtraction is 32-bit (wraps) */
void go_dequantize_i32(float *dst, const int32_t *src, size_t n, float scale, int32_t offset) {
  for (size_t i = 0; i < n; i++)
    dst[i] = scale * (float)(int32_t)((uint32_t)src[i] - (uint32_t)offset);
}

/* libjit.cpp:3040-3047 */
void go_rescale_i16(int16_t *dst, const int16_t *src, size_t n, int32_t outOffset,
                    int32_t inOffset, int32_t pre, int32_t post, int32_t scale) {
  for (size_t i = 0; i < n; i++)
    dst[i] = clip_i16(scale_i64((int64_t)((int32_t)src[i] - inOffset), pre, post, scale,
                                outOffset));
}

/* libjit.cpp:3049-3056: in - inOffset is 32-bit (wraps), then widened */
void go_rescale_i32(int32_t *dst, const int32_t *src, size_t n, int32_t outOffset,
                    int32_t inOffset, int32_t pre, int32_t post, int32_t scale) {
  for (size_t i = 0; i < n; i++)
    dst[i] = scale_i64((int64_t)(int32_t)((uint32_t)src[i] - (uint32_t)inOffset), pre, post,
                       scale, outOffset);
}

/* libjit.cpp:565-653 (libjit_transpose_generic; the tiling there only orders
 * the copies): out[x0..] = in[source coordinate], where source dimension
 * shuffle[d] runs with output dimension d. elemSize bytes per element
 * (libjit_transpose_i8 / _f / _u / _b: 1, 4, 8, 1). */
void go_transpose(void *out, const void *in, const size_t *idim, const size_t *shuffle,
                  size_t numDims, size_t elemSize) {
  size_t odim[6], istride[6], oc[6] = {0, 0, 0, 0, 0, 0};
  size_t total = 1;
  for (size_t d = 0; d < numDims; d++) {
    odim[d] = idim[shuffle[d]];
    total *= idim[d];
  }
  size_t st = 1;
  for (size_t d = numDims; d-- > 0;) {
    istride[d] = st;
    st *= idim[d];
  }
  for (size_t o = 0; o < total; o++) {
    size_t src = 0;
    for (size_t d = 0; d < numDims; d++) src += oc[d] * istride[shuffle[d]];
    memcpy((char *)out + o * elemSize, (const char *)in + src * elemSize, elemSize);
    for (size_t d = numDims; d-- > 0;) {
      if (++oc[d] < odim[d]) break;
      oc[d] = 0;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* FullyConnected / MatMul                                                  */
/* ------------------------------------------------------------------------ */

static inline int32_t bias_at(const void *bias, int biasIsI8, size_t j) {
  return biasIsI8 ? (int32_t)((const int8_t *)bias)[j]
                  : ((const int32_t *)bias)[j];
}

/* wrapping multiply-accumulate */
static inline int32_t mac32(int32_t acc, int32_t a, int32_t b) {
  return (int32_t)((uint32_t)acc + (uint32_t)a * (uint32_t)b);
}

/* libjit_matmul.cpp:254-280 */
void go_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
              const void *bias, int biasIsI8, size_t M, size_t K, size_t N,
              int32_t outOffset, int32_t inOffset, int32_t weightsOffset,
              int32_t biasOffset, int32_t biasPre, int32_t biasPost,
              int32_t biasScale, int32_t outPre, int32_t outPost,
              int32_t outScale) {
  for (size_t i = 0; i < M; i++) {
    for (size_t j = 0; j < N; j++) {
      int32_t sum = go_scale_i32(
          (int32_t)((uint32_t)bias_at(bias, biasIsI8, j) - (uint32_t)biasOffset),
          biasPre, biasPost, biasScale, 0);
      for (size_t k = 0; k < K; k++) {
        int32_t I = in[i * K + k];
        int32_t W = weights[k * N + j];
        sum = mac32(sum, I - inOffset, W - weightsOffset);
      }
      out[i * N + j] =
          go_clip_i8(go_scale_i32(sum, outPre, outPost, outScale, outOffset));
    }
  }
}

/* libjit_matmul.cpp:284-316 */
void go_rwq_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                  const void *bias, int biasIsI8, const int32_t *weightsOffsets,
                  const int32_t *biasPre, const int32_t *biasPost,
                  const int32_t *biasScale, const int32_t *outPre,
                  const int32_t *outPost, const int32_t *outScale, size_t M,
                  size_t K, size_t N, int32_t outOffset, int32_t inOffset,
                  int32_t biasOffset) {
  for (size_t i = 0; i < M; i++) {
    const int8_t *irow = in + i * K;
    for (size_t j = 0; j < N; j++) {
      const int8_t *wrow = weights + j * K;
      const int32_t wo = weightsOffsets[j];
      int32_t sum = 0;
      for (size_t k = 0; k < K; k++) {
        sum = mac32(sum, (int32_t)wrow[k] - wo, (int32_t)irow[k] - inOffset);
      }
      int32_t B = go_scale_i32(
          (int32_t)((uint32_t)bias_at(bias, biasIsI8, j) - (uint32_t)biasOffset),
          biasPre[j], biasPost[j], biasScale[j], 0);
      sum = (int32_t)((uint32_t)sum + (uint32_t)B);
      out[i * N + j] = go_clip_i8(
          go_scale_i32(sum, outPre[j], outPost[j], outScale[j], outOffset));
    }
  }
}

/* libjit_matmul.cpp:353-371 */
void go_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs, size_t M,
                  size_t K, size_t N, int32_t outOffset, int32_t lhsOffset,
                  int32_t rhsOffset, int32_t outPre, int32_t outPost,
                  int32_t outScale) {
  for (size_t x = 0; x < M; x++) {
    for (size_t y = 0; y < N; y++) {
      int32_t sum = 0;
      for (size_t i = 0; i < K; i++) {
        sum = mac32(sum, (int32_t)lhs[x * K + i] - lhsOffset,
                    (int32_t)rhs[i * N + y] - rhsOffset);
      }
      out[x * N + y] =
          go_clip_i8(go_scale_i32(sum, outPre, outPost, outScale, outOffset));
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Convolution                                                              */
/* ------------------------------------------------------------------------ */

/* One output element of either convolution: bias seeds the accumulator,
 * out-of-bounds taps are skipped (libjit_conv.cpp:198-224). */
static inline int8_t conv_point(const int8_t *in, const int8_t *filter,
                                const go_conv_geom *g, int n, int grp, int d,
                                int ax, int ay, int32_t biasScaled,
                                int32_t inOffset, int32_t filterOffset,
                                int32_t outPre, int32_t outPost,
                                int32_t outScale, int32_t outOffset,
                                int32_t actType, const int32_t *actArgs) {
  const int inCperG = g->IC / g->group;
  int32_t sum = biasScaled;
  const long x = (long)ax * g->strideH - g->padT;
  const long y = (long)ay * g->strideW - g->padL;
  for (int fx = 0; fx < g->KH; fx++) {
    for (int fy = 0; fy < g->KW; fy++) {
      long ox = x + (long)fx * g->dilH;
      long oy = y + (long)fy * g->dilW;
      if (ox < 0 || oy < 0 || ox >= g->IH || oy >= g->IW) continue;
      const int8_t *ip =
          in + (((size_t)n * g->IH + (size_t)ox) * g->IW + (size_t)oy) * g->IC +
          (size_t)grp * inCperG;
      const int8_t *fp =
          filter + (((size_t)d * g->KH + fx) * g->KW + fy) * (size_t)inCperG;
      for (int fd = 0; fd < inCperG; fd++) {
        sum = mac32(sum, (int32_t)fp[fd] - filterOffset,
                    (int32_t)ip[fd] - inOffset);
      }
    }
  }
  int32_t s = go_scale_i32(sum, outPre, outPost, outScale, outOffset);
  s = go_activation_i32(s, outOffset, actType, actArgs);
  return go_clip_i8(s);
}

/* libjit_conv.cpp:49-147 */
void go_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                  const void *bias, int biasIsI8, const go_conv_geom *g,
                  int32_t outOffset, int32_t inOffset, int32_t filterOffset,
                  int32_t biasOffset, int32_t biasPre, int32_t biasPost,
                  int32_t biasScale, int32_t outPre, int32_t outPost,
                  int32_t outScale, int32_t actType, const int32_t *actArgs) {
  const int outCperG = g->OC / g->group;
  for (int n = 0; n < g->N; n++)
    for (int grp = 0; grp < g->group; grp++)
      for (int d = grp * outCperG; d < (grp + 1) * outCperG; d++) {
        int32_t b = go_scale_i32(
            (int32_t)((uint32_t)bias_at(bias, biasIsI8, (size_t)d) -
                      (uint32_t)biasOffset),
            biasPre, biasPost, biasScale, 0);
        for (int ax = 0; ax < g->OH; ax++)
          for (int ay = 0; ay < g->OW; ay++)
            out[(((size_t)n * g->OH + ax) * g->OW + ay) * g->OC + d] =
                conv_point(in, filter, g, n, grp, d, ax, ay, b, inOffset,
                           filterOffset, outPre, outPost, outScale, outOffset,
                           actType, actArgs);
      }
}

/* libjit_conv.cpp:151-239 */
void go_cwq_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                      const void *bias, int biasIsI8, const go_conv_geom *g,
                      int32_t outOffset, int32_t inOffset,
                      const int32_t *filterOffsets, const int32_t *biasOffsets,
                      const int32_t *biasPre, const int32_t *biasPost,
                      const int32_t *biasScale, const int32_t *outPre,
                      const int32_t *outPost, const int32_t *outScale,
                      int32_t actType, const int32_t *actArgs) {
  const int outCperG = g->OC / g->group;
  for (int n = 0; n < g->N; n++)
    for (int grp = 0; grp < g->group; grp++)
      for (int d = grp * outCperG; d < (grp + 1) * outCperG; d++) {
        int32_t b = go_scale_i32(
            (int32_t)((uint32_t)bias_at(bias, biasIsI8, (size_t)d) -
                      (uint32_t)biasOffsets[d]),
            biasPre[d], biasPost[d], biasScale[d], 0);
        for (int ax = 0; ax < g->OH; ax++)
          for (int ay = 0; ay < g->OW; ay++)
            out[(((size_t)n * g->OH + ax) * g->OW + ay) * g->OC + d] =
                conv_point(in, filter, g, n, grp, d, ax, ay, b, inOffset,
                           filterOffsets[d], outPre[d], outPost[d], outScale[d],
                           outOffset, actType, actArgs);
      }
}

/* ------------------------------------------------------------------------ */
/* FusedRowwiseQuantizedSparseLengthsWeightedSum                            */
/* libjit_conv.cpp:244-349 (channelwise quantized 3-D convolution, NTHWC;
 * pads are {near, far, top, bottom, left, right}, of which the near, top and
 * left ones are read; the dilation is ignored there as here). */
void go_cwq_conv3d_i8(int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
                      int biasIsI8, const go_conv3d_geom *g, int32_t outOffset,
                      int32_t inOffset, const int32_t *filterOffsets,
                      const int32_t *biasOffsets, const int32_t *biasPre,
                      const int32_t *biasPost, const int32_t *biasScale, const int32_t *outPre,
                      const int32_t *outPost, const int32_t *outScale, int32_t actType,
                      const int32_t *actArgs) {
  const size_t icg = (size_t)(g->IC / g->group), ocg = (size_t)(g->OC / g->group);
  for (size_t n = 0; n < (size_t)g->N; n++)
    for (size_t grp = 0; grp < (size_t)g->group; grp++)
      for (size_t d = grp * ocg; d < (grp + 1) * ocg; d++)
        for (size_t at = 0; at < (size_t)g->OT; at++)
          for (size_t ax = 0; ax < (size_t)g->OH; ax++)
            for (size_t ay = 0; ay < (size_t)g->OW; ay++) {
              int32_t sum = go_scale_i32(bias_at(bias, biasIsI8, d) - biasOffsets[d], biasPre[d],
                                         biasPost[d], biasScale[d], 0);
              for (size_t ft = 0; ft < (size_t)g->KT; ft++)
                for (size_t fx = 0; fx < (size_t)g->KH; fx++)
                  for (size_t fy = 0; fy < (size_t)g->KW; fy++) {
                    const long ot = (long)(at * g->strideT + ft) - g->padN;
                    const long ox = (long)(ax * g->strideH + fx) - g->padT;
                    const long oy = (long)(ay * g->strideW + fy) - g->padL;
                    if (ot < 0 || ox < 0 || oy < 0 || ot >= g->IT || ox >= g->IH || oy >= g->IW)
                      continue;
                    const int8_t *ip =
                        in + ((((n * g->IT + (size_t)ot) * g->IH + (size_t)ox) * g->IW +
                               (size_t)oy) * g->IC + grp * icg);
                    const int8_t *fp =
                        filter + ((((d * g->KT + ft) * g->KH + fx) * g->KW + fy) * icg);
                    for (size_t fd = 0; fd < icg; fd++)
                      sum = mac32(sum, (int32_t)fp[fd] - filterOffsets[d],
                                  (int32_t)ip[fd] - inOffset);
                  }
              int32_t v = go_scale_i32(sum, outPre[d], outPost[d], outScale[d], outOffset);
              v = go_activation_i32(v, outOffset, actType, actArgs);
              out[(((n * g->OT + at) * g->OH + ax) * g->OW + ay) * g->OC + d] = go_clip_i8(v);
            }
}

/* ------------------------------------------------------------------------ */

static inline int64_t index_at(const void *idx, int is64, size_t i) {
  return is64 ? ((const int64_t *)idx)[i] : (int64_t)((const int32_t *)idx)[i];
}

/* libjit.cpp:1253-1276 */
void go_frwq_slws_f32(float *dest, const uint8_t *data, const float *weights,
                      const void *indices, int idxIs64, const int32_t *lengths,
                      size_t segments, size_t inLineSize, size_t outLineSize) {
  memset(dest, 0, segments * outLineSize * sizeof(float));
  size_t cur = 0;
  for (size_t i = 0; i < segments; i++) {
    float *d = dest + i * outLineSize;
    for (int32_t j = 0, e = lengths[i]; j < e; j++) {
      const float w = weights[cur];
      const size_t line = (size_t)index_at(indices, idxIs64, cur);
      const uint8_t *row = data + line * inLineSize;
      float scale, offset;
      memcpy(&scale, row + inLineSize - 8, 4);
      memcpy(&offset, row + inLineSize - 4, 4);
      for (size_t k = 0; k < outLineSize; k++) {
        const float f = (scale * (float)row[k]) + offset;
        d[k] += w * f;
      }
      cur++;
    }
  }
}

/* InterpreterNodes.cpp:5764-5841; dispatch :5843-5889 */
void go_frwq_slws_generic(void *dest, int outIsF16, const uint8_t *data,
                          int kind, const void *weights, int weightsAreF16,
                          const void *indices, int idxIs64,
                          const int32_t *lengths, size_t segments,
                          size_t inLineSize, size_t outLineSize,
                          int fp16Accum) {
  const int is4 = (kind == GO_U4_F16 || kind == GO_U4_F32);
  const int soF16 = (kind == GO_U8_F16 || kind == GO_U4_F16);
  const int accF16 = outIsF16 && fp16Accum && soF16;
  float *accF = (float *)malloc(outLineSize * sizeof(float));
  uint16_t *accH = (uint16_t *)malloc(outLineSize * sizeof(uint16_t));
  size_t cur = 0;
  for (size_t i = 0; i < segments; i++) {
    for (size_t k = 0; k < outLineSize; k++) {
      accF[k] = 0.0f;
      accH[k] = 0;
    }
    for (int32_t j = 0, e = lengths[i]; j < e; j++) {
      float w = 1.0f;
      if (weights) {
        w = weightsAreF16 ? go_f16_to_f32(((const uint16_t *)weights)[cur])
                          : ((const float *)weights)[cur];
      }
      const size_t line = (size_t)index_at(indices, idxIs64, cur);
      cur++;
      const uint8_t *row = data + line * inLineSize;
      float scale, offset;
      if (soF16) {
        uint16_t hs, ho;
        memcpy(&hs, row + inLineSize - 4, 2);
        memcpy(&ho, row + inLineSize - 2, 2);
        scale = go_f16_to_f32(hs);
        offset = go_f16_to_f32(ho);
      } else {
        memcpy(&scale, row + inLineSize - 8, 4);
        memcpy(&offset, row + inLineSize - 4, 4);
      }
      for (size_t k = 0; k < outLineSize; k++) {
        float d;
        if (!is4) {
          d = ((float)row[k] * scale) + offset; /* Base.h:383-393 */
        } else {
          uint8_t b = row[k / 2];
          if (k & 1) b >>= 4;
          b &= 0x0f;
          d = ((float)b * scale) + offset; /* Base.h:399-406 */
        }
        if (accF16) {
          /* accum(fp16) += fp16(d * w): float16::operator+= , Float16.h */
          float term = go_f16_to_f32(go_f32_to_f16(d * w));
          accH[k] = go_f32_to_f16(go_f16_to_f32(accH[k]) + term);
        } else {
          accF[k] += d * w;
        }
      }
    }
    for (size_t k = 0; k < outLineSize; k++) {
      if (outIsF16) {
        ((uint16_t *)dest)[i * outLineSize + k] =
            accF16 ? accH[k] : go_f32_to_f16(accF[k]);
      } else {
        ((float *)dest)[i * outLineSize + k] = accF[k];
      }
    }
  }
  free(accF);
  free(accH);
}

/* libjit.cpp:2454-2481 */
void go_embedding_bag_byte_rowwise_offsets_f32(
    float *dest, const uint8_t *data, const float *weights,
    const int32_t *indices, const int32_t *offsets, size_t segments,
    size_t numIndices, size_t inLineSize, size_t outLineSize,
    int hasEndOffset) {
  if (hasEndOffset) --segments;
  memset(dest, 0, segments * outLineSize * sizeof(float));
  for (size_t i = 0; i < segments; i++) {
    size_t start = (size_t)offsets[i];
    size_t end = (!hasEndOffset && i == segments - 1) ? numIndices
                                                      : (size_t)offsets[i + 1];
    float *d = dest + i * outLineSize;
    for (size_t j = start; j < end; j++) {
      const float w = weights[j];
      const uint8_t *row = data + (size_t)indices[j] * inLineSize;
      float scale, offset;
      memcpy(&scale, row + inLineSize - 8, 4);
      memcpy(&offset, row + inLineSize - 4, 4);
      for (size_t k = 0; k < outLineSize; k++) {
        const float f = (scale * (float)row[k]) + offset;
        d[k] += w * f;
      }
    }
  }
}

/* ---- int8 glue operators ----------------------------------------------- */

/* libjit.cpp:1593-1603 with body lhs + rhs (:1675-1676) */
void go_add_i8(int8_t *dest, const int8_t *lhs, const int8_t *rhs, size_t n,
               int32_t destOffset, int32_t lhsOffset, int32_t rhsOffset,
               int32_t lhsPre, int32_t lhsPost, int32_t lhsScale,
               int32_t rhsPre, int32_t rhsPost, int32_t rhsScale) {
  for (size_t i = 0; i < n; i++) {
    const int32_t l = go_scale_i32(lhs[i] - lhsOffset, lhsPre, lhsPost, lhsScale, 0);
    const int32_t r = go_scale_i32(rhs[i] - rhsOffset, rhsPre, rhsPost, rhsScale, 0);
    dest[i] = go_clip_i8((int32_t)((uint32_t)l + (uint32_t)r + (uint32_t)destOffset));
  }
}

/* libjit.cpp:1851-1858 */
void go_relu_i8(int8_t *dest, const int8_t *src, size_t n, int8_t srcOffset,
                int8_t destOffset, int32_t destPre, int32_t destPost,
                int32_t destScale) {
  for (size_t i = 0; i < n; i++) {
    const int32_t v = src[i] > srcOffset ? src[i] : srcOffset;
    dest[i] = go_clip_i8(go_scale_i32(v - srcOffset, destPre, destPost, destScale, destOffset));
  }
}

/* libjit.cpp:1865-1873 */
void go_clip_elem_i8(int8_t *dest, const int8_t *src, size_t n, int8_t clipMin, int8_t clipMax,
                     int8_t srcOffset, int8_t destOffset, int32_t destPre, int32_t destPost,
                     int32_t destScale) {
  for (size_t i = 0; i < n; i++) {
    int32_t v = src[i] > clipMin ? src[i] : clipMin;
    v = v < clipMax ? v : clipMax;
    dest[i] = go_clip_i8(go_scale_i32(v - srcOffset, destPre, destPost, destScale, destOffset));
  }
}

/* libjit.cpp:1880-1892 */
void go_leaky_relu_i8(int8_t *dest, const int8_t *src, size_t n, int8_t srcOffset,
                      int8_t destOffset, int32_t posPre, int32_t posPost, int32_t posScale,
                      int32_t negPre, int32_t negPost, int32_t negScale) {
  for (size_t i = 0; i < n; i++) {
    const int32_t v = src[i];
    dest[i] = go_clip_i8(v >= srcOffset
                             ? go_scale_i32(v - srcOffset, posPre, posPost, posScale, destOffset)
                             : go_scale_i32(v - srcOffset, negPre, negPost, negScale, destOffset));
  }
}

/* lib/Backends/CPU/libjit_cpu/libjit_cpu.cpp:45-46 */
void go_max_splat_i8(int8_t *dest, const int8_t *src, size_t n, int8_t value) {
  for (size_t i = 0; i < n; i++) dest[i] = src[i] > value ? src[i] : value;
}

/* libjit.cpp:997-1015 (libjit_batchedadd_i8 and _i32_i8, :1945-1969); the
 * subtraction and the sum wrap in 32 bits like the compiled reference */
void go_batched_add_i8(int8_t *dest, const int8_t *batch, const void *slice, int sliceIsI32,
                       size_t numSlice, size_t sliceSize, int32_t destOffset,
                       int32_t batchOffset, int32_t sliceOffset, int32_t batchPre,
                       int32_t batchPost, int32_t batchScale, int32_t slicePre,
                       int32_t slicePost, int32_t sliceScale) {
  for (size_t n = 0; n < numSlice; n++) {
    const size_t base = n * sliceSize;
    for (size_t i = 0; i < sliceSize; i++) {
      const int32_t sv = sliceIsI32 ? ((const int32_t *)slice)[i] : ((const int8_t *)slice)[i];
      const int32_t b = (int32_t)((uint32_t)batch[base + i] - (uint32_t)batchOffset);
      const int32_t s = (int32_t)((uint32_t)sv - (uint32_t)sliceOffset);
      const int32_t x = go_scale_i32(b, batchPre, batchPost, batchScale, 0);
      const int32_t y = go_scale_i32(s, slicePre, slicePost, sliceScale, 0);
      dest[base + i] = go_clip_i8((int32_t)((uint32_t)x + (uint32_t)y + (uint32_t)destOffset));
    }
  }
}

/* window limits of libjit_defs.h:257-275 */
static void window(ptrdiff_t inMin, size_t inSize, size_t k, ptrdiff_t *lo, ptrdiff_t *len) {
  const ptrdiff_t fmin = inMin < 0 ? -inMin : 0;
  ptrdiff_t fmax = (ptrdiff_t)inSize - inMin;
  if ((ptrdiff_t)k < fmax) fmax = (ptrdiff_t)k;
  *lo = fmin;
  *len = fmax - fmin > 0 ? fmax - fmin : 0;
}

/* libjit.cpp:812-884 */
void go_max_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH,
                    size_t IW, size_t C, size_t OH, size_t OW, size_t kH,
                    size_t kW, size_t sH, size_t sW, size_t padT, size_t padL,
                    int32_t outOffset) {
  for (size_t n = 0; n < N; n++)
    for (size_t oh = 0; oh < OH; oh++) {
      ptrdiff_t h0, hl;
      const ptrdiff_t ihMin = (ptrdiff_t)(oh * sH) - (ptrdiff_t)padT;
      window(ihMin, IH, kH, &h0, &hl);
      for (size_t ow = 0; ow < OW; ow++) {
        ptrdiff_t w0, wl;
        const ptrdiff_t iwMin = (ptrdiff_t)(ow * sW) - (ptrdiff_t)padL;
        window(iwMin, IW, kW, &w0, &wl);
        for (size_t c = 0; c < C; c++) {
          int8_t m = INT8_MIN;
          for (ptrdiff_t fh = 0; fh < hl; fh++)
            for (ptrdiff_t fw = 0; fw < wl; fw++) {
              const int8_t v = in[((n * IH + (size_t)(ihMin + h0 + fh)) * IW +
                                   (size_t)(iwMin + w0 + fw)) * C + c];
              if (v > m) m = v;
            }
          *out++ = (hl > 0 && wl > 0) ? m : (int8_t)outOffset;
        }
      }
    }
}

/* libjit_defs.h:239-244 */
static int32_t div_round_i32(int32_t input, int32_t divider) {
  const int32_t rnd = divider >> 1;
  return input > 0 ? (input + rnd) / divider : (input - rnd) / divider;
}

/* libjit.cpp:2812-2880 */
void go_avg_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH,
                    size_t IW, size_t C, size_t OH, size_t OW, size_t kH,
                    size_t kW, size_t sH, size_t sW, size_t padT, size_t padL,
                    int countIncludePads, int32_t outOffset, int32_t inOffset,
                    int32_t outPre, int32_t outPost, int32_t outScale) {
  for (size_t n = 0; n < N; n++)
    for (size_t oh = 0; oh < OH; oh++) {
      ptrdiff_t h0, hl;
      const ptrdiff_t ihMin = (ptrdiff_t)(oh * sH) - (ptrdiff_t)padT;
      window(ihMin, IH, kH, &h0, &hl);
      for (size_t ow = 0; ow < OW; ow++) {
        ptrdiff_t w0, wl;
        const ptrdiff_t iwMin = (ptrdiff_t)(ow * sW) - (ptrdiff_t)padL;
        window(iwMin, IW, kW, &w0, &wl);
        for (size_t c = 0; c < C; c++) {
          int32_t sum = 0;
          for (ptrdiff_t fh = 0; fh < hl; fh++)
            for (ptrdiff_t fw = 0; fw < wl; fw++)
              sum += in[((n * IH + (size_t)(ihMin + h0 + fh)) * IW +
                         (size_t)(iwMin + w0 + fw)) * C + c] - inOffset;
          if (countIncludePads) {
            *out++ = go_clip_i8(go_scale_i32(sum, outPre, outPost, outScale, outOffset));
          } else {
            const int32_t area = (int32_t)(hl * wl);
            if (area == 0) {
              *out++ = (int8_t)outOffset;
            } else {
              sum = go_scale_i32(sum, outPre, outPost, outScale, 0);
              *out++ = go_clip_i8(div_round_i32(sum, area) + outOffset);
            }
          }
        }
      }
    }
}

/* libjit.cpp:3058-3082 */
void go_softmax_f32(float *out, const float *in, size_t rows, size_t cols) {
  for (size_t n = 0; n < rows; n++) {
    const float *x = in + n * cols;
    float *y = out + n * cols;
    float mx = x[0];
    for (size_t i = 1; i < cols; i++) mx = x[i] > mx ? x[i] : mx;
    float sum = 0;
    for (size_t i = 0; i < cols; i++) {
      const float e = expf(x[i] - mx);
      sum += e;
      y[i] = e;
    }
    for (size_t i = 0; i < cols; i++) y[i] = y[i] / sum;
  }
}

/* libjit.cpp:1913-1916 */
void go_sigmoid_f32(float *out, const float *in, size_t n) {
  for (size_t i = 0; i < n; i++) {
    const float e = expf(-in[i]);
    out[i] = 1 / (e + 1);
  }
}

/* libjit.cpp:418-440 */
void go_gather(uint8_t *dest, const uint8_t *data, const int64_t *indices,
               size_t numIndices, size_t sliceBytes, size_t numSamples,
               size_t sampleBytes) {
  size_t outIdx = 0;
  for (size_t s = 0; s < numSamples; s++)
    for (size_t i = 0; i < numIndices; i++) {
      memcpy(dest + outIdx * sliceBytes,
             data + s * sampleBytes + (size_t)indices[i] * sliceBytes, sliceBytes);
      outIdx++;
    }
}

/* libjit.cpp:1232-1251 */
void go_rwq_slws_f32(float *dest, const uint8_t *data, const float *scales,
                     const float *offsets, const float *weights,
                     const void *indices, int indicesAre64, const int32_t *lengths,
                     size_t segments, size_t lineSize) {
  memset(dest, 0, segments * lineSize * sizeof(float));
  size_t cur = 0;
  for (size_t i = 0; i < segments; i++) {
    for (int32_t j = 0; j < lengths[i]; j++) {
      const float weight = weights[cur];
      const size_t line = indicesAre64 ? (size_t)((const int64_t *)indices)[cur]
                                       : (size_t)((const int32_t *)indices)[cur];
      const float scale = scales[line], offset = offsets[line];
      for (size_t k = 0; k < lineSize; k++) {
        const float f = scale * (float)data[line * lineSize + k] + offset;
        dest[i * lineSize + k] += weight * f;
      }
      cur++;
    }
  }
}
