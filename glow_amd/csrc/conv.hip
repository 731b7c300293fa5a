// Quantized and ChannelwiseQuantized 2-D convolution for int8 NHWC tensors as
// an implicit GEMM on the int8 matrix cores (reference
// lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:49-239, 496-562).
//
// GEMM view per group: rows = output pixels (n, oh, ow), columns = output
// channels of the group, K = (fx, fy, c) in the filter's own memory order
// [OC][KH][KW][IC/group]. A-tile rows are gathered from the NHWC input on the
// fly, 16 channel bytes at a time. The CPU loop skips taps that fall into the
// padding; a tap whose bytes all equal the input offset contributes
// (in - inOffset) = 0 just the same, so out-of-image taps are filled with the
// input offset and the dense contraction of gemm_i8.h applies unchanged.
#include "gemm_i8.h"
#include "conv_halo.h"
#include "conv_halo_wide.h"
#include "gemm_stream.h"

namespace mi355x {

struct ConvRows {
  const int8_t *in;
  int N, IH, IW, IC, OH, OW;
  int KW, ICg;
  int strideH, strideW, padT, padL, dilH, dilW;
  int M;                 // N*OH*OW
  int fill;              // input offset replicated into four bytes
  int c_base;            // first input channel of the group

  struct Row {
    const int8_t *img;   // input image n, channel c_base
    int ih0, iw0;
    bool ok;
  };
  __device__ __forceinline__ void set_group(int g) { c_base = g * ICg; }
  __device__ __forceinline__ Row row(int m) const {
    Row r;
    r.ok = m < M;
    const int mm = r.ok ? m : 0;
    const int n = mm / (OH * OW);
    const int rem = mm - n * (OH * OW);
    const int oh = rem / OW, ow = rem - oh * OW;
    r.img = in + (long long)n * IH * IW * IC + c_base;
    r.ih0 = oh * strideH - padT;
    r.iw0 = ow * strideW - padL;
    return r;
  }
  // the filter tap and channel that the 16 bytes A[m][k..k+15] of any row
  // come from (ICg % 16 == 0, so a chunk never straddles a tap)
  struct Loc {
    int dh, dw, c;
    int k, fy; // the K position and the tap's column, for advance()
  };
  __device__ __forceinline__ Loc locate(int k) const {
    const int tap = k / ICg, c = k - tap * ICg;
    const int fx = tap / KW, fy = tap - fx * KW;
    return Loc{fx * dilH, fy * dilW, c, k, fy};
  }
  // The location one K step (64 bytes) further on. With at least 64 channels
  // per group a step crosses at most one tap boundary, which takes a compare
  // and a few selects instead of the two integer divisions of locate().
  __device__ __forceinline__ void advance(Loc &l) const {
    l.k += 64;
    if (ICg < 64) {
      l = locate(l.k);
      return;
    }
    l.c += 64;
    if (l.c >= ICg) {
      l.c -= ICg;
      l.fy += 1;
      l.dw += dilW;
      if (l.fy == KW) {
        l.fy = 0;
        l.dw = 0;
        l.dh += dilH;
      }
    }
  }
  // address of those bytes for an existing row: inside the image, or a chunk
  // of input-offset bytes for a padding tap
  __device__ __forceinline__ const int8_t *chunk_ptr(const Row &r, const Loc &l) const {
    const int ih = r.ih0 + l.dh, iw = r.iw0 + l.dw;
    if (ih < 0 || iw < 0 || ih >= IH || iw >= IW)
      return reinterpret_cast<const int8_t *>(g_fill_table.b) + ((fill & 0xff) << 4);
    return r.img + ((long long)ih * IW + iw) * IC + l.c;
  }
  // 16 bytes A[m][k..k+15]; ALIGNED needs ICg % 16 == 0 so a chunk never
  // straddles a tap, and 16-byte aligned pixels.
  template <bool ALIGNED>
  __device__ __forceinline__ int4 load(const Row &r, int k, int K) const {
    if (!r.ok || k >= K) return make_int4(0, 0, 0, 0);
    if constexpr (ALIGNED) {
      const int tap = k / ICg, c = k - tap * ICg;
      const int fx = tap / KW, fy = tap - fx * KW;
      const int ih = r.ih0 + fx * dilH, iw = r.iw0 + fy * dilW;
      if (ih < 0 || iw < 0 || ih >= IH || iw >= IW)
        return make_int4(fill, fill, fill, fill);
      return *reinterpret_cast<const int4 *>(
          r.img + ((long long)ih * IW + iw) * IC + c);
    } else {
      uint32_t w[4] = {0, 0, 0, 0};
      const int n = min(16, K - k);
      for (int b = 0; b < n; b++) {
        const int kk = k + b;
        const int tap = kk / ICg, c = kk - tap * ICg;
        const int fx = tap / KW, fy = tap - fx * KW;
        const int ih = r.ih0 + fx * dilH, iw = r.iw0 + fy * dilW;
        uint32_t v = (uint32_t)fill & 0xff;
        if (ih >= 0 && iw >= 0 && ih < IH && iw < IW)
          v = (uint8_t)r.img[((long long)ih * IW + iw) * IC + c];
        w[b >> 2] |= v << (8 * (b & 3));
      }
      return make_int4((int)w[0], (int)w[1], (int)w[2], (int)w[3]);
    }
  }
};

static int conv_common(int8_t *out, const int8_t *in, const int8_t *filter,
                       const mi355x_conv_geom *g, Epilogue ep, bool need_sa,
                       void *stream) {
  MI355X_REQUIRE(g, "geom is NULL");
  MI355X_REQUIRE(g->N >= 0 && g->IH > 0 && g->IW > 0 && g->IC > 0 &&
                     g->OH >= 0 && g->OW >= 0 && g->OC > 0 && g->KH > 0 &&
                     g->KW > 0 && g->strideH > 0 && g->strideW > 0 &&
                     g->dilH > 0 && g->dilW > 0 && g->group > 0 &&
                     g->padT >= 0 && g->padL >= 0,
                 "invalid convolution geometry");
  MI355X_REQUIRE(g->IC % g->group == 0 && g->OC % g->group == 0,
                 "channels not divisible by group");
  const long long M = (long long)g->N * g->OH * g->OW;
  if (M == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in && filter, "NULL tensor");
  const int ICg = g->IC / g->group, OCg = g->OC / g->group;
  const long long K = (long long)g->KH * g->KW * ICg;
  MI355X_REQUIRE(M < (1LL << 30) && K < (1LL << 30), "convolution too large");
  // (OH, OW carry the bottom and right padding: an output pixel whose window
  // lies wholly in the padding is legal and sees the input offset everywhere)
  MI355X_REQUIRE(ep.a_off >= -128 && ep.a_off <= 127,
                 "input offset %d outside the int8 range", ep.a_off);
  MI355X_REQUIRE(ep.act == MI355X_ACT_NONE || ep.act == MI355X_ACT_RELU ||
                     ep.act == MI355X_ACT_CLIP ||
                     ep.act == MI355X_ACT_LEAKY_RELU,
                 "fused activation %d is not supported for quantized types",
                 ep.act);
  if (ep.act == MI355X_ACT_LEAKY_RELU)
    MI355X_REQUIRE(shift_ok(ep.a0) && shift_ok(ep.a1),
                   "leaky-relu pre/post shift outside [0, 31]");
  if (ep.add.res) {
    MI355X_REQUIRE(shift_ok(ep.add.own_pre) && shift_ok(ep.add.own_post) &&
                       shift_ok(ep.add.res_pre) && shift_ok(ep.add.res_post) &&
                       (!ep.add.relu || (shift_ok(ep.add.dest_pre) &&
                                         shift_ok(ep.add.dest_post))),
                   "fused add: pre/post shift outside [0, 31]");
    MI355X_REQUIRE(!ep.add.relu || (ep.add.sum_off >= -128 && ep.add.sum_off <= 127),
                   "fused add: sum offset outside the int8 range");
  }

  ConvRows A;
  A.in = in;
  A.N = g->N; A.IH = g->IH; A.IW = g->IW; A.IC = g->IC;
  A.OH = g->OH; A.OW = g->OW;
  A.KW = g->KW; A.ICg = ICg;
  A.strideH = g->strideH; A.strideW = g->strideW;
  A.padT = g->padT; A.padL = g->padL;
  A.dilH = g->dilH; A.dilW = g->dilW;
  A.M = (int)M;
  A.fill = (int)(0x01010101u * (uint32_t)(uint8_t)(int8_t)ep.a_off);
  A.c_base = 0;
  DenseRows B{filter, K, OCg};
  ep.out = out;
  ep.ldc = g->OC;
  const bool al_a = (ICg % 16 == 0) && (g->IC % 16 == 0) &&
                    ((((uintptr_t)in) & 15) == 0);
  const bool al_b = (K % 16 == 0) && ((((uintptr_t)filter) & 15) == 0);
  const bool need_sb = ep.a_off != 0 && !ep.sum_b;
  // 3x3, stride 1, 64 input channels, symmetric filters: operands resident in
  // LDS (conv_halo.h). Tile 7 forces it, tiles 0..6 keep the implicit GEMM.
  const bool al_out = ((((uintptr_t)out) | ((uintptr_t)ep.add.res)) & 15) == 0;
  if ((g_tile_override < 0 || g_tile_override == 7) && !need_sa && !need_sb && al_a && al_b &&
      al_out) {
    size_t lds = 0;
    const int rows = conv_halo_rows(g, device_cus(), lds);
    if (rows != 0 && lds <= lds_limit()) {
      ep.fast = g_requant_hint & 3;
      return conv_halo_launch(in, filter, g, ep, lds, rows, as_stream(stream));
    }
  }
  // The same over 128, 256 or 512 input channels: the input patch resident in
  // LDS, the filter slice streamed through it tap by tap (conv_halo_wide.h).
  if ((g_tile_override < 0 || g_tile_override == 7) && !need_sa && !need_sb && al_a && al_b &&
      al_out) {
    HaloWide cv{};
    size_t lds = 0;
    const size_t lds_max = lds_limit();
    const int waves = conv_halo_wide_plan(g, lds_max, cv, lds);
    if (waves != 0) {
      ep.fast = g_requant_hint & 3;
      return conv_halo_wide_launch(in, filter, g, ep, cv, lds, lds_max, waves, as_stream(stream));
    }
  }
  // Pointwise convolutions (any stride) over 64, 128 or 256 channels, and
  // windows without padding or dilation whose rows are whole 32-byte chunks
  // (KW * IC of 32, 64 or 128 bytes; the stem of an image network after
  // space-to-depth: 4x4 over 16 channels) with K of 64, 128 or 256: the
  // streaming kernel (gemm_stream.h), by its shape rule or when tile 8 is
  // asked for.
  const long long seg = (long long)g->KW * g->IC;        // bytes per window row
  const bool seg_ok = g->KH == 1 ? g->KW == 1
                                 : (seg == 32 || seg == 64 || seg == 128) && g->dilH == 1 &&
                                       g->dilW == 1 && g->IC % 16 == 0;
  if (seg_ok && g->padT == 0 && g->padL == 0 && g->group == 1 &&
      (long long)(g->OH - 1) * g->strideH + g->KH <= g->IH &&
      (long long)(g->OW - 1) * g->strideW + g->KW <= g->IW &&
      (g_tile_override == 8 || (g_tile_override < 0 && stream_applies((int)M, OCg))) &&
      stream_can_run((int)M, OCg, (int)K, need_sa, need_sb, al_a && al_b, ep)) {
    StreamRows R;
    R.in = in; R.ld = g->IC;
    R.dense = g->KH == 1 && g->strideH == 1 && g->strideW == 1 && g->OH == g->IH && g->OW == g->IW;
    R.OW = g->OW; R.OHW = g->OH * g->OW; R.IH = g->IH; R.IW = g->IW; R.IC = g->IC;
    R.sH = g->strideH; R.sW = g->strideW;
    R.seg_chunks = g->KH > 1 ? (int)(seg / 32) : (int)(K / 32);
    R.seg_stride = (long long)g->IW * g->IC;
    ep.fast = g_requant_hint & 3;
    return gemm_stream_launch(R, filter, ep, (int)M, OCg, (int)K, as_stream(stream));
  }
  // Tiles 6..8 name one special kernel each; a launch that kernel cannot serve
  // says so instead of running another kernel under the asked-for number.
  if (g_tile_override >= 6 && g_tile_override <= 8)
    return fail(MI355X_ERR_NOT_SUPPORTED,
                "tile %d does not apply to this convolution (shape, alignment or offsets)",
                g_tile_override);
  // A pointwise convolution over the whole image is a plain matrix product:
  // row m of A is pixel m of the input, no taps to locate and no padding.
  if (g->KH == 1 && g->KW == 1 && g->strideH == 1 && g->strideW == 1 &&
      g->padT == 0 && g->padL == 0 && g->group == 1 && g->OH == g->IH &&
      g->OW == g->IW) {
    DenseRows Ad{in, g->IC, (int)M};
    return gemm_dispatch(Ad, B, ep, (int)M, OCg, (int)K, 1, 0, need_sa, need_sb,
                         al_a && al_b, as_stream(stream));
  }
  return gemm_dispatch(A, B, ep, (int)M, OCg, (int)K, g->group,
                       (long long)OCg * K, need_sa, need_sb, al_a && al_b,
                       as_stream(stream));
}

static void set_act(Epilogue &ep, int32_t act_type, const int32_t *act_args) {
  ep.act = act_type;
  ep.a0 = ep.a1 = ep.a2 = 0;
  if (act_args) {
    if (act_type == MI355X_ACT_CLIP) {
      ep.a0 = act_args[0];
      ep.a1 = act_args[1];
    } else if (act_type == MI355X_ACT_LEAKY_RELU) {
      ep.a0 = act_args[0];
      ep.a1 = act_args[1];
      ep.a2 = act_args[2];
    }
  }
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

static int mi355x_cwq_conv2d_i8_impl(int8_t *out, const int8_t *in, const int8_t *filter,
                         const void *bias, int bias_is_i8,
                         const mi355x_conv_geom *geom, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type,
                         const int32_t *act_args, int filter_offsets_all_zero,
                         const int32_t *filter_row_sums, void *stream) {
  MI355X_REQUIRE(bias && filter_offsets && bias_offsets && bias_pre &&
                     bias_post && bias_scale && out_pre && out_post && out_scale,
                 "NULL per-channel parameter vector");
  MI355X_REQUIRE(act_args || (act_type != MI355X_ACT_CLIP &&
                              act_type != MI355X_ACT_LEAKY_RELU),
                 "act_args is NULL");
  Epilogue ep{};
  ep.bias = bias;
  ep.bias_is_i8 = bias_is_i8;
  ep.b_off = ColParam{bias_offsets, 0};
  ep.bias_pre = ColParam{bias_pre, 0};
  ep.bias_post = ColParam{bias_post, 0};
  ep.bias_scale = ColParam{bias_scale, 0};
  ep.w_off = ColParam{filter_offsets, 0};
  ep.out_pre = ColParam{out_pre, 0};
  ep.out_post = ColParam{out_post, 0};
  ep.out_scale = ColParam{out_scale, 0};
  ep.a_off = in_offset;
  ep.out_off = out_offset;
  set_act(ep, act_type, act_args);
  ep.sum_b = filter_row_sums;
  return conv_common(out, in, filter, geom, ep, !filter_offsets_all_zero,
                     stream);
}

int mi355x_cwq_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                         const void *bias, int bias_is_i8,
                         const mi355x_conv_geom *geom, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type,
                         const int32_t *act_args, int filter_offsets_all_zero,
                         const int32_t *filter_row_sums, void *stream) {
  return mi355x_cwq_conv2d_i8_impl(out, in, filter, bias, bias_is_i8, geom, out_offset, in_offset, filter_offsets, bias_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, act_type, act_args, filter_offsets_all_zero, filter_row_sums, stream);
}

int mi355x_cwq_conv2d_i8_opts(int8_t *out, const int8_t *in, const int8_t *filter,
                         const void *bias, int bias_is_i8,
                         const mi355x_conv_geom *geom, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type,
                         const int32_t *act_args, int filter_offsets_all_zero,
                         const int32_t *filter_row_sums, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_cwq_conv2d_i8_impl(out, in, filter, bias, bias_is_i8, geom, out_offset, in_offset, filter_offsets, bias_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, act_type, act_args, filter_offsets_all_zero, filter_row_sums, stream);
}

static int mi355x_cwq_conv2d_add_i8_impl(
    int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
    int bias_is_i8, const mi355x_conv_geom *geom, int32_t conv_offset,
    int32_t in_offset, const int32_t *filter_offsets,
    const int32_t *bias_offsets, const int32_t *bias_pre,
    const int32_t *bias_post, const int32_t *bias_scale, const int32_t *out_pre,
    const int32_t *out_post, const int32_t *out_scale, int32_t act_type,
    const int32_t *act_args, int filter_offsets_all_zero,
    const int32_t *filter_row_sums, const int8_t *residual,
    const mi355x_fused_add *add, void *stream) {
  MI355X_REQUIRE(bias && filter_offsets && bias_offsets && bias_pre &&
                     bias_post && bias_scale && out_pre && out_post && out_scale,
                 "NULL per-channel parameter vector");
  MI355X_REQUIRE(act_args || (act_type != MI355X_ACT_CLIP &&
                              act_type != MI355X_ACT_LEAKY_RELU),
                 "act_args is NULL");
  MI355X_REQUIRE(residual && add, "NULL residual or add parameters");
  Epilogue ep{};
  ep.bias = bias;
  ep.bias_is_i8 = bias_is_i8;
  ep.b_off = ColParam{bias_offsets, 0};
  ep.bias_pre = ColParam{bias_pre, 0};
  ep.bias_post = ColParam{bias_post, 0};
  ep.bias_scale = ColParam{bias_scale, 0};
  ep.w_off = ColParam{filter_offsets, 0};
  ep.out_pre = ColParam{out_pre, 0};
  ep.out_post = ColParam{out_post, 0};
  ep.out_scale = ColParam{out_scale, 0};
  ep.a_off = in_offset;
  ep.out_off = conv_offset;
  set_act(ep, act_type, act_args);
  ep.sum_b = filter_row_sums;
  ep.add.res = residual;
  ep.add.sum_off = add->sum_offset;
  ep.add.own_off = conv_offset;
  ep.add.res_off = add->residual_offset;
  ep.add.own_pre = add->conv_pre;
  ep.add.own_post = add->conv_post;
  ep.add.own_scale = add->conv_scale;
  ep.add.res_pre = add->residual_pre;
  ep.add.res_post = add->residual_post;
  ep.add.res_scale = add->residual_scale;
  ep.add.relu = add->relu;
  ep.add.dest_off = add->dest_offset;
  ep.add.dest_pre = add->dest_pre;
  ep.add.dest_post = add->dest_post;
  ep.add.dest_scale = add->dest_scale;
  auto fits = [](int32_t v) { return v > -(1 << 23) && v < (1 << 23); };
  ep.add.small = fits(add->conv_scale) && fits(add->residual_scale) &&
                 (!add->relu || fits(add->dest_scale)) && conv_offset >= -128 &&
                 conv_offset <= 127 && add->residual_offset > -(1 << 22) &&
                 add->residual_offset < (1 << 22);
  return conv_common(out, in, filter, geom, ep, !filter_offsets_all_zero,
                     stream);
}

int mi355x_cwq_conv2d_add_i8(
    int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
    int bias_is_i8, const mi355x_conv_geom *geom, int32_t conv_offset,
    int32_t in_offset, const int32_t *filter_offsets,
    const int32_t *bias_offsets, const int32_t *bias_pre,
    const int32_t *bias_post, const int32_t *bias_scale, const int32_t *out_pre,
    const int32_t *out_post, const int32_t *out_scale, int32_t act_type,
    const int32_t *act_args, int filter_offsets_all_zero,
    const int32_t *filter_row_sums, const int8_t *residual,
    const mi355x_fused_add *add, void *stream) {
  return mi355x_cwq_conv2d_add_i8_impl(out, in, filter, bias, bias_is_i8, geom, conv_offset, in_offset, filter_offsets, bias_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, act_type, act_args, filter_offsets_all_zero, filter_row_sums, residual, add, stream);
}

int mi355x_cwq_conv2d_add_i8_opts(
    int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
    int bias_is_i8, const mi355x_conv_geom *geom, int32_t conv_offset,
    int32_t in_offset, const int32_t *filter_offsets,
    const int32_t *bias_offsets, const int32_t *bias_pre,
    const int32_t *bias_post, const int32_t *bias_scale, const int32_t *out_pre,
    const int32_t *out_post, const int32_t *out_scale, int32_t act_type,
    const int32_t *act_args, int filter_offsets_all_zero,
    const int32_t *filter_row_sums, const int8_t *residual,
    const mi355x_fused_add *add, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_cwq_conv2d_add_i8_impl(out, in, filter, bias, bias_is_i8, geom, conv_offset, in_offset, filter_offsets, bias_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, act_type, act_args, filter_offsets_all_zero, filter_row_sums, residual, add, stream);
}

static int mi355x_conv2d_i8_impl(int8_t *out, const int8_t *in, const int8_t *filter,
                     const void *bias, int bias_is_i8,
                     const mi355x_conv_geom *geom, int32_t out_offset,
                     int32_t in_offset, int32_t filter_offset,
                     int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                     int32_t bias_scale, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, int32_t act_type,
                     const int32_t *act_args, const int32_t *filter_row_sums,
                     void *stream) {
  MI355X_REQUIRE(bias, "bias is NULL");
  MI355X_REQUIRE(shift_ok(bias_pre) && shift_ok(bias_post) &&
                     shift_ok(out_pre) && shift_ok(out_post),
                 "pre/post shift outside [0, 31]");
  MI355X_REQUIRE(act_args || (act_type != MI355X_ACT_CLIP &&
                              act_type != MI355X_ACT_LEAKY_RELU),
                 "act_args is NULL");
  Epilogue ep{};
  ep.bias = bias;
  ep.bias_is_i8 = bias_is_i8;
  ep.b_off = ColParam{nullptr, bias_offset};
  ep.bias_pre = ColParam{nullptr, bias_pre};
  ep.bias_post = ColParam{nullptr, bias_post};
  ep.bias_scale = ColParam{nullptr, bias_scale};
  ep.w_off = ColParam{nullptr, filter_offset};
  ep.out_pre = ColParam{nullptr, out_pre};
  ep.out_post = ColParam{nullptr, out_post};
  ep.out_scale = ColParam{nullptr, out_scale};
  ep.a_off = in_offset;
  ep.out_off = out_offset;
  set_act(ep, act_type, act_args);
  ep.sum_b = filter_row_sums;
  return conv_common(out, in, filter, geom, ep, filter_offset != 0, stream);
}

int mi355x_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                     const void *bias, int bias_is_i8,
                     const mi355x_conv_geom *geom, int32_t out_offset,
                     int32_t in_offset, int32_t filter_offset,
                     int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                     int32_t bias_scale, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, int32_t act_type,
                     const int32_t *act_args, const int32_t *filter_row_sums,
                     void *stream) {
  return mi355x_conv2d_i8_impl(out, in, filter, bias, bias_is_i8, geom, out_offset, in_offset, filter_offset, bias_offset, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, act_type, act_args, filter_row_sums, stream);
}

int mi355x_conv2d_i8_opts(int8_t *out, const int8_t *in, const int8_t *filter,
                     const void *bias, int bias_is_i8,
                     const mi355x_conv_geom *geom, int32_t out_offset,
                     int32_t in_offset, int32_t filter_offset,
                     int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                     int32_t bias_scale, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, int32_t act_type,
                     const int32_t *act_args, const int32_t *filter_row_sums,
                     void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_conv2d_i8_impl(out, in, filter, bias, bias_is_i8, geom, out_offset, in_offset, filter_offset, bias_offset, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, act_type, act_args, filter_row_sums, stream);
}

} // extern "C"
