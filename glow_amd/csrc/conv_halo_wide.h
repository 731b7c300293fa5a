// 3x3, stride-1 convolution over 128, 256 or 512 input channels (the later
// stages of an image network; reference
// lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:49-239): the scheme of conv_halo.h
// for channel counts whose filter slice no longer fits LDS beside the input.
//
//   * a workgroup computes 64 output channels for a tile of at most 256 pixels:
//     whole output rows of one image, or, when images are small (14 x 14,
//     7 x 7), several whole images; one wave per 32 consecutive pixels;
//   * the tile's input patch (its rows plus one above and below per image, one
//     pixel left and right; padding materialised as input-offset bytes) is
//     staged in LDS once and stays: every input byte is read from memory once
//     per tile and channel slice instead of once per tap;
//   * the filter slice (64 x 9 x IC bytes: 74 to 295 KB) passes through LDS one
//     tap at a time in a ring of slots, loaded global -> LDS directly by the
//     first four waves (global_load_lds_dwordx4, explicit s_waitcnt): while
//     the matrix cores work on tap t the next taps are in flight; one barrier
//     per tap. Filter rows lie unpadded in a slot, 16-byte chunks XOR-swizzled
//     by the row (a direct load writes LDS linearly, so the swizzle is applied
//     to the address each lane fetches from);
//   * per tap the K loop is ds_read_b128 + v_mfma over IC / 32 slices, filter
//     first, as in conv_halo.h; requantisation, the optional fused residual
//     add and the copy-out through a wave-private transpose are the same code.
//
// Results are bit for bit those of the implicit-GEMM path.
#ifndef GLOW_MI355X_CONV_HALO_WIDE_H
#define GLOW_MI355X_CONV_HALO_WIDE_H

#include "conv_halo.h"

namespace mi355x {

struct HaloWide {
  const int8_t *in;      // NHWC, IC channels
  const int8_t *filter;  // [OC][3][3][IC]
  int N, IH, IW, OH, OW, OC;
  int padT, padL;
  int rows;              // output rows of an image in a tile (OH when imgs > 1)
  int imgs;              // whole images per tile (1 when a tile is part of an image)
  int tiles_per_image;   // for imgs == 1
  uint32_t fill;         // input offset replicated into four bytes
};

constexpr int kWideMaxPix = 256, kWideBN = 64;
constexpr int kWideParBytes = kParArrays * kWideBN * 4;

template <int IC> struct WideDims {
  static constexpr int kPix = IC + 16;              // bytes between pixels in LDS
  static constexpr int kSlot = kWideBN * IC;        // one tap of the slice, rows unpadded
  static constexpr int kK = 9 * IC;
  // 1 KB load instructions per tap and issuing wave (four waves issue)
  static constexpr int kLoads = IC / 64;
  // slots of the ring: three taps in flight ahead of the multiplies where LDS
  // allows, one for 512 channels (32 KB per tap)
  static constexpr int kSlots = IC == 512 ? 2 : 4;
};
constexpr int kWideMinWaves = 4;

template <int IC>
__global__ __launch_bounds__(512, 2) void conv3x3_halo_wide_kernel(HaloWide cv, Epilogue ep) {
  using D = WideDims<IC>;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int32_t *s_par = reinterpret_cast<int32_t *>(lds);
  int8_t *s_filter = lds + kWideParBytes;                 // the ring of slots
  int8_t *s_halo = s_filter + D::kSlots * D::kSlot;

  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int n0 = blockIdx.y * kWideBN;        // first output channel of the slice

  // the tile: n_imgs images from n_first on, rows output rows of each from oh_first on
  int n_first, oh_first, rows, n_imgs;
  if (cv.imgs == 1) {
    n_first = blockIdx.x / cv.tiles_per_image;
    oh_first = (blockIdx.x - n_first * cv.tiles_per_image) * cv.rows;
    rows = min(cv.rows, cv.OH - oh_first);
    n_imgs = 1;
  } else {
    n_first = blockIdx.x * cv.imgs;
    oh_first = 0;
    rows = cv.OH;
    n_imgs = min(cv.imgs, cv.N - n_first);
  }
  const int per_img = rows * cv.OW;
  const int npix = n_imgs * per_img;
  const int hw = cv.OW + 2;                   // patch pixels per row
  const int prow = rows + 2;                  // patch rows per image
  const int mode = requant_mode(ep);

  // ---- the filter ring: taps 0 .. kSlots - 2 requested first ---------------------------
  // Load instruction j of a tap fills bytes [1024 j, 1024 j + 1024) of a slot:
  // lane i writes slot row s = (1024 j + 16 i) / IC at chunk position cp; what it
  // fetches is chunk cp ^ (s & 7) of the filter row that belongs in slot row s
  // (perm_row16: a lane's sixteen accumulators are sixteen consecutive channels).
  const bool issues = wave < 4;
  const uint32_t ring0 = lds_address(s_filter);
  const int8_t *f_src[D::kLoads];
#pragma unroll
  for (int i = 0; i < D::kLoads; i++) {
    const int j = min(wave, 3) * D::kLoads + i;
    const int byte = j * 1024 + lane * 16;
    const int srow = byte / IC, cp = (byte - srow * IC) >> 4;
    const int c = (srow & ~31) + perm_row16(srow & 31);
    f_src[i] = cv.filter + (long long)(n0 + c) * D::kK + ((cp ^ (srow & 7)) << 4);
  }
  auto request_tap = [&](int t, int slot) {
    if (issues) {
#pragma unroll
      for (int i = 0; i < D::kLoads; i++)
        dma16(f_src[i] + t * IC, ring0 + slot * D::kSlot, (uint32_t)((wave * D::kLoads + i) * 1024));
    }
  };
#pragma unroll
  for (int t = 0; t < D::kSlots - 1; t++) request_tap(t, t);

  // the channels' raw parameters (by the last wave)
  const bool par_wave = wave == (int)(nthreads >> 6) - 1;
  ColRaw col[1];
  if (par_wave) load_col_raw<1, 64>(col, ep, cv.OC, n0, 0, 0, lane);

  // ---- stage the input patch -----------------------------------------------------------
  {
    const int4 fill4 = make_int4((int)cv.fill, (int)cv.fill, (int)cv.fill, (int)cv.fill);
    const int halo_chunks = n_imgs * prow * hw * (IC / 16);
    constexpr int HU = 10;        // all of a 14 x 14 x 256 patch in one round trip
    auto halo_load = [&](int c) -> int4 {
      int4 v = fill4;
      if (c < halo_chunks) {
        const int px = c / (IC / 16), kc = c - px * (IC / 16);
        const int hr = px / hw, hc = px - hr * hw;
        const int il = hr / prow, rr = hr - il * prow;
        const int ih = oh_first - cv.padT + rr, iw = hc - cv.padL;
        if (ih >= 0 && ih < cv.IH && iw >= 0 && iw < cv.IW)
          v = *reinterpret_cast<const int4 *>(
              cv.in + (((long long)(n_first + il) * cv.IH + ih) * cv.IW + iw) * IC + kc * 16);
      }
      return v;
    };
    auto halo_store = [&](int c, const int4 &v) {
      if (c < halo_chunks) {
        const int px = c / (IC / 16), kc = c - px * (IC / 16);
        *reinterpret_cast<int4 *>(s_halo + px * D::kPix + kc * 16) = v;
      }
    };
    for (int base = 0; base < halo_chunks; base += HU * nthreads) {
      int4 hv[HU];
#pragma unroll
      for (int u = 0; u < HU; u++) hv[u] = halo_load(base + tid + u * nthreads);
#pragma unroll
      for (int u = 0; u < HU; u++) halo_store(base + tid + u * nthreads, hv[u]);
    }
  }
  if (par_wave) par_table_store<kWideBN>(s_par, lane, col[0], ep, D::kK, mode);

  // ---- nine taps ------------------------------------------------------------------------
  v16i acc[2];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[j][r] = 0;
  // this lane's pixel (lanes past the tile's end recompute its last pixel; the
  // copy-out does not store them)
  const int p = min(wave * 32 + l32, npix - 1);
  const int il = p / per_img, q = p - il * per_img;
  const int orow = q / cv.OW, ow = q - orow * cv.OW;
  const int8_t *a_base = s_halo + ((il * prow + orow) * hw + ow) * D::kPix + lhi * 16;
  const int row_step = hw * D::kPix;
  const int swz = l32 & 7;
  int slot = 0;                               // of tap t
  for (int t = 0; t < 9; t++) {
    // tap t has landed once only the kSlots - 2 newer requests are pending; the
    // barrier shows it (and, the first time, the patch) to every wave and says
    // that every wave is done with tap t - 1, whose slot the next request takes
    // (towards the end fewer newer requests exist)
    if (8 - t >= D::kSlots - 2) dma_wait<(D::kSlots - 2) * D::kLoads>();
    else if (8 - t == 1) dma_wait<D::kLoads>();
    else dma_wait<0>();
    __syncthreads();
    if (t + D::kSlots - 1 < 9) {
      const int far = slot == 0 ? D::kSlots - 1 : slot - 1;
      request_tap(t + D::kSlots - 1, far);
    }
    const int fx = t / 3, fy = t - fx * 3;
    const int8_t *a_tap = a_base + fx * row_step + fy * D::kPix;
    const int8_t *b_tap = s_filter + slot * D::kSlot + l32 * IC;
    if constexpr (IC == 512) {
      // The fragments of K slice ks + kAhead are asked for before the multiplies
      // of slice ks. Left to itself the compiler reads a slice and waits for it;
      // a 7 x 7 tile of two images is four waves alone on their CU, one to a
      // SIMD, and nothing covers that wait (64 x 7 x 7 x 512: 19.8 -> 18.9 us).
      // With seven waves (14 x 14 x 256, 28 x 28 x 128) the fixed order costs
      // more than it hides (14.5 -> 15.6 us), so those keep the plain loop.
      constexpr int KS = IC / 32, kAhead = 3;
      v4i af[KS], b0[KS], b1[KS];
      auto read_slice = [&](int ks) {
        const int kc = ((ks * 2 + lhi) ^ swz) << 4;
        af[ks] = *reinterpret_cast<const v4i *>(a_tap + ks * 32);
        b0[ks] = *reinterpret_cast<const v4i *>(b_tap + kc);
        b1[ks] = *reinterpret_cast<const v4i *>(b_tap + 32 * IC + kc);
      };
#pragma unroll
      for (int ks = 0; ks < kAhead; ks++) read_slice(ks);
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        if (ks + kAhead < KS) read_slice(ks + kAhead);
        __builtin_amdgcn_sched_barrier(0);
        // filter rows first: the result's rows are channels, its columns pixels
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b0[ks], af[ks], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b1[ks], af[ks], acc[1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < IC / 32; ks++) {
        const v4i af = *reinterpret_cast<const v4i *>(a_tap + ks * 32);
        const int kc = ((ks * 2 + lhi) ^ swz) << 4;
        const v4i b0 = *reinterpret_cast<const v4i *>(b_tap + kc);
        const v4i b1 = *reinterpret_cast<const v4i *>(b_tap + 32 * IC + kc);
        // filter rows first: the result's rows are channels, its columns pixels
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b0, af, acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b1, af, acc[1], 0, 0, 0);
      }
    }
    slot = slot + 1 == D::kSlots ? 0 : slot + 1;
  }
  __syncthreads();
  // every wave has read its pixels: the patch area becomes output staging, and
  // from here on each wave works on its own
  const int m0 = (n_first * cv.OH + oh_first) * cv.OW;
  int8_t *stage = s_halo + wave * (32 * kHaloStageStride);
  if (ep.act == 5) halo_finish<0, true>(acc, s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
  else if (mode == 3) halo_finish<3, false>(acc, s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
  else if (mode == 1) halo_finish<1, false>(acc, s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
  else halo_finish<0, false>(acc, s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
}

// The tiling for this geometry: fills rows / imgs / tiles_per_image of cv and
// returns the number of waves per workgroup, or 0 when the shape is not the
// kernel's own; lds receives the dynamic LDS a block needs.
static int conv_halo_wide_plan(const mi355x_conv_geom *g, size_t lds_max, HaloWide &cv, size_t &lds) {
  if (g->KH != 3 || g->KW != 3 || g->strideH != 1 || g->strideW != 1 || g->dilH != 1 ||
      g->dilW != 1 || g->group != 1 || g->OC % kWideBN != 0)
    return 0;
  if (g->IC != 128 && g->IC != 256 && g->IC != 512) return 0;
  if (g->OH <= 0 || g->OW <= 0 || g->OW > kWideMaxPix || g->N <= 0) return 0;
  const size_t pix = (size_t)g->IC + 16;
  const size_t fixed = kWideParBytes + (size_t)(g->IC == 512 ? 2 : 4) * kWideBN * g->IC;
  auto need = [&](int imgs, int rows) {
    const size_t patch = (size_t)imgs * (rows + 2) * (g->OW + 2) * pix;
    const size_t stage = (size_t)((imgs * rows * g->OW + 31) / 32) * 32 * kHaloStageStride;
    return fixed + (patch > stage ? patch : stage);
  };
  int imgs = 1, rows;
  const int per_img = g->OH * g->OW;
  if (per_img <= kWideMaxPix / 2) {
    // small images: as many whole ones as fit the pixel budget and LDS
    rows = g->OH;
    imgs = kWideMaxPix / per_img;
    if (imgs > g->N) imgs = g->N;
    while (imgs > 1 && need(imgs, rows) > lds_max) imgs--;
  } else {
    // rows of one image: the fewest tiles of at most 256 pixels, evenly sized
    int most = kWideMaxPix / g->OW;
    if (most > g->OH) most = g->OH;
    while (most > 1 && need(1, most) > lds_max) most--;
    const int tiles = (g->OH + most - 1) / most;
    rows = (g->OH + tiles - 1) / tiles;
  }
  if (need(imgs, rows) > lds_max) return 0;
  const int waves = (imgs * rows * g->OW + 31) / 32;
  // four waves load the filter taps
  if (waves < kWideMinWaves) return 0;
  cv.rows = rows;
  cv.imgs = imgs;
  cv.tiles_per_image = (g->OH + rows - 1) / rows;
  lds = need(imgs, rows);
  return waves;
}

template <int IC>
static int conv_halo_wide_launch_ic(const HaloWide &cv, const Epilogue &ep, size_t lds, size_t lds_max,
                                    int waves, unsigned tiles, hipStream_t st) {
  static std::atomic<uint64_t> attr_set{0};
  // the attribute is set once per device: to the most the device allows
  int rc = set_lds_attr(conv3x3_halo_wide_kernel<IC>, lds_max, attr_set);
  if (rc != MI355X_OK) return rc;
  hipLaunchKernelGGL(conv3x3_halo_wide_kernel<IC>, dim3(tiles, (unsigned)(cv.OC / kWideBN)),
                     dim3(64 * waves), lds, st, cv, ep);
  return check_launch("conv3x3_halo_wide");
}

static int conv_halo_wide_launch(const int8_t *in, const int8_t *filter, const mi355x_conv_geom *g,
                                 const Epilogue &ep, HaloWide cv, size_t lds, size_t lds_max,
                                 int waves, hipStream_t st) {
  cv.in = in;
  cv.filter = filter;
  cv.N = g->N; cv.IH = g->IH; cv.IW = g->IW; cv.OH = g->OH; cv.OW = g->OW; cv.OC = g->OC;
  cv.padT = g->padT; cv.padL = g->padL;
  const long long tiles = cv.imgs == 1 ? (long long)g->N * cv.tiles_per_image
                                       : ((long long)g->N + cv.imgs - 1) / cv.imgs;
  MI355X_REQUIRE(tiles < 0x7fffffffLL && (long long)g->N * g->OH * g->OW < 0x7fffffffLL &&
                     (long long)g->OC / kWideBN < 65536,
                 "problem too large");
  cv.fill = 0x01010101u * (uint32_t)(uint8_t)(int8_t)ep.a_off;
  switch (g->IC) {
  case 128: return conv_halo_wide_launch_ic<128>(cv, ep, lds, lds_max, waves, (unsigned)tiles, st);
  case 256: return conv_halo_wide_launch_ic<256>(cv, ep, lds, lds_max, waves, (unsigned)tiles, st);
  default: return conv_halo_wide_launch_ic<512>(cv, ep, lds, lds_max, waves, (unsigned)tiles, st);
  }
}

} // namespace mi355x
#endif
