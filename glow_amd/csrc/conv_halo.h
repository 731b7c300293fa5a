// 3x3, stride-1 convolution over 64 input channels (the first-stage layers of
// an image network; reference lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:49-239)
// with the operands held in LDS the way the matrix cores want them, instead
// of the implicit-GEMM gather of gemm_i8.h:
//
//   * a workgroup computes a tile of whole output rows of one image (as many
//     rows as give at most 256 pixels: four rows of a 56-wide image) for 64
//     output channels, one wave per 32 consecutive pixels, so the block size
//     follows the image (seven waves for 4 x 56 pixels);
//   * the filter slice (64 output channels x 576 bytes, 37 KB) and the input
//     rows the tile needs (its rows plus one above and below, one pixel left
//     and right; padding materialised as input-offset bytes) are staged in LDS
//     once, all loads of a thread in flight together: every input byte is read
//     from memory once per tile instead of once per tap;
//   * the nine taps are then LDS address arithmetic: a lane's fragment of tap
//     (fx, fy) sits a constant distance from its pixel's base address, so the
//     K loop is ds_read_b128 + v_mfma with nothing else in it;
//   * the filter is the first matrix-core operand and its rows are placed in LDS
//     in such an order that a lane's sixteen accumulators of a channel tile are
//     sixteen consecutive channels of one pixel: they are requantised and
//     packed in registers, and leave through a wave-private transpose in the
//     (by then free) halo area, so that whole 64-byte pixels are stored (stores
//     of 16-byte pieces straight from registers wrote 1.5 x the bytes at the
//     memory side).
//
// Pixels and filter rows are 16 bytes apart from a power-of-two stride in LDS
// (80 and 592 bytes), which spreads the 16-byte fragment reads of consecutive
// rows over all banks. The arithmetic is that of the shared epilogue of
// gemm_i8.h (requantisation, activation, the optional fused residual add).
//
// Padded taps hold the input offset, so (in - inOffset) contributes zero for
// them exactly as the CPU loop's skipped taps do; the results are bit for bit
// those of the implicit-GEMM path.
#ifndef GLOW_MI355X_CONV_HALO_H
#define GLOW_MI355X_CONV_HALO_H

#include "gemm_i8.h"

namespace mi355x {

struct HaloConv {
  const int8_t *in;      // NHWC, 64 channels
  const int8_t *filter;  // [OC][3][3][64]
  int IH, IW, OH, OW, OC;
  int padT, padL;
  int rows;              // output rows per tile
  int tiles_per_image;
  uint32_t fill;         // input offset replicated into four bytes
};

constexpr int kHaloMaxPix = 256, kHaloBN = 64, kHaloIC = 64, kHaloK = 9 * kHaloIC;
constexpr int kHaloPix = kHaloIC + 16;        // bytes between pixels in LDS
constexpr int kHaloFRow = kHaloK + 16;        // bytes between filter rows in LDS
constexpr int kHaloFilterBytes = kHaloBN * kHaloFRow;
// (rows + 2) x (OW + 2) pixels with rows * OW <= 256 is largest for one row of 256
constexpr size_t kHaloMaxLds =
    kHaloFilterBytes + 5 * kHaloBN * 4 + (size_t)3 * (kHaloMaxPix + 2) * kHaloPix;   // > 8 staging tiles
constexpr int kHaloFilterChunks = kHaloBN * (kHaloK / 16);   // 16-byte chunks

// Filter row (output channel) c of a workgroup's 64 sits in LDS slot
// perm_slot16(c): lane (pixel, h) then holds channels 32 j + 16 h + [0, 16) of
// its pixel in the sixteen accumulators of tile j, in order (see gemm_i8.h).
constexpr int kHaloParBytes = kParArrays * kHaloBN * 4;

// Requantises a wave's 32 pixels x 64 channels and writes them as whole rows
// through its staging tile (gemm_i8.h: requant_pack16, wave_rows_copy_out).
constexpr int kHaloStageStride = kHaloBN + 16;
// Copy-out of one staged block of 32 pixels x 64 channels: eight consecutive
// lanes read the same 16-byte piece of eight consecutive pixels (eight
// different bank groups at the 80-byte stride; four lanes per pixel put every
// second pixel's piece on the banks of the one before), and a wave's store
// instruction still covers sixteen whole pixels of 64 bytes.
__device__ __forceinline__ void halo_rows_copy_out(const int8_t *s_stage, int lane, int m0, int M,
                                                   int col0, const Epilogue &ep,
                                                   const FusedAddConsts &fc, bool fast) {
  const int seg = (lane >> 3) & 3;
  const int row_in_pass = (lane & 7) + 8 * (lane >> 5);
#pragma unroll
  for (int r0 = 0; r0 < 32; r0 += 16) {
    const int row = r0 + row_in_pass, m = m0 + row;
    if (m < M) {
      int4 v = *reinterpret_cast<const int4 *>(s_stage + row * kHaloStageStride + seg * 16);
      const long long at = (long long)m * ep.ldc + col0 + seg * 16;
      v = fused_out_words(v, ep.add.res ? ep.add.res + at : nullptr, ep, fc, fast);
      *reinterpret_cast<int4 *>(ep.out + at) = v;
    }
  }
}

template <int MODE, bool LEAKY>
__device__ __forceinline__ void halo_finish(const v16i (&acc)[2], const int32_t *s_par,
                                            int8_t *stage, const Epilogue &ep, int lane, int m0,
                                            int M, int n0) {
  const int l32 = lane & 31, lhi = lane >> 5;
  int32_t lo, hi;
  activation_clamp(ep, lo, hi);
  const bool fast = fused_out_is_fast(ep);
  const FusedAddConsts fc = fused_add_consts(ep.add);
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int cl = 32 * j + 16 * lhi;
    const int4 v = requant_pack16<MODE, LEAKY, kHaloBN>(acc[j], s_par + cl, ep, lo, hi);
    *reinterpret_cast<int4 *>(stage + l32 * kHaloStageStride + cl) = v;
  }
  wave_fence();
  halo_rows_copy_out(stage, lane, m0, M, n0, ep, fc, fast);
}

// SKIP leaves phases out so that the others can be timed (1: staging, 2: the
// matrix-core loop, 4: requantisation and copy-out); the library uses 0.
template <int SKIP = 0>
__global__ __launch_bounds__(512, 2) void conv3x3_halo_kernel(HaloConv cv, Epilogue ep) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int8_t *s_filter = lds;
  int32_t *s_par = reinterpret_cast<int32_t *>(lds + kHaloFilterBytes);
  int8_t *s_halo = lds + kHaloFilterBytes + kHaloParBytes;

  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int n0 = blockIdx.y * kHaloBN;        // first output channel of the slice

  const int n = blockIdx.x / cv.tiles_per_image;
  const int oh_first = (blockIdx.x - n * cv.tiles_per_image) * cv.rows;
  const int rows = min(cv.rows, cv.OH - oh_first);
  const int npix = rows * cv.OW;
  const int hw = cv.OW + 2;                   // halo pixels per row
  const int mode = requant_mode(ep);

  // the channels' raw parameters are requested by the last wave (the first
  // ones carry the staging loop's remainders), behind its share of the staging
  // loads: in front of them their address arithmetic (ten optional arrays)
  // would hold back loads the whole workgroup waits for at the barrier
  const bool par_wave = wave == (int)(nthreads >> 6) - 1;
  ColRaw col[1];

  // ---- stage the tile's input rows and the filter slice -------------------------
  if constexpr (!(SKIP & 1)) {
    const int4 fill4 = make_int4((int)cv.fill, (int)cv.fill, (int)cv.fill, (int)cv.fill);
    const int8_t *img = cv.in + (long long)n * cv.IH * cv.IW * kHaloIC;
    const int8_t *f = cv.filter + (long long)n0 * kHaloK;
    const int halo_pixels = (rows + 2) * hw;
    const float inv_hw = __frcp_rn((float)hw);
    // work items of the halo: 32 per group of eight pixels
    const int halo_chunks = ((halo_pixels + 7) >> 3) * 32;
    constexpr int HU = 4, FU = 6;
    // item c of the halo: pixel 8 (c / 32) + c % 8 of the (rows + 2) x hw patch,
    // bytes 16 * ((c / 8) % 4) of its channels. Eight consecutive lanes then
    // store the same 16-byte piece of eight consecutive pixels, 80 bytes apart:
    // eight different bank groups (four lanes per pixel, the plain order, put
    // the piece of every second pixel on the banks of the one before).
    auto halo_load = [&](int c) -> int4 {
      int4 v = fill4;
      const int px = ((c >> 5) << 3) + (c & 7), kc = (c >> 3) & 3;
      if (px < halo_pixels) {
        // px / hw for px < 4096 and hw >= 3 in three instructions: the error
        // of the product is below 4096 * 2^-22, the margin 0.5 / hw
        const int hr = (int)(((float)px + 0.5f) * inv_hw), hc = px - hr * hw;
        const int ih = oh_first - cv.padT + hr, iw = hc - cv.padL;
        if (ih >= 0 && ih < cv.IH && iw >= 0 && iw < cv.IW)
          v = *reinterpret_cast<const int4 *>(img + ((long long)ih * cv.IW + iw) * kHaloIC +
                                              kc * 16);
      }
      return v;
    };
    auto halo_store = [&](int c, const int4 &v) {
      const int px = ((c >> 5) << 3) + (c & 7), kc = (c >> 3) & 3;
      if (px < halo_pixels) *reinterpret_cast<int4 *>(s_halo + px * kHaloPix + kc * 16) = v;
    };
    auto filter_load = [&](int c) -> int4 {
      int4 v = fill4;
      if (c < kHaloFilterChunks) {
        const int row = c / (kHaloK / 16), kc = c - row * (kHaloK / 16);
        v = *reinterpret_cast<const int4 *>(f + (long long)row * kHaloK + kc * 16);
      }
      return v;
    };
    auto filter_store = [&](int c, const int4 &v) {
      if (c < kHaloFilterChunks) {
        const int row = c / (kHaloK / 16), kc = c - row * (kHaloK / 16);
        *reinterpret_cast<int4 *>(s_filter + perm_slot16(row) * kHaloFRow + kc * 16) = v;
      }
    };
    // first batch of both in flight together
    int4 hv[HU], fv[FU];
#pragma unroll
    for (int u = 0; u < HU; u++) hv[u] = halo_load(tid + u * nthreads);
#pragma unroll
    for (int u = 0; u < FU; u++) fv[u] = filter_load(tid + u * nthreads);
    if constexpr (SKIP == 0) {
      __builtin_amdgcn_sched_barrier(0);
      if (par_wave) load_col_raw<1, 64>(col, ep, cv.OC, n0, 0, 0, lane);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int u = 0; u < HU; u++) halo_store(tid + u * nthreads, hv[u]);
#pragma unroll
    for (int u = 0; u < FU; u++) filter_store(tid + u * nthreads, fv[u]);
    for (int base = HU * nthreads; base < halo_chunks; base += HU * nthreads) {
#pragma unroll
      for (int u = 0; u < HU; u++) hv[u] = halo_load(base + tid + u * nthreads);
#pragma unroll
      for (int u = 0; u < HU; u++) halo_store(base + tid + u * nthreads, hv[u]);
    }
    for (int base = FU * nthreads; base < kHaloFilterChunks; base += FU * nthreads) {
#pragma unroll
      for (int u = 0; u < FU; u++) fv[u] = filter_load(base + tid + u * nthreads);
#pragma unroll
      for (int u = 0; u < FU; u++) filter_store(base + tid + u * nthreads, fv[u]);
    }
  }

  if constexpr (SKIP != 0) {
    if (par_wave) load_col_raw<1, 64>(col, ep, cv.OC, n0, 0, 0, lane);
  }
  // ---- the channels' requantisation constants -> LDS --------------------------------
  if (par_wave) par_table_store<kHaloBN>(s_par, lane, col[0], ep, kHaloK, mode);
  __syncthreads();

  // ---- nine taps x two 32-byte k slices -------------------------------------------
  v16i acc[1][2];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[0][j][r] = (SKIP & 2) ? tid + r : 0;
  if constexpr (!(SKIP & 2)) {
    // this lane's pixel (lanes past the tile's end recompute its last pixel;
    // the copy-out does not store them)
    const int p = min(wave * 32 + l32, npix - 1);
    const int orow = p / cv.OW, ow = p - orow * cv.OW;
    const int8_t *a_base = s_halo + (orow * hw + ow) * kHaloPix + lhi * 16;
    // this lane's filter slot l32 (+32 for the second channel tile), k-bytes lhi*16..
    const int8_t *b_base = s_filter + l32 * kHaloFRow + lhi * 16;
    const int row_step = hw * kHaloPix;
#pragma unroll
    for (int fx = 0; fx < 3; fx++) {
#pragma unroll
      for (int fy = 0; fy < 3; fy++) {
#pragma unroll
        for (int ks = 0; ks < kHaloIC / 32; ks++) {
          const v4i af = *reinterpret_cast<const v4i *>(a_base + fx * row_step +
                                                        fy * kHaloPix + ks * 32);
          const int kb = (fx * 3 + fy) * kHaloIC + ks * 32;
          const v4i b0 = *reinterpret_cast<const v4i *>(b_base + kb);
          const v4i b1 = *reinterpret_cast<const v4i *>(b_base + 32 * kHaloFRow + kb);
          // filter rows first: the result's rows are channels, its columns pixels
          acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b0, af, acc[0][0], 0, 0, 0);
          acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b1, af, acc[0][1], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();   // every wave has read its halo: the area becomes output staging

  // from here on each wave works on its own 32 pixels
  if constexpr (!(SKIP & 4)) {
    // rows past the tile's end belong to the next tile (or image): M bounds them
    const int m0 = (n * cv.OH + oh_first) * cv.OW;
    int8_t *stage = s_halo + wave * (32 * kHaloStageStride);
    if (ep.act == 5) halo_finish<0, true>(acc[0], s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
    else if (mode == 3) halo_finish<3, false>(acc[0], s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
    else if (mode == 1) halo_finish<1, false>(acc[0], s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
    else halo_finish<0, false>(acc[0], s_par, stage, ep, lane, m0 + wave * 32, m0 + npix, n0);
  } else {
    int x = 0;
#pragma unroll
    for (int r = 0; r < 16; r++) x += acc[0][0][r] ^ acc[0][1][r];
    if (x == 0x12345678) ep.out[tid] = (int8_t)x;
  }
}

// Output rows per tile for this geometry, or 0 when the shape is not the
// kernel's own; lds receives the dynamic LDS a block needs.
static int conv_halo_rows(const mi355x_conv_geom *g, int cus, size_t &lds) {
  if (g->KH != 3 || g->KW != 3 || g->strideH != 1 || g->strideW != 1 || g->dilH != 1 ||
      g->dilW != 1 || g->group != 1 || g->IC != kHaloIC || g->OC % kHaloBN != 0)
    return 0;
  if (g->OH <= 0 || g->OW <= 0 || g->OW > kHaloMaxPix) return 0;
  int rows = kHaloMaxPix / g->OW;
  if (rows > g->OH) rows = g->OH;
  // fewer rows per tile while that gives the chip more tiles than CUs and a
  // tile keeps at least a wave's worth of pixels
  const long long slices = g->OC / kHaloBN;
  while (rows > 1 && (long long)g->N * ((g->OH + rows - 1) / rows) * slices < cus &&
         (rows - 1) * g->OW >= 32)
    rows--;
  const size_t halo = (size_t)(rows + 2) * (g->OW + 2) * kHaloPix;
  const size_t stage = (size_t)((rows * g->OW + 31) / 32) * 32 * kHaloStageStride;
  lds = kHaloFilterBytes + kHaloParBytes + (halo > stage ? halo : stage);
  return rows;
}

static int conv_halo_launch(const int8_t *in, const int8_t *filter, const mi355x_conv_geom *g,
                            const Epilogue &ep, size_t lds, int rows, hipStream_t st) {
  HaloConv cv;
  cv.in = in;
  cv.filter = filter;
  cv.IH = g->IH; cv.IW = g->IW; cv.OH = g->OH; cv.OW = g->OW; cv.OC = g->OC;
  cv.padT = g->padT; cv.padL = g->padL;
  cv.rows = rows;
  cv.tiles_per_image = (g->OH + rows - 1) / rows;
  const long long total = (long long)g->N * cv.tiles_per_image;
  MI355X_REQUIRE(total < 0x7fffffffLL && (long long)g->N * g->OH * g->OW < 0x7fffffffLL,
                 "problem too large");
  cv.fill = 0x01010101u * (uint32_t)(uint8_t)(int8_t)ep.a_off;
  static std::atomic<uint64_t> attr_set{0};
  // the attribute is set once per device: to the most any geometry can ask for
  int rc = set_lds_attr(conv3x3_halo_kernel<0>, kHaloMaxLds, attr_set);
  if (rc != MI355X_OK) return rc;
  const int waves = (rows * g->OW + 31) / 32;
  hipLaunchKernelGGL(conv3x3_halo_kernel<0>, dim3((unsigned)total, (unsigned)(g->OC / kHaloBN)),
                     dim3(64 * waves), lds, st, cv, ep);
  return check_launch("conv3x3_halo");
}

static int device_cus() {
  int dev = 0, v = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
    return v;
  return 256;
}

} // namespace mi355x
#endif
