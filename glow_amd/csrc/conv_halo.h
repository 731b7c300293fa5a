// 3x3, stride-1 convolution over 64 input channels (the first-stage layers of
// an image network; reference lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:49-239)
// with the operands held in LDS the way the matrix cores want them, instead
// of the implicit-GEMM gather of gemm_i8.h:
//
//   * the filter slice of a workgroup (64 output channels x 576 bytes, 37 KB)
//     is loaded once and stays in LDS while the workgroup walks over output
//     tiles (persistent workgroups, tiles taken round-robin);
//   * per tile of 128 consecutive output pixels of one image, the input rows
//     those pixels need (at most six rows of 58 pixels for a 56x56 image,
//     padding columns and rows materialised as input-offset bytes) are staged
//     once: every input byte is read from memory once per tile instead of once
//     per tap;
//   * the nine taps are then LDS address arithmetic: a lane's fragment of tap
//     (fx, fy) sits a constant distance from its pixel's base address, so the
//     K loop is ds_read_b128 + v_mfma with nothing else in it.
//
// Pixels and filter rows are 16 bytes apart from a power-of-two stride in LDS
// (80 and 592 bytes), which spreads the 16-byte fragment reads of consecutive
// rows over all banks. A wave owns 32 pixels x 64 channels (two 32x32x32
// accumulator tiles), four waves a tile. The epilogue is the shared one of
// gemm_i8.h (requantisation, activation, optional fused residual add).
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
  int N, IH, IW, OH, OW, OC;
  int padT, padL;
  int tiles_per_image, total_tiles;
  int halo_rows;         // LDS rows reserved: rows a tile can span + 2
  uint32_t fill;         // input offset replicated into four bytes
};

constexpr int kHaloBM = 128, kHaloBN = 64, kHaloIC = 64, kHaloK = 9 * kHaloIC;
constexpr int kHaloPix = kHaloIC + 16;        // bytes between pixels in LDS
constexpr int kHaloFRow = kHaloK + 16;        // bytes between filter rows in LDS
constexpr int kHaloFilterBytes = kHaloBN * kHaloFRow;

__global__ __launch_bounds__(256, 2) void conv3x3_halo_kernel(HaloConv cv, Epilogue ep) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int8_t *s_filter = lds;
  int8_t *s_halo = lds + kHaloFilterBytes;    // also the epilogue's staging area

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int n0 = blockIdx.y * kHaloBN;        // first output channel of the slice

  // the epilogue's per-column parameters, requested first
  ColRaw col[2];
  load_col_raw<2, 64>(col, ep, cv.OC, n0, 0, 0, l32);

  // filter slice -> LDS, once
  {
    constexpr int kChunks = kHaloBN * (kHaloK / 16);   // 16-byte chunks
    const int8_t *f = cv.filter + (long long)n0 * kHaloK;
#pragma unroll
    for (int i = 0; i < (kChunks + 255) / 256; i++) {
      const int c = tid + i * 256;
      if (c < kChunks) {
        const int row = c / (kHaloK / 16), kc = c - row * (kHaloK / 16);
        *reinterpret_cast<int4 *>(s_filter + row * kHaloFRow + kc * 16) =
            *reinterpret_cast<const int4 *>(f + (long long)row * kHaloK + kc * 16);
      }
    }
  }

  const int hw = cv.OW + 2;                    // halo pixels per row
  const int pix_per_image = cv.OH * cv.OW;
  const int4 fill4 = make_int4((int)cv.fill, (int)cv.fill, (int)cv.fill, (int)cv.fill);
  // where this lane's B fragments start: filter row l32 (+32 for the second
  // column tile), k-bytes lhi*16..
  const int b_base = l32 * kHaloFRow + lhi * 16;

  for (int t = blockIdx.x; t < cv.total_tiles; t += gridDim.x) {
    const int n = t / cv.tiles_per_image;
    const int p0 = (t - n * cv.tiles_per_image) * kHaloBM;
    const int npix = min(kHaloBM, pix_per_image - p0);
    const int oh_first = p0 / cv.OW;
    const int oh_last = (p0 + npix - 1) / cv.OW;
    const int hrows = oh_last - oh_first + 3;

    __syncthreads();   // the previous tile's copy-out has left the staging area
    // ---- stage the input rows of this tile ------------------------------------
    {
      const int total = hrows * hw * (kHaloIC / 16);
      const int8_t *img = cv.in + (long long)n * cv.IH * cv.IW * kHaloIC;
      for (int base = 0; base < total; base += 256 * 8) {
        int4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int c = base + tid + u * 256;
          v[u] = fill4;
          if (c < total) {
            const int px = c >> 2, kc = c & 3;
            const int hr = px / hw, hc = px - hr * hw;
            const int ih = oh_first - cv.padT + hr, iw = hc - cv.padL;
            if (ih >= 0 && ih < cv.IH && iw >= 0 && iw < cv.IW)
              v[u] = *reinterpret_cast<const int4 *>(
                  img + ((long long)ih * cv.IW + iw) * kHaloIC + kc * 16);
          }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int c = base + tid + u * 256;
          if (c < total) {
            const int px = c >> 2, kc = c & 3;
            *reinterpret_cast<int4 *>(s_halo + px * kHaloPix + kc * 16) = v[u];
          }
        }
      }
    }
    __syncthreads();

    // ---- nine taps x two 32-byte k slices ---------------------------------------
    v16i acc[1][2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[0][j][r] = 0;
    {
      // this lane's pixel (lanes past the tile's end recompute its last pixel;
      // the epilogue does not store them)
      const int p = p0 + min(wave * 32 + l32, npix - 1);
      const int oh = p / cv.OW, ow = p - oh * cv.OW;
      const int8_t *a_base = s_halo + ((oh - oh_first) * hw + ow) * kHaloPix + lhi * 16;
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
            const v4i b0 = *reinterpret_cast<const v4i *>(s_filter + b_base + kb);
            const v4i b1 =
                *reinterpret_cast<const v4i *>(s_filter + b_base + 32 * kHaloFRow + kb);
            acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, b1, acc[0][1], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();   // every wave has read its halo: the area becomes staging

    int sa[1] = {0}, sb[2] = {0, 0};
    const int m0 = n * pix_per_image + p0;
    // rows past the tile's end belong to the next tile (or image): M bounds them
    gemm_epilogue<kHaloBM, kHaloBN, 32, 64, false, false>(acc, sa, sb, s_halo, ep, m0 + npix,
                                                          cv.OC, kHaloK, m0, n0, 0, col);
  }
}

// LDS the kernel needs for this geometry, or 0 when the shape is not its own.
static size_t conv_halo_lds_bytes(const mi355x_conv_geom *g, int &halo_rows) {
  if (g->KH != 3 || g->KW != 3 || g->strideH != 1 || g->strideW != 1 || g->dilH != 1 ||
      g->dilW != 1 || g->group != 1 || g->IC != kHaloIC || g->OC % kHaloBN != 0)
    return 0;
  if (g->OH <= 0 || g->OW <= 0) return 0;
  // rows that 128 consecutive pixels of one image can touch
  int rows = (kHaloBM + g->OW - 2) / g->OW + 1;
  if (rows > g->OH) rows = g->OH;
  halo_rows = rows + 2;
  const size_t halo = (size_t)halo_rows * (g->OW + 2) * kHaloPix;
  const size_t epi = gemm_epilogue_lds_bytes<kHaloBM, kHaloBN>();
  return kHaloFilterBytes + (halo > epi ? halo : epi);
}

static int conv_halo_launch(const int8_t *in, const int8_t *filter, const mi355x_conv_geom *g,
                            const Epilogue &ep, size_t lds, int halo_rows, hipStream_t st) {
  HaloConv cv;
  cv.in = in;
  cv.filter = filter;
  cv.N = g->N; cv.IH = g->IH; cv.IW = g->IW; cv.OH = g->OH; cv.OW = g->OW; cv.OC = g->OC;
  cv.padT = g->padT; cv.padL = g->padL;
  cv.tiles_per_image = (g->OH * g->OW + kHaloBM - 1) / kHaloBM;
  const long long total = (long long)g->N * cv.tiles_per_image;
  MI355X_REQUIRE(total < 0x7fffffffLL, "problem too large");
  cv.total_tiles = (int)total;
  cv.halo_rows = halo_rows;
  cv.fill = 0x01010101u * (uint32_t)(uint8_t)(int8_t)ep.a_off;
  static std::atomic<uint64_t> attr_set{0};
  int rc = set_lds_attr(conv3x3_halo_kernel, lds, attr_set);
  if (rc != MI355X_OK) return rc;
  // persistent workgroups: as many as stay resident (two per CU while the LDS
  // allows), fewer when there are fewer tiles
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
  }
  const int slices = g->OC / kHaloBN;
  const int per_cu = lds * 2 <= 160 * 1024 ? 2 : 1;
  long long gx = (long long)cus * per_cu / slices;
  if (gx < 1) gx = 1;
  if (gx > total) gx = total;
  hipLaunchKernelGGL(conv3x3_halo_kernel, dim3((unsigned)gx, (unsigned)slices), dim3(256), lds, st,
                     cv, ep);
  return check_launch("conv3x3_halo");
}

} // namespace mi355x
#endif
