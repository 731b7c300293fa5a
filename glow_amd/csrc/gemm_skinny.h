// The int8 contraction for outputs too small to fill the chip with 64x64
// tiles (a FullyConnected over a small batch): 32x32 output tiles, and the K
// loop of a tile split over the four waves of its workgroup, so that a
// 128 x 1024 result runs on 128 workgroups of four waves instead of 32.
//
// A wave takes every fourth 32-byte K step. Its operand fragments go from
// global memory straight into registers in the matrix-core layout (lane l
// feeds 16 consecutive k-bytes of row l % 32; no LDS staging: each byte is
// used by one wave only), all loads of a chunk of steps in flight before the
// first multiply. The four partial 32x32 accumulators meet in LDS; each wave
// then finishes a quarter of the tile (8 of its 32 rows) and writes it.
// int32 partial sums add in any order to the same bits, so the result is that
// of the unsplit loop.
//
// Handles what the rowwise FullyConnected of a trained network has: 16-byte
// aligned rows, K a multiple of 32, weight offsets all zero and weight row
// sums precomputed (no in-kernel row sums). Everything else stays on the
// tiled kernels.
#ifndef GLOW_MI355X_GEMM_SKINNY_H
#define GLOW_MI355X_GEMM_SKINNY_H

#include "gemm_i8.h"

namespace mi355x {

constexpr int kSkinnyChunk = 8;   // K steps a wave has in flight at a time

template <int FAST>
__device__ __forceinline__ int32_t skinny_requant(uint32_t acc, uint32_t colc, int32_t opre,
                                                  int32_t opost, int32_t oscale, uint32_t fold,
                                                  int32_t out_off) {
  if constexpr (FAST == 2) {
    return (int32_t)((uint32_t)__mul24((int32_t)acc, oscale) + fold) >> opost;
  } else if constexpr (FAST == 1) {
    return (int32_t)((uint32_t)__mul24((int32_t)(acc + colc) >> opre, oscale) + fold) >> opost;
  } else {
    return scale_i32((int32_t)(acc + colc), opre, opost, oscale, out_off);
  }
}

__global__ __launch_bounds__(256, 2) void gemm_i8_skinny_kernel(DenseRows A, DenseRows B,
                                                                Epilogue ep, int M, int N,
                                                                int K, int tiles_n) {
  __shared__ int32_t s_part[4][16][64];   // [wave][accumulator register][lane]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x - tm * tiles_n;
  const int m0 = tm * 32, n0 = tn * 32;

  // rows past the end re-read the last row; their results are not stored
  const int8_t *arow = A.p + (long long)min(m0 + l32, M - 1) * A.ld + lhi * 16;
  const int8_t *brow = B.p + (long long)min(n0 + l32, N - 1) * B.ld + lhi * 16;

  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0;

  const int steps = K / 32;                       // 32-byte K steps in all
  // wave w takes steps w, w + 4, w + 8, ..., kSkinnyChunk of them in flight at
  // a time
  v4i af[kSkinnyChunk], bf[kSkinnyChunk];
  auto request = [&](int base) {
#pragma unroll
    for (int u = 0; u < kSkinnyChunk; u++) {
      // steps past the end re-read the last step of this wave and are not used
      const int s = min(base + 4 * u, steps - 1);
      af[u] = *reinterpret_cast<const v4i *>(arow + s * 32);
      bf[u] = *reinterpret_cast<const v4i *>(brow + s * 32);
    }
  };
  int base = wave;
  request(base);
  // The epilogue's per-column parameters of this lane's column are asked for
  // behind the first operands: their ten optional arrays are some two hundred
  // instructions of address arithmetic and null checks, which in front of the
  // operand loads is time the whole launch waits (it is a few microseconds
  // long), and behind them runs while the operands are on their way.
  __builtin_amdgcn_sched_barrier(0);
  ColRaw col[1];
  load_col_raw<1, 32>(col, ep, N, n0, 0, 0, l32);
  __builtin_amdgcn_sched_barrier(0);
  while (true) {
#pragma unroll
    for (int u = 0; u < kSkinnyChunk; u++)
      if (base + 4 * u < steps)
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[u], bf[u], acc, 0, 0, 0);
    base += 4 * kSkinnyChunk;
    if (base >= steps) break;
    request(base);
  }

  // the four partial tiles meet in LDS
#pragma unroll
  for (int r = 0; r < 16; r++) s_part[wave][r][lane] = acc[r];
  __syncthreads();

  // wave w finishes accumulator registers 4w..4w+3: rows 8w + 4*(l/32) + 0..3
  const int32_t woff = col[0].woff;
  const int32_t opre = col[0].opre, opost = col[0].opost, oscale = col[0].oscale;
  uint32_t colc = (uint32_t)K * (uint32_t)ep.a_off * (uint32_t)woff;
  if (ep.sum_b) colc -= (uint32_t)ep.a_off * (uint32_t)col[0].sumb;
  if (ep.bias)
    colc += (uint32_t)scale_i32((int32_t)((uint32_t)col[0].bias - (uint32_t)col[0].boff),
                                col[0].bpre, col[0].bpost, col[0].bscale, 0);
  int32_t lo = -128, hi = 127;
  if (ep.act == 1) lo = clip_i8(ep.out_off);
  if (ep.act == 2) {
    lo = clip_i8(ep.a0);
    hi = clip_i8(ep.a1);
    if (lo > hi) lo = hi;
  }
  uint32_t fold = (opost > 0 ? (1u << (opost - 1)) : 0u) + ((uint32_t)ep.out_off << opost);
  const int fast = ep.act == 5 ? 0 : ep.fast & 3;
  if (fast == 3) fold += colc * (uint32_t)oscale;

  const int n = n0 + l32;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int r = wave * 4 + q;
    const uint32_t sum = (uint32_t)s_part[0][r][lane] + (uint32_t)s_part[1][r][lane] +
                         (uint32_t)s_part[2][r][lane] + (uint32_t)s_part[3][r][lane];
    int32_t y;
    if (fast == 3) y = skinny_requant<2>(sum, colc, opre, opost, oscale, fold, ep.out_off);
    else if (fast == 1) y = skinny_requant<1>(sum, colc, opre, opost, oscale, fold, ep.out_off);
    else y = skinny_requant<0>(sum, colc, opre, opost, oscale, fold, ep.out_off);
    if (ep.act == 5 && y < ep.out_off)
      y = scale_i32((int32_t)((uint32_t)y - (uint32_t)ep.out_off), ep.a0, ep.a1, ep.a2, ep.out_off);
    int32_t v = med3_i32(y, lo, hi);
    if (ep.add.relu && !ep.add.res) {
      // the Relu stage alone (a Relu instruction behind the FullyConnected)
      const uint32_t w = ep.add.small ? fused_relu_word_t<true>((uint32_t)v & 0xff, ep.add)
                                      : fused_relu_word_t<false>((uint32_t)v & 0xff, ep.add);
      v = (int32_t)(int8_t)w;
    }
    const int m = m0 + wave * 8 + lhi * 4 + q;
    if (m < M && n < N) ep.out[(long long)m * ep.ldc + n] = (int8_t)v;
  }
}

// Whether the skinny kernel takes this product, and its launch.
static bool skinny_applies(const GemmShape &g, const Epilogue &ep, bool need_sa, bool need_sb,
                           bool aligned) {
  if (!aligned || need_sa || need_sb || g.groups != 1 || ep.add.res) return false;
  if (g.K < 1024 || g.K % 32 != 0) return false;
  // Measured against the 64x64 tile: M128 K1024 N1024 4.9 vs 5.5 us, M64 K2048
  // N1000 6.7 vs 9.9; but M256 K512 N512 4.8 vs 4.5 and M32 K4096 N4096 12.1 vs
  // 11.5 (each 32x32 tile re-reads whole operand rows, which stops paying once
  // the 64x64 tiles occupy a quarter of the chip or the K loop is short).
  const long long tiles64 = (long long)((g.M + 63) / 64) * ((g.N + 63) / 64);
  return tiles64 <= 32;
}

static int gemm_skinny_launch(const DenseRows &A, const DenseRows &B, const Epilogue &ep,
                              const GemmShape &g, hipStream_t st) {
  const int tiles_m = (g.M + 31) / 32, tiles_n = (g.N + 31) / 32;
  hipLaunchKernelGGL(gemm_i8_skinny_kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, st,
                     A, B, ep, g.M, g.N, g.K, tiles_n);
  return check_launch("gemm_i8_skinny");
}

} // namespace mi355x
#endif
