// The int8 contraction for short K and many rows: pointwise convolutions of an
// image network's early stages and FullyConnected layers over 64, 128 or 256
// inputs, where a launch is all memory traffic and requantisation and the
// tiled kernels of gemm_i8.h spend their time in load latency, barriers and
// output staging.
//
//   * the weights of a workgroup's column slice (128 columns, at most 35 KB)
//     and the columns' requantisation constants are put in LDS once; from then
//     on the workgroup's waves never meet again;
//   * a wave walks over tiles of 32 rows: a lane loads its row's K bytes
//     straight from global memory into registers in the matrix-core layout
//     (every byte of A is read by exactly one lane), multiplies them with the
//     weight fragments read from LDS, 32 columns at a time, and requantises and
//     packs sixteen output bytes per lane (the transposed-accumulator epilogue
//     of gemm_i8.h); groups of up to 128 columns go through a wave-private
//     transpose in LDS so that they are written as whole 128-byte lines, with
//     the fused residual add read the same way;
//   * a wave asks for its next tile's rows before it works on the current one
//     and for a column group's residual bytes before that group's multiplies,
//     so that neither is waited for (K = 64 and 128; at K = 256 the rows alone
//     are 32 registers a lane and the loop stays plain); three workgroups per
//     CU, the registers allow no more, cover what is left.
//
// Results are bit for bit those of the tiled kernels (same integer sums, same
// requantisation).
#ifndef GLOW_MI355X_GEMM_STREAM_H
#define GLOW_MI355X_GEMM_STREAM_H

#include "gemm_i8.h"

namespace mi355x {

constexpr int kStreamMaxBN = 256;   // most columns a slice may have (the constants table's stride);
                                    // launches use slices of 128
constexpr int kStreamParBytes = kParArrays * kStreamMaxBN * 4;

// Rows of A: dense (row m at in + m * ld), or the window a convolution without
// padding and dilation reads for output pixel m of an [N, OH, OW] grid: it
// starts at input pixel (n, oh * sH, ow * sW) of an [N, IH, IW, IC] tensor and
// has KH segments of KW * IC contiguous bytes, one input row apart (a pointwise
// convolution: one segment of IC bytes).
struct StreamRows {
  const int8_t *in;
  long long ld;
  int dense;
  int OW, OHW, IH, IW, IC, sH, sW;
  int seg_chunks;        // 32-byte chunks per segment (a power of two; K / 32: one segment)
  long long seg_stride;  // bytes between segments
  __device__ __forceinline__ const int8_t *row(int m) const {
    if (dense) return in + (long long)m * ld;
    const int n = m / OHW, r = m - n * OHW;
    const int oh = r / OW, ow = r - oh * OW;
    return in + (((long long)n * IH + (long long)oh * sH) * IW + (long long)ow * sW) * IC;
  }
  // byte offset of chunk ks of a row from the row's start
  __device__ __forceinline__ long long chunk(int ks) const {
    return (long long)(ks / seg_chunks) * seg_stride + (ks % seg_chunks) * 32;
  }
};

// Bytes between the rows of a wave's staging tile: a group of up to 128 output
// columns plus 16 (consecutive rows start 36 banks apart).
constexpr int kStreamGroup = 128;
constexpr int kStreamStageStride = kStreamGroup + 16;
constexpr int kStreamStageBytes = 32 * kStreamStageStride;   // per wave

// The results leave through a wave-private transpose in LDS: groups of up to
// 128 columns are staged, then read back with group / 16 lanes per row, so that
// a store instruction writes whole lines and the residual is read the same way.
// NP: passes of the copy-out (four for groups of 96 and 128 columns, two for
// narrower ones); RES: a residual is added. Both are template parameters so
// that every load has exactly one place that uses it, on every path: the
// compiler then waits for a load where it is used and nowhere else.
// A lane's share of the rows of tile t: KS pieces of 16 bytes in the
// matrix-core layout (rows past the end re-read the last row; their results are
// not stored).
template <int KS>
__device__ __forceinline__ void stream_load_rows(const StreamRows &A, v4i (&dst)[KS], int t, int M,
                                                 int lane) {
  const int8_t *ar = A.row(min(t * 32 + (lane & 31), M - 1)) + (lane >> 5) * 16;
  if (A.seg_chunks >= KS) {
#pragma unroll
    for (int ks = 0; ks < KS; ks++) dst[ks] = *reinterpret_cast<const v4i *>(ar + ks * 32);
  } else {
#pragma unroll
    for (int ks = 0; ks < KS; ks++) dst[ks] = *reinterpret_cast<const v4i *>(ar + A.chunk(ks));
  }
}

// af: the rows of the wave's first tile, asked for by the caller.
template <int KS, int NP, bool RES, int MODE, bool LEAKY>
__device__ __forceinline__ void stream_tiles(const StreamRows &A, v4i (&af)[KS], const int8_t *s_w,
                                             const int32_t *s_par, int8_t *s_stage,
                                             const Epilogue &ep, int M, int N, int n0,
                                             int bn, int tiles32, int first, int step, int lane) {
  constexpr int WSTRIDE = KS * 32 + 16;
  const int l32 = lane & 31, lhi = lane >> 5;
  int32_t lo, hi;
  activation_clamp(ep, lo, hi);
  const bool fast = fused_out_is_fast(ep);
  const FusedAddConsts fc = fused_add_consts(ep.add);
  const int8_t *w_lane = s_w + l32 * WSTRIDE + lhi * 16;
  // column groups of this slice: 128 columns, or all of a narrower slice
  const int group = min(bn, kStreamGroup);         // bytes per row and group
  // copy-out: lpr lanes per row, rpp rows per pass
  const int lpr = group / 16, rpp = 64 / lpr;
  const int rb_row = lane / lpr, rb_seg = lane - rb_row * lpr;
  v4i an[KS];
  // (waited for here, once: inside the loop af is known to have arrived, and no
  // multiply waits behind the stores of the tile before)
#pragma unroll
  for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(af[ks]));
  for (int t = first; t < tiles32; t += step) {
    const int m0 = t * 32;
    const int last_row = min(31, M - 1 - m0);      // of this tile
    // the next tile's rows are on their way while this one is worked on
    stream_load_rows<KS>(A, an, min(t + step, tiles32 - 1), M, lane);
    for (int c0 = 0; c0 < bn; c0 += group) {
      // the group's residual bytes, in the layout of the copy-out, asked for
      // before the arithmetic they are added to. A lane whose row is past the
      // tile or the end works on the tile's last row instead and stores the
      // same bytes to the same place as that row's own lane: with every load
      // and store issued by every lane the waits can be counted exactly.
      int4 rq[NP];
      if constexpr (RES) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
          const int m = m0 + min(p * rpp + rb_row, last_row);
          rq[p] = *reinterpret_cast<const int4 *>(ep.add.res + (long long)m * ep.ldc + n0 + c0 +
                                                  rb_seg * 16);
        }
      }
      for (int j = c0 / 32; j < (c0 + group) / 32; j++) {
        v16i acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          const v4i b = *reinterpret_cast<const v4i *>(w_lane + j * 32 * WSTRIDE + ks * 32);
          // weights first: the result's rows are columns of the output
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, af[ks], acc, 0, 0, 0);
        }
        const int cl = j * 32 + 16 * lhi;
        const int4 v = requant_pack16<MODE, LEAKY, kStreamMaxBN>(acc, s_par + cl, ep, lo, hi);
        *reinterpret_cast<int4 *>(s_stage + l32 * kStreamStageStride + (cl - c0)) = v;
      }
      wave_fence();
#pragma unroll
      for (int p = 0; p < NP; p++) {
        const int row = min(p * rpp + rb_row, last_row), m = m0 + row;
        int4 v = *reinterpret_cast<const int4 *>(s_stage + row * kStreamStageStride + rb_seg * 16);
        if constexpr (RES)
          v = fused_out_words_loaded(v, rq[p], true, ep, fc, fast);
        else
          v = fused_out_words_loaded(v, v, false, ep, fc, fast);
        *reinterpret_cast<int4 *>(ep.out + (long long)m * ep.ldc + n0 + c0 + rb_seg * 16) = v;
      }
      wave_fence();
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) af[ks] = an[ks];
  }
}

// K = 256: the plain form of the loop. A lane's rows alone are 32 registers
// there; with the next tile's rows and a group's residual bytes asked for ahead
// the loop needs more registers than three waves per SIMD leave (spills, whose
// reloads wait behind the stores), and at two waves per SIMD it is slower than
// this: rows asked for at the top of the tile, the residual where it is added,
// four waves per SIMD if the LDS allows.
template <int KS, int MODE, bool LEAKY>
__device__ __forceinline__ void stream_tiles_simple(const StreamRows &A, const int8_t *s_w,
                                             const int32_t *s_par, int8_t *s_stage,
                                             const Epilogue &ep, int M, int N, int n0, int bn,
                                             int tiles32, int first, int step, int lane) {
  constexpr int WSTRIDE = KS * 32 + 16;
  const int l32 = lane & 31, lhi = lane >> 5;
  int32_t lo, hi;
  activation_clamp(ep, lo, hi);
  const bool fast = fused_out_is_fast(ep);
  const FusedAddConsts fc = fused_add_consts(ep.add);
  const int8_t *w_lane = s_w + l32 * WSTRIDE + lhi * 16;
  // column groups of this slice: 128 columns, or all of a narrower slice
  const int group = min(bn, kStreamGroup);         // bytes per row and group
  for (int t = first; t < tiles32; t += step) {
    const int m0 = t * 32;
    // rows past the end re-read the last row; their results are not stored
    const int8_t *ar = A.row(min(m0 + l32, M - 1)) + lhi * 16;
    v4i af[KS];
    if (A.seg_chunks >= KS) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) af[ks] = *reinterpret_cast<const v4i *>(ar + ks * 32);
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) af[ks] = *reinterpret_cast<const v4i *>(ar + A.chunk(ks));
    }
    for (int c0 = 0; c0 < bn; c0 += group) {
      for (int j = c0 / 32; j < (c0 + group) / 32; j++) {
        v16i acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          const v4i b = *reinterpret_cast<const v4i *>(w_lane + j * 32 * WSTRIDE + ks * 32);
          // weights first: the result's rows are columns of the output
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, af[ks], acc, 0, 0, 0);
        }
        const int cl = j * 32 + 16 * lhi;
        const int4 v = requant_pack16<MODE, LEAKY, kStreamMaxBN>(acc, s_par + cl, ep, lo, hi);
        *reinterpret_cast<int4 *>(s_stage + l32 * kStreamStageStride + (cl - c0)) = v;
      }
      wave_fence();
      wave_rows_copy_out(s_stage, kStreamStageStride, group, lane, m0, M, n0 + c0, ep, fc, fast);
      wave_fence();
    }
  }
}

// The requantisation variant is a template parameter as well (each variant
// keeps its own constants in registers; all four in one loop spill).
template <int KS, int NP, bool RES>
__device__ __forceinline__ void stream_tiles_mode(const StreamRows &A, v4i (&af)[KS],
                                                  const int8_t *s_w, const int32_t *s_par,
                                                  int8_t *s_stage, const Epilogue &ep, int mode,
                                                  int M, int N, int n0, int bn, int tiles32,
                                                  int first, int step, int lane) {
  if (ep.act == 5)
    stream_tiles<KS, NP, RES, 0, true>(A, af, s_w, s_par, s_stage, ep, M, N, n0, bn, tiles32, first,
                                       step, lane);
  else if (mode == 3)
    stream_tiles<KS, NP, RES, 3, false>(A, af, s_w, s_par, s_stage, ep, M, N, n0, bn, tiles32,
                                        first, step, lane);
  else if (mode == 1)
    stream_tiles<KS, NP, RES, 1, false>(A, af, s_w, s_par, s_stage, ep, M, N, n0, bn, tiles32,
                                        first, step, lane);
  else
    stream_tiles<KS, NP, RES, 0, false>(A, af, s_w, s_par, s_stage, ep, M, N, n0, bn, tiles32,
                                        first, step, lane);
}

// KS: K / 32 (2, 4 or 8). blockIdx.y: column slice of bn columns.
template <int KS>
__global__ __launch_bounds__(256, KS == 8 ? 4 : 3) void gemm_i8_stream_kernel(StreamRows A, const int8_t *W,
                                                                Epilogue ep, int M, int N, int bn,
                                                                int tiles32) {
  constexpr int K = KS * 32, WSTRIDE = K + 16;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int32_t *s_par = reinterpret_cast<int32_t *>(lds);
  int8_t *s_stage = lds + kStreamParBytes;               // one tile per wave
  int8_t *s_w = s_stage + 4 * kStreamStageBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.y * bn;
  const int cols = min(bn, N - n0);          // a multiple of 32
  const int mode = requant_mode(ep);

  // the wave's first rows are asked for before anything else, so that they
  // arrive while the slice is being put in LDS
  const int first = blockIdx.x * 4 + wave, step = gridDim.x * 4;
  v4i af[KS];
  if constexpr (KS < 8) stream_load_rows<KS>(A, af, min(first, tiles32 - 1), M, lane);

  // the slice's constants and weights -> LDS, once
  if (tid < cols) {
    ColRaw col[1];
    load_col_raw<1, kStreamMaxBN>(col, ep, N, n0, 0, 0, tid);
    par_table_store<kStreamMaxBN>(s_par, tid, col[0], ep, K, mode);
  }
  {
    constexpr int CH = K / 16;               // 16-byte chunks per weight row
    const int chunks = cols * CH;
    const int8_t *w0 = W + (long long)n0 * K;
    for (int base = 0; base < chunks; base += 256 * 4) {
      int4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int c = min(base + tid + u * 256, chunks - 1);
        v[u] = *reinterpret_cast<const int4 *>(w0 + (long long)c * 16);
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int c = base + tid + u * 256;
        if (c < chunks) {
          const int row = c / CH, kc = c - row * CH;
          *reinterpret_cast<int4 *>(s_w + perm_slot16(row) * WSTRIDE + kc * 16) = v[u];
        }
      }
    }
  }
  __syncthreads();

  // from here on every wave is on its own
  int8_t *stage = s_stage + wave * kStreamStageBytes;
  if constexpr (KS == 8) {
    if (ep.act == 5)
      stream_tiles_simple<KS, 0, true>(A, s_w, s_par, stage, ep, M, N, n0, cols, tiles32, first,
                                       step, lane);
    else if (mode == 3)
      stream_tiles_simple<KS, 3, false>(A, s_w, s_par, stage, ep, M, N, n0, cols, tiles32, first,
                                        step, lane);
    else if (mode == 1)
      stream_tiles_simple<KS, 1, false>(A, s_w, s_par, stage, ep, M, N, n0, cols, tiles32, first,
                                        step, lane);
    else
      stream_tiles_simple<KS, 0, false>(A, s_w, s_par, stage, ep, M, N, n0, cols, tiles32, first,
                                        step, lane);
  } else {
  const bool narrow = cols <= 64;            // two passes of the copy-out, not four
  if (ep.add.res) {
    if (narrow)
      stream_tiles_mode<KS, 2, true>(A, af, s_w, s_par, stage, ep, mode, M, N, n0, cols, tiles32, first,
                                step, lane);
    else
      stream_tiles_mode<KS, 4, true>(A, af, s_w, s_par, stage, ep, mode, M, N, n0, cols, tiles32, first,
                                step, lane);
  } else {
    if (narrow)
      stream_tiles_mode<KS, 2, false>(A, af, s_w, s_par, stage, ep, mode, M, N, n0, cols, tiles32, first,
                                 step, lane);
    else
      stream_tiles_mode<KS, 4, false>(A, af, s_w, s_par, stage, ep, mode, M, N, n0, cols, tiles32, first,
                                 step, lane);
  }
  }
}

// Whether the streaming kernel can run this product at all: K of 64, 128 or
// 256, 16-byte aligned operands and output, whole 32-column tiles, weight
// offsets all zero with their row sums precomputed (no in-kernel row sums).
static bool stream_can_run(int M, int N, int K, bool need_sa, bool need_sb, bool aligned,
                           const Epilogue &ep) {
  if (need_sa || need_sb || !aligned) return false;
  if (K != 64 && K != 128 && K != 256) return false;
  // whole 32-column tiles, and whole 128-column groups once there are more than 128
  if (N % 32 != 0 || (N > kStreamGroup && N % kStreamGroup != 0) || M < 1) return false;
  if (ep.ldc % 16 != 0 || (((((uintptr_t)ep.out) | ((uintptr_t)ep.add.res)) & 15) != 0))
    return false;
  return true;
}

// Whether it is the default for such a product. Measured with the backend's
// requantisation hint against the best tiled kernel (us): M200704 K64 N64 8.8
// vs 12.2, K64 N256 23.8 vs 28.0, K256 N64 15.3 vs 18.5, K256 N128 23.6 vs 25.0;
// M50176 K128 N512 17.5 vs 18.6, K256 N512 24.1 vs 23.9; M12544 K256 N1024 14.5
// vs 14.3: level once the weight slices multiply the reads of A.
static bool stream_applies(int M, int N) { return M >= 4096 && N <= 512; }

static int gemm_stream_launch(const StreamRows &A, const int8_t *W, const Epilogue &ep, int M,
                              int N, int K, hipStream_t st) {
  // 128 columns per slice: a slice's weights stay under 35 KB beside 18 KB of
  // staging tiles and the 5 KB constants table, and a unit of work (32 rows of
  // one slice) is small enough that the last round of tiles, which only some of
  // the waves take part in, costs little (K = 64, 256 output columns, 200704
  // rows: 37.7 us in slices of 128 against 38.6 us in one of 256, though the
  // rows are then read twice)
  const int bn = 128;
  const int slices = (N + bn - 1) / bn;
  const size_t lds = (size_t)kStreamParBytes + 4 * (size_t)kStreamStageBytes +
                     (size_t)std::min(bn, N) * (K + 16);
  const int tiles32 = (M + 31) / 32;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
  }
  const int per_cu = (int)std::min<size_t>(K == 256 ? 4 : 3, (160 * 1024) / lds);
  long long gx = std::max(1LL, (long long)cus * per_cu / slices);
  gx = std::min<long long>(gx, (tiles32 + 3) / 4);
  MI355X_REQUIRE(slices < 65536, "problem too large");
  const dim3 grid((unsigned)gx, (unsigned)slices), block(256);
  switch (K) {
  case 64:
    hipLaunchKernelGGL(gemm_i8_stream_kernel<2>, grid, block, lds, st, A, W, ep, M, N, bn, tiles32);
    break;
  case 128:
    hipLaunchKernelGGL(gemm_i8_stream_kernel<4>, grid, block, lds, st, A, W, ep, M, N, bn, tiles32);
    break;
  default: {
    // 128 columns x 272 bytes of weights: past the 48 KiB a launch gets unasked
    static std::atomic<uint64_t> attr_set{0};
    const int rc = set_lds_attr(gemm_i8_stream_kernel<8>, 64 * 1024, attr_set);
    if (rc != MI355X_OK) return rc;
    hipLaunchKernelGGL(gemm_i8_stream_kernel<8>, grid, block, lds, st, A, W, ep, M, N, bn, tiles32);
    break;
  }
  }
  return check_launch("gemm_i8_stream");
}

} // namespace mi355x
#endif
