// int8 x int8 -> int32 tiled contraction on the gfx950 matrix cores with
// Glow's integer requantisation fused into the epilogue. Shared by the
// FullyConnected family (fc.hip) and the implicit-GEMM convolutions (conv.hip).
//
//   C[m][n] = clip8(act(scale(sum_k (A[m][k]-aOff)(B[n][k]-bOff[n]) + bias'[n])))
//
// Both operands are K-contiguous (activations [M x K]; RowwiseQuantized FC
// weights [N x K]; conv filters [OC x KH*KW*IC]), which is exactly the
// per-lane operand layout of v_mfma_i32_32x32x32_i8: a lane feeds 16
// consecutive k-bytes of one row. Offsets cannot be subtracted in int8, so the
// matrix cores contract the raw bytes and the epilogue applies
//   sum(A-aOff)(B-bOff) = sum AB - aOff*sum_k B[n] - bOff[n]*sum_k A[m]
//                         + K*aOff*bOff[n]
// with the row sums taken from the operand fragments (v_dot4) while they pass
// through registers. Everything is exact modulo 2^32, like the CPU loop.
//
// Block tile BM x BN, K step 64 bytes, waves own WM x WN sub-tiles. Global ->
// registers -> LDS with two LDS stages (one barrier per K step); LDS rows are
// padded to 80 bytes so the 16-byte fragment reads of 16 consecutive rows
// fall on distinct banks. The int8 results are staged through LDS and leave
// as 16-byte row segments.
#ifndef GLOW_MI355X_GEMM_I8_H
#define GLOW_MI355X_GEMM_I8_H

#include "common.h"
#include "requant.h"

namespace mi355x {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;            // bytes of K per step
constexpr int kLdsStride = kBK + 16;

// A per-column parameter: a device vector, or one scalar for all columns.
struct ColParam {
  const int32_t *v;
  int32_t s;
  __device__ __forceinline__ int32_t at(int n) const { return v ? v[n] : s; }
};

struct Epilogue {
  int8_t *out;
  long long ldc;        // elements between output rows
  const void *bias;     // int32[N] / int8[N] / NULL (no bias term)
  int bias_is_i8;
  ColParam b_off, bias_pre, bias_post, bias_scale;
  ColParam w_off, out_pre, out_post, out_scale;
  int32_t a_off;        // offset of the A operand (activations)
  int32_t out_off;
  int32_t act, a0, a1, a2;
};

// Row-major [rows x K] operand (activations, or weights with K contiguous).
struct DenseRows {
  const int8_t *p;
  long long ld;
  int rows;
  struct Row {
    const int8_t *base;
    bool ok;
  };
  __device__ __forceinline__ void set_group(int) {}
  __device__ __forceinline__ Row row(int r) const {
    return Row{p + (long long)r * ld, r < rows};
  }
  template <bool ALIGNED>
  __device__ __forceinline__ int4 load(const Row &r, int k, int K) const {
    int4 v = make_int4(0, 0, 0, 0);
    if (!r.ok || k >= K) return v;
    if constexpr (ALIGNED) {
      return *reinterpret_cast<const int4 *>(r.base + k);
    } else {
      uint32_t w[4] = {0, 0, 0, 0};
      const int n = min(16, K - k);
      for (int b = 0; b < n; b++)
        w[b >> 2] |= (uint32_t)(uint8_t)r.base[k + b] << (8 * (b & 3));
      return make_int4((int)w[0], (int)w[1], (int)w[2], (int)w[3]);
    }
  }
};

// Output-tile to block mapping. Consecutive block ids land on different XCDs
// (round-robin dispatch over 8 dies, each with its own L2), so ids are first
// regrouped per die and then walked in panels of kPanel tile rows so that the
// blocks resident on one die share A and B tiles in its L2.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n,
                                              int &tm, int &tn) {
  const int total = tiles_m * tiles_n;
  constexpr int kXcd = 8;
  int id = bid;
  if (total % kXcd == 0) id = (bid % kXcd) * (total / kXcd) + bid / kXcd;
  constexpr int kPanel = 8;
  const int per_panel = kPanel * tiles_n;
  const int panel = id / per_panel;
  const int in_panel = id - panel * per_panel;
  const int rows_here = min(kPanel, tiles_m - panel * kPanel);
  tm = panel * kPanel + in_panel % rows_here;
  tn = in_panel / rows_here;
}

template <int BM, int BN, int WM, int WN, bool NEED_SA, bool NEED_SB,
          bool AL_A, bool AL_B, class ARows>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void gemm_i8_kernel(
    ARows A, DenseRows B, Epilogue ep, int M, int N, int K, int tiles_m,
    int tiles_n, long long b_group_stride, int n_per_group) {
  constexpr int WAVES_N = BN / WN;
  constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int CH_ROW = kBK / 16;                 // 16-byte chunks per tile row
  constexpr int A_CH = BM * CH_ROW / THREADS;      // chunks per thread
  constexpr int B_CH = BN * CH_ROW / THREADS;
  static_assert(BM * CH_ROW % THREADS == 0 && BN * CH_ROW % THREADS == 0, "");
  constexpr int STAGE = (BM + BN) * kLdsStride;
  constexpr int OUT_STRIDE = BN + 16;

  extern __shared__ __attribute__((aligned(16))) int8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, lhi = lane >> 5;

  // grouped convolution: blockIdx.y selects the group
  const int grp = blockIdx.y;
  A.set_group(grp);
  B.p += (long long)grp * b_group_stride;
  const int n_base = grp * n_per_group;            // first output column

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  typename ARows::Row arow[A_CH];
  DenseRows::Row brow[B_CH];
  int a_lds[A_CH], b_lds[B_CH], a_k[A_CH], b_k[B_CH];
#pragma unroll
  for (int i = 0; i < A_CH; i++) {
    const int c = tid + i * THREADS;
    const int r = c / CH_ROW, kc = c % CH_ROW;
    arow[i] = A.row(m0 + r);
    a_k[i] = kc * 16;
    a_lds[i] = r * kLdsStride + kc * 16;
  }
#pragma unroll
  for (int i = 0; i < B_CH; i++) {
    const int c = tid + i * THREADS;
    const int r = c / CH_ROW, kc = c % CH_ROW;
    brow[i] = B.row(n0 + r);
    b_k[i] = kc * 16;
    b_lds[i] = (BM + r) * kLdsStride + kc * 16;
  }

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
  int sa[TM], sb[TN];
#pragma unroll
  for (int i = 0; i < TM; i++) sa[i] = 0;
#pragma unroll
  for (int j = 0; j < TN; j++) sb[j] = 0;

  const int KT = (K + kBK - 1) / kBK;
  int4 ra[A_CH], rb[B_CH];
#pragma unroll
  for (int i = 0; i < A_CH; i++) ra[i] = A.template load<AL_A>(arow[i], a_k[i], K);
#pragma unroll
  for (int i = 0; i < B_CH; i++) rb[i] = B.template load<AL_B>(brow[i], b_k[i], K);
#pragma unroll
  for (int i = 0; i < A_CH; i++) *reinterpret_cast<int4 *>(lds + a_lds[i]) = ra[i];
#pragma unroll
  for (int i = 0; i < B_CH; i++) *reinterpret_cast<int4 *>(lds + b_lds[i]) = rb[i];
  __syncthreads();

  const int a_frag = (wm * WM + l32) * kLdsStride + lhi * 16;
  const int b_frag = (BM + wn * WN + l32) * kLdsStride + lhi * 16;

  for (int kt = 0; kt < KT; kt++) {
    const int8_t *cur = lds + (kt & 1) * STAGE;
    const bool more = kt + 1 < KT;
    if (more) {
      const int k0 = (kt + 1) * kBK;
#pragma unroll
      for (int i = 0; i < A_CH; i++)
        ra[i] = A.template load<AL_A>(arow[i], k0 + a_k[i], K);
#pragma unroll
      for (int i = 0; i < B_CH; i++)
        rb[i] = B.template load<AL_B>(brow[i], k0 + b_k[i], K);
    }
#pragma unroll
    for (int ks = 0; ks < kBK / 32; ks++) {
      v4i af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        af[i] = *reinterpret_cast<const v4i *>(cur + a_frag + i * 32 * kLdsStride + ks * 32);
#pragma unroll
      for (int j = 0; j < TN; j++)
        bf[j] = *reinterpret_cast<const v4i *>(cur + b_frag + j * 32 * kLdsStride + ks * 32);
      if constexpr (NEED_SA) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int q = 0; q < 4; q++)
            sa[i] = __builtin_amdgcn_sdot4(af[i][q], 0x01010101, sa[i], false);
      }
      if constexpr (NEED_SB) {
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int q = 0; q < 4; q++)
            sb[j] = __builtin_amdgcn_sdot4(bf[j][q], 0x01010101, sb[j], false);
      }
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      int8_t *nxt = lds + ((kt + 1) & 1) * STAGE;
#pragma unroll
      for (int i = 0; i < A_CH; i++) *reinterpret_cast<int4 *>(nxt + a_lds[i]) = ra[i];
#pragma unroll
      for (int i = 0; i < B_CH; i++) *reinterpret_cast<int4 *>(nxt + b_lds[i]) = rb[i];
    }
    __syncthreads();
  }

  // ---- epilogue --------------------------------------------------------------
  // LDS is free now: [row sums of A per wave | int8 output tile]
  int32_t *s_sumA = reinterpret_cast<int32_t *>(lds);            // BM ints
  int8_t *s_out = lds + BM * 4;
  if constexpr (NEED_SA) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      sa[i] += __shfl_xor(sa[i], 32, 64);
      // waves of one block row hold identical sums; all may write
      if (lhi == 0) s_sumA[wm * WM + i * 32 + l32] = sa[i];
    }
  }
  if constexpr (NEED_SB) {
#pragma unroll
    for (int j = 0; j < TN; j++) sb[j] += __shfl_xor(sb[j], 32, 64);
  }
  __syncthreads();

#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nl = n0 + wn * WN + j * 32 + l32;   // column within the group
    const bool n_ok = nl < N;
    const int n = n_base + (n_ok ? nl : 0);       // global output column
    const int32_t woff = ep.w_off.at(n);
    const int32_t opre = ep.out_pre.at(n), opost = ep.out_post.at(n);
    const int32_t oscale = ep.out_scale.at(n);
    uint32_t colc = (uint32_t)K * (uint32_t)ep.a_off * (uint32_t)woff;
    if constexpr (NEED_SB) colc -= (uint32_t)ep.a_off * (uint32_t)sb[j];
    if (ep.bias) {
      const int32_t b = ep.bias_is_i8
                            ? (int32_t) reinterpret_cast<const int8_t *>(ep.bias)[n]
                            : reinterpret_cast<const int32_t *>(ep.bias)[n];
      colc += (uint32_t)scale_i32((int32_t)((uint32_t)b - (uint32_t)ep.b_off.at(n)),
                                  ep.bias_pre.at(n), ep.bias_post.at(n),
                                  ep.bias_scale.at(n), 0);
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ml = wm * WM + i * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
        uint32_t v = (uint32_t)acc[i][j][r] + colc;
        if constexpr (NEED_SA) v -= (uint32_t)woff * (uint32_t)s_sumA[ml];
        int32_t y = scale_i32((int32_t)v, opre, opost, oscale, ep.out_off);
        y = activation_i32(y, ep.out_off, ep.act, ep.a0, ep.a1, ep.a2);
        s_out[ml * OUT_STRIDE + wn * WN + j * 32 + l32] = (int8_t)clip_i8(y);
      }
    }
  }
  __syncthreads();

  // coalesced copy-out: 16-byte row segments where the output allows it
  const int cols_here = min(BN, N - n0);
  const int rows_here = min(BM, M - m0);
  int8_t *obase = ep.out + (long long)m0 * ep.ldc + n_base + n0;
  const bool vec_ok = (cols_here % 16 == 0) && (ep.ldc % 16 == 0) &&
                      ((((uintptr_t)obase) & 15) == 0);
  if (vec_ok) {
    const int segs = cols_here / 16;
    for (int c = tid; c < rows_here * segs; c += THREADS) {
      const int r = c / segs, s = c - r * segs;
      *reinterpret_cast<int4 *>(obase + (long long)r * ep.ldc + s * 16) =
          *reinterpret_cast<const int4 *>(s_out + r * OUT_STRIDE + s * 16);
    }
  } else {
    for (int c = tid; c < rows_here * cols_here; c += THREADS) {
      const int r = c / cols_here, s = c - r * cols_here;
      obase[(long long)r * ep.ldc + s] = s_out[r * OUT_STRIDE + s];
    }
  }
}

template <int BM, int BN> constexpr size_t gemm_lds_bytes() {
  constexpr size_t stages = 2 * (size_t)(BM + BN) * kLdsStride;
  constexpr size_t epi = (size_t)BM * 4 + (size_t)BM * (BN + 16);
  return stages > epi ? stages : epi;
}

// Launches one tile configuration. `groups` > 1 is the grouped convolution.
template <int BM, int BN, int WM, int WN, bool SA, bool SB, bool AL_A,
          bool AL_B, class ARows>
static int gemm_launch(const ARows &A, const DenseRows &B, const Epilogue &ep,
                       int M, int N, int K, int groups,
                       long long b_group_stride, hipStream_t st) {
  constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
  constexpr size_t lds = gemm_lds_bytes<BM, BN>();
  auto kern = gemm_i8_kernel<BM, BN, WM, WN, SA, SB, AL_A, AL_B, ARows>;
  if (lds > 48 * 1024) {
    static bool attr_set = false; // per instantiation
    if (!attr_set) {
      MI355X_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
      attr_set = true;
    }
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const long long total = (long long)tiles_m * tiles_n;
  MI355X_REQUIRE(total < 0x7fffffffLL && groups < 65536, "problem too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)groups),
                     dim3(THREADS), lds, st, A, B, ep, M, N, K, tiles_m,
                     tiles_n, b_group_stride, N);
  return check_launch("gemm_i8");
}

// LDS a block may use on the current device (cached per process).
static size_t lds_limit() {
  static size_t limit = 0;
  if (!limit) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipGetDeviceProperties(&p, dev) == hipSuccess)
      limit = p.sharedMemPerBlock;
    else
      limit = 64 * 1024;
  }
  return limit;
}

// Picks the tile configuration from the problem size: the 256x256 tile for
// large problems (a wave owns 128x128, which halves LDS traffic per MFMA), and
// smaller tiles when the grid would otherwise not fill 256 CUs.
template <bool SA, bool SB, bool AL_A, bool AL_B, class ARows>
static int gemm_dispatch_tiles(const ARows &A, const DenseRows &B,
                               const Epilogue &ep, int M, int N, int K,
                               int groups, long long b_group_stride,
                               hipStream_t st) {
  auto tiles = [&](int bm, int bn) {
    return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn) * groups;
  };
  if (tiles(256, 256) >= 256 && N >= 192 &&
      gemm_lds_bytes<256, 256>() <= lds_limit())
    return gemm_launch<256, 256, 128, 128, SA, SB, AL_A, AL_B>(
        A, B, ep, M, N, K, groups, b_group_stride, st);
  if (tiles(128, 128) >= 256 && N >= 96)
    return gemm_launch<128, 128, 64, 64, SA, SB, AL_A, AL_B>(
        A, B, ep, M, N, K, groups, b_group_stride, st);
  if (tiles(128, 64) >= 256 || M >= 1024)
    return gemm_launch<128, 64, 32, 64, SA, SB, AL_A, AL_B>(
        A, B, ep, M, N, K, groups, b_group_stride, st);
  return gemm_launch<64, 64, 32, 32, SA, SB, AL_A, AL_B>(
      A, B, ep, M, N, K, groups, b_group_stride, st);
}

template <class ARows>
static int gemm_dispatch(const ARows &A, const DenseRows &B, const Epilogue &ep,
                         int M, int N, int K, int groups,
                         long long b_group_stride, bool need_sa, bool need_sb,
                         bool al_a, bool al_b, hipStream_t st) {
#define MI355X_GEMM_CASE(SA, SB, AA, AB)                                       \
  if (need_sa == SA && need_sb == SB && al_a == AA && al_b == AB)              \
    return gemm_dispatch_tiles<SA, SB, AA, AB>(A, B, ep, M, N, K, groups,      \
                                               b_group_stride, st);
  // aligned operands: all four row-sum combinations
  MI355X_GEMM_CASE(false, false, true, true)
  MI355X_GEMM_CASE(false, true, true, true)
  MI355X_GEMM_CASE(true, false, true, true)
  MI355X_GEMM_CASE(true, true, true, true)
#undef MI355X_GEMM_CASE
  // any unaligned operand: the byte-wise loaders with both row sums
  return gemm_dispatch_tiles<true, true, false, false>(A, B, ep, M, N, K, groups,
                                                       b_group_stride, st);
}

} // namespace mi355x
#endif
