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
// Block tile BM x BN, K step 64 bytes, waves own WM x WN sub-tiles. Two main
// loops share one epilogue:
//   gemm_i8_dma_kernel  K % 64 == 0 and 16-byte aligned operands. Tiles go
//       global -> LDS directly (global_load_lds_dwordx4, no staging registers)
//       through a ring of STAGES LDS buffers, so loads run STAGES-1 K steps
//       ahead of the matrix cores; one barrier per K step. LDS rows are 64
//       bytes, unpadded; the 16-byte chunk kc of row r sits at position
//       kc ^ ((r >> 2) & 3), which makes the fragment reads of 16 consecutive
//       rows fall on distinct banks.
//   gemm_i8_kernel      everything else (K tails, unaligned rows, 3-channel
//       convolutions): global -> registers -> LDS with two stages and rows
//       padded to 80 bytes.
// The int8 results are staged through LDS and leave as 16-byte row segments.
#ifndef GLOW_MI355X_GEMM_I8_H
#define GLOW_MI355X_GEMM_I8_H

#include "common.h"
#include "requant.h"

#include <atomic>
#include <type_traits>

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

// A residual tensor added to the (already clipped) int8 result while the
// output tile is written, optionally followed by Relu: what ElementAdd and Relu
// instructions behind a convolution compute, without the round trip through
// memory. Same arithmetic as the standalone kernels.
// With res == NULL and relu != 0 only the Relu stage runs, on this kernel's own
// result: a Relu instruction (with its own output scale and offset) behind a
// FullyConnected. sum_off is then the offset of the kernel's result.
struct FusedAdd {
  const int8_t *res;    // [M x ldc] like the output, or NULL
  int32_t sum_off, own_off, res_off;
  int32_t own_pre, own_post, own_scale;   // rescale of this kernel's result
  int32_t res_pre, res_post, res_scale;   // rescale of the residual
  int32_t relu;                           // apply the Relu stage below
  int32_t dest_off, dest_pre, dest_post, dest_scale;
  int32_t small;                          // every scale is below 2^23 in magnitude
};

template <bool SMALL>
__device__ __forceinline__ int32_t fused_add_one(int32_t own, int32_t res,
                                                 const FusedAdd &f) {
  const int32_t a =
      scale_i32_sel<SMALL>(own - f.own_off, f.own_pre, f.own_post, f.own_scale, 0);
  const int32_t b =
      scale_i32_sel<SMALL>(res - f.res_off, f.res_pre, f.res_post, f.res_scale, 0);
  int32_t v = clip_i8((int32_t)((uint32_t)a + (uint32_t)b + (uint32_t)f.sum_off));
  if (f.relu) {
    const int32_t so = (int32_t)(int8_t)f.sum_off;
    v = max(v, so);
    v = clip_i8(scale_i32_sel<SMALL>(v - so, f.dest_pre, f.dest_post, f.dest_scale,
                                     f.dest_off));
  }
  return v;
}

template <bool SMALL>
__device__ __forceinline__ uint32_t fused_add_word_t(uint32_t own, uint32_t res,
                                                     const FusedAdd &f) {
  uint32_t o = 0;
#pragma unroll
  for (int b = 0; b < 4; b++)
    o |= (uint32_t)(fused_add_one<SMALL>((int32_t)(int8_t)(own >> (8 * b)),
                                         (int32_t)(int8_t)(res >> (8 * b)), f) & 0xff)
         << (8 * b);
  return o;
}

// libjit_element_relu_i8-style stage alone: clip(scale(max(v, so) - so) + dest_off)
template <bool SMALL>
__device__ __forceinline__ uint32_t fused_relu_word_t(uint32_t own, const FusedAdd &f) {
  const int32_t so = (int32_t)(int8_t)f.sum_off;
  uint32_t o = 0;
#pragma unroll
  for (int b = 0; b < 4; b++) {
    const int32_t v = max((int32_t)(int8_t)(own >> (8 * b)), so);
    o |= (uint32_t)(clip_i8(scale_i32_sel<SMALL>(v - so, f.dest_pre, f.dest_post,
                                                 f.dest_scale, f.dest_off)) & 0xff)
         << (8 * b);
  }
  return o;
}
__device__ __forceinline__ uint32_t fused_relu_word(uint32_t own, const FusedAdd &f) {
  return f.small ? fused_relu_word_t<true>(own, f) : fused_relu_word_t<false>(own, f);
}

// The common case of both stages: every scale below 2^23 in magnitude and no
// pre-shift (rescale factors near one). Then ((x - off) * s + rtn) equals
// x * s + (rtn - off * s) modulo 2^32, one 24-bit multiply-add per value with
// a constant formed once, and the result is bit for bit that of scale_i32.
// The Relu stage folds further (fused_out_is_fast checks the bounds that keep
// every sum inside 32 bits): clip to int8 followed by max(., so) is one clamp
// to [max(-128, so), 127], and the offset added behind the post-shift goes
// into the constant in front of it ((X >> p) + d == (X + (d << p)) >> p).
struct FusedAddConsts {
  int32_t own_c, res_c, relu_c, sum_lo;
  int32_t relu_scale, relu_post;   // 1 and 0 (with relu_c 0) when no Relu follows the add
};
__device__ __forceinline__ FusedAddConsts fused_add_consts(const FusedAdd &f) {
  auto rtn = [](int32_t post) { return post > 0 ? (1u << (post - 1)) : 0u; };
  const int32_t so = (int32_t)(int8_t)f.sum_off;
  FusedAddConsts c;
  c.own_c = (int32_t)(rtn(f.own_post) - (uint32_t)f.own_off * (uint32_t)f.own_scale);
  c.res_c = (int32_t)(rtn(f.res_post) - (uint32_t)f.res_off * (uint32_t)f.res_scale);
  c.relu_c = (int32_t)(rtn(f.dest_post) - (uint32_t)so * (uint32_t)f.dest_scale +
                       ((uint32_t)f.dest_off << (f.dest_post & 31)));
  c.sum_lo = max(-128, so);
  c.relu_scale = f.dest_scale;
  c.relu_post = f.dest_post;
  if (!f.relu) {
    // the same instructions leave the clipped sum as it is: v * 1 + 0 >> 0
    c.relu_c = 0;
    c.sum_lo = -128;
    c.relu_scale = 1;
    c.relu_post = 0;
  }
  asm volatile("" : "+v"(c.own_c), "+v"(c.res_c), "+v"(c.relu_c), "+v"(c.sum_lo));
  return c;
}
template <bool ADD>
__device__ __forceinline__ uint32_t fused_word_fast(uint32_t own, uint32_t res,
                                                    const FusedAdd &f,
                                                    const FusedAddConsts &c) {
  int32_t r[4];
#pragma unroll
  for (int b = 0; b < 4; b++) {
    int32_t v = (int32_t)(int8_t)(own >> (8 * b));
    if constexpr (ADD) {
      const int32_t x = (int32_t)(int8_t)(res >> (8 * b));
      const int32_t a = (int32_t)((uint32_t)__mul24(v, f.own_scale) + (uint32_t)c.own_c) >> f.own_post;
      const int32_t bb = (int32_t)((uint32_t)__mul24(x, f.res_scale) + (uint32_t)c.res_c) >> f.res_post;
      // the int8 clip of the sum and the Relu's lower bound in one clamp
      v = med3_i32((int32_t)((uint32_t)a + (uint32_t)bb + (uint32_t)f.sum_off), c.sum_lo, 127);
    } else {
      v = max(v, c.sum_lo);
    }
    v = (int32_t)((uint32_t)__mul24(v, c.relu_scale) + (uint32_t)c.relu_c) >> c.relu_post;
    v = med3_i32(v, -128, 127);
    r[b] = v;
  }
  return __builtin_amdgcn_perm(
      __builtin_amdgcn_perm((uint32_t)r[3], (uint32_t)r[2], 0x0c0c0400u),
      __builtin_amdgcn_perm((uint32_t)r[1], (uint32_t)r[0], 0x0c0c0400u), 0x05040100u);
}

// int8 operands minus int8-range offsets stay far below 2^23, so the 24-bit
// multiplier applies whenever the scales do (f.small, set on the host).
__device__ __forceinline__ uint32_t fused_add_word(uint32_t own, uint32_t res,
                                                   const FusedAdd &f) {
  return f.small ? fused_add_word_t<true>(own, res, f)
                 : fused_add_word_t<false>(own, res, f);
}

struct Epilogue {
  int8_t *out;
  long long ldc;        // elements between output rows
  const void *bias;     // int32[N] / int8[N] / NULL (no bias term)
  int bias_is_i8;
  ColParam b_off, bias_pre, bias_post, bias_scale;
  ColParam w_off, out_pre, out_post, out_scale;
  const int32_t *sum_b; // precomputed sum_k B[n][k] per output column, or NULL
  int32_t a_off;        // offset of the A operand (activations)
  int32_t out_off;
  int32_t act, a0, a1, a2;
  FusedAdd add;         // add.res == NULL: none
  // Requantisation hints from the caller (mi355x_gemm_requant_hint):
  // bit 0: every value this launch can form in front of the output multiply
  //        fits 24 bits after its column's pre-shift, every output scale fits
  //        24 bits, and product + rounding term + (out_off << post) stays
  //        inside 32 bits; bit 1: every output pre-shift is zero.
  int32_t fast;
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
  // where the 16 bytes [k, k+16) sit inside any row
  struct Loc {
    int k;
  };
  __device__ __forceinline__ Loc locate(int k) const { return Loc{k}; }
  // the location one K step (kBK bytes) further on
  __device__ __forceinline__ void advance(Loc &l) const { l.k += 64; }
  // address of those bytes in a row that exists
  __device__ __forceinline__ const int8_t *chunk_ptr(const Row &r, const Loc &l) const {
    return r.base + l.k;
  }
  template <bool ALIGNED>
  __device__ __forceinline__ int4 load(const Row &r, int k, int K) const {
    int4 v = make_int4(0, 0, 0, 0);
    if (!r.ok || k >= K) return v;
    if constexpr (ALIGNED) {
      return *reinterpret_cast<const int4 *>(r.base + k);
    } else {
      // a whole chunk inside the row: one 16-byte load from a byte-aligned
      // address (global memory takes unaligned vector loads)
      if (k + 16 <= K) {
        struct __attribute__((packed, aligned(1))) Chunk { int x, y, z, w; };
        const Chunk c = *reinterpret_cast<const Chunk *>(r.base + k);
        return make_int4(c.x, c.y, c.z, c.w);
      }
      // The row's last, partial chunk (n = K - k bytes, 1..15), without a
      // chain of dependent byte loads.
      const int n = K - k;
      if (K >= 16) {
        // the 16 bytes that end with the row, moved down by 16 - n bytes
        struct __attribute__((packed, aligned(1))) Chunk { uint32_t x, y, z, w; };
        const Chunk c = *reinterpret_cast<const Chunk *>(r.base + K - 16);
        const int s = 16 - n, ws = s >> 2, bs = (s & 3) * 8;
        const uint32_t in[8] = {c.x, c.y, c.z, c.w, 0, 0, 0, 0};
        uint32_t t[5];
#pragma unroll
        for (int j = 0; j < 5; j++)
          t[j] = ws == 0 ? in[j] : ws == 1 ? in[j + 1] : ws == 2 ? in[j + 2] : in[j + 3];
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = __funnelshift_r(t[j], t[j + 1], bs);
        return make_int4((int)o[0], (int)o[1], (int)o[2], (int)o[3]);
      }
      // rows shorter than a chunk: every byte on its own, all loads in flight
      // (slots beyond the row re-read its last byte and are masked)
      uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 16; b++) {
        const uint32_t v = (uint8_t)r.base[k + min(b, n - 1)];
        w[b >> 2] |= (b < n ? v : 0u) << (8 * (b & 3));
      }
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

// The per-column parameters one lane's output columns need in the epilogue,
// as they lie in memory. The direct-to-LDS kernel requests them before its
// first tile load, so that they have long arrived when the K loop ends and
// the epilogue starts without a memory round trip of its own.
struct ColRaw {
  int32_t woff, opre, opost, oscale, sumb, bias, boff, bpre, bpost, bscale;
};
template <int TN, int WN>
__device__ __forceinline__ void load_col_raw(ColRaw (&c)[TN], const Epilogue &ep, int N, int n0,
                                             int n_base, int wn, int l32) {
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int nl = n0 + wn * WN + j * 32 + l32;   // column within the group
    const int n = n_base + (nl < N ? nl : 0);     // global output column
    c[j].woff = ep.w_off.at(n);
    c[j].opre = ep.out_pre.at(n);
    c[j].opost = ep.out_post.at(n);
    c[j].oscale = ep.out_scale.at(n);
    c[j].sumb = ep.sum_b ? ep.sum_b[n] : 0;
    c[j].bias = 0;
    c[j].boff = c[j].bpre = c[j].bpost = c[j].bscale = 0;
    if (ep.bias) {
      c[j].bias = ep.bias_is_i8 ? (int32_t) reinterpret_cast<const int8_t *>(ep.bias)[n]
                                : reinterpret_cast<const int32_t *>(ep.bias)[n];
      c[j].boff = ep.b_off.at(n);
      c[j].bpre = ep.bias_pre.at(n);
      c[j].bpost = ep.bias_post.at(n);
      c[j].bscale = ep.bias_scale.at(n);
    }
  }
}

// The fused residual add / Relu on 16 staged output bytes; res16 points at the
// 16 residual bytes of the same place (NULL: no residual). `fast`: every scale
// small and no pre-shift in the stages that run.
__device__ __forceinline__ bool fused_out_is_fast(const Epilogue &ep) {
  // Relu stage: (v - so) * scale is below 2^8 * 2^22, the folded offset
  // |dest_off| << post at most 2^7 * 2^22, the rounding term 2^21
  const bool relu_ok = ep.add.dest_pre == 0 && ep.add.dest_post <= 22 &&
                       ep.add.dest_scale > -(1 << 22) && ep.add.dest_scale < (1 << 22) &&
                       ep.add.dest_off >= -128 && ep.add.dest_off <= 127;
  return ep.add.small &&
         (!ep.add.res || (ep.add.own_pre == 0 && ep.add.res_pre == 0)) &&
         (!ep.add.relu || relu_ok);
}
__device__ __forceinline__ int4 fused_out_words(int4 v, const int8_t *res16, const Epilogue &ep,
                                                const FusedAddConsts &fc, bool fast) {
  if (res16 && fast) {
    const int4 q = *reinterpret_cast<const int4 *>(res16);
    // (a word at a time: sixteen values in flight at once cost the tiled kernels
    // twenty registers)
    v.x = (int)fused_word_fast<true>((uint32_t)v.x, (uint32_t)q.x, ep.add, fc);
    __builtin_amdgcn_sched_barrier(0);
    v.y = (int)fused_word_fast<true>((uint32_t)v.y, (uint32_t)q.y, ep.add, fc);
    __builtin_amdgcn_sched_barrier(0);
    v.z = (int)fused_word_fast<true>((uint32_t)v.z, (uint32_t)q.z, ep.add, fc);
    __builtin_amdgcn_sched_barrier(0);
    v.w = (int)fused_word_fast<true>((uint32_t)v.w, (uint32_t)q.w, ep.add, fc);
  } else if (!res16 && ep.add.relu && fast) {
    v.x = (int)fused_word_fast<false>((uint32_t)v.x, 0u, ep.add, fc);
    v.y = (int)fused_word_fast<false>((uint32_t)v.y, 0u, ep.add, fc);
    v.z = (int)fused_word_fast<false>((uint32_t)v.z, 0u, ep.add, fc);
    v.w = (int)fused_word_fast<false>((uint32_t)v.w, 0u, ep.add, fc);
  } else if (res16) {
    const int4 q = *reinterpret_cast<const int4 *>(res16);
    v.x = (int)fused_add_word((uint32_t)v.x, (uint32_t)q.x, ep.add);
    v.y = (int)fused_add_word((uint32_t)v.y, (uint32_t)q.y, ep.add);
    v.z = (int)fused_add_word((uint32_t)v.z, (uint32_t)q.z, ep.add);
    v.w = (int)fused_add_word((uint32_t)v.w, (uint32_t)q.w, ep.add);
  } else if (ep.add.relu) {
    v.x = (int)fused_relu_word((uint32_t)v.x, ep.add);
    v.y = (int)fused_relu_word((uint32_t)v.y, ep.add);
    v.z = (int)fused_relu_word((uint32_t)v.z, ep.add);
    v.w = (int)fused_relu_word((uint32_t)v.w, ep.add);
  }
  return v;
}

// The same on a residual that is already in registers (loaded ahead of the
// arithmetic that produced v, so that its latency is not waited for here).
__device__ __forceinline__ int4 fused_out_words_loaded(int4 v, int4 q, bool has_res,
                                                       const Epilogue &ep,
                                                       const FusedAddConsts &fc, bool fast) {
  if (has_res && fast) {
    v.x = (int)fused_word_fast<true>((uint32_t)v.x, (uint32_t)q.x, ep.add, fc);
    __builtin_amdgcn_sched_barrier(0);
    v.y = (int)fused_word_fast<true>((uint32_t)v.y, (uint32_t)q.y, ep.add, fc);
    __builtin_amdgcn_sched_barrier(0);
    v.z = (int)fused_word_fast<true>((uint32_t)v.z, (uint32_t)q.z, ep.add, fc);
    __builtin_amdgcn_sched_barrier(0);
    v.w = (int)fused_word_fast<true>((uint32_t)v.w, (uint32_t)q.w, ep.add, fc);
  } else if (!has_res && ep.add.relu && fast) {
    v.x = (int)fused_word_fast<false>((uint32_t)v.x, 0u, ep.add, fc);
    v.y = (int)fused_word_fast<false>((uint32_t)v.y, 0u, ep.add, fc);
    v.z = (int)fused_word_fast<false>((uint32_t)v.z, 0u, ep.add, fc);
    v.w = (int)fused_word_fast<false>((uint32_t)v.w, 0u, ep.add, fc);
  } else if (has_res) {
    v.x = (int)fused_add_word((uint32_t)v.x, (uint32_t)q.x, ep.add);
    v.y = (int)fused_add_word((uint32_t)v.y, (uint32_t)q.y, ep.add);
    v.z = (int)fused_add_word((uint32_t)v.z, (uint32_t)q.z, ep.add);
    v.w = (int)fused_add_word((uint32_t)v.w, (uint32_t)q.w, ep.add);
  } else if (ep.add.relu) {
    v.x = (int)fused_relu_word((uint32_t)v.x, ep.add);
    v.y = (int)fused_relu_word((uint32_t)v.y, ep.add);
    v.z = (int)fused_relu_word((uint32_t)v.z, ep.add);
    v.w = (int)fused_relu_word((uint32_t)v.w, ep.add);
  }
  return v;
}

// Copy-out of a staged int8 output tile (rows OUT_STRIDE = BN + 16 bytes apart
// in LDS), with the fused residual add / Relu applied on the way: 16-byte row
// segments where the output allows it. WAVE_ROWS: a wave copies out rows
// [wm * WM, wm * WM + WM) of the tile, the ones its own lanes staged; otherwise
// the block's THREADS threads share all rows.
template <int BM, int BN, int WM, int THREADS, bool WAVE_ROWS>
__device__ __forceinline__ void epilogue_copy_out(const int8_t *s_out, const Epilogue &ep, int M,
                                                  int N, int m0, int n0, int n_base, int wm) {
  constexpr int OUT_STRIDE = BN + 16;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int cols_here = min(BN, N - n0);
  const int rows_here = min(BM, M - m0);
  int8_t *obase = ep.out + (long long)m0 * ep.ldc + n_base + n0;
  const bool vec_ok = (cols_here % 16 == 0) && (ep.ldc % 16 == 0) &&
                      ((((uintptr_t)obase) & 15) == 0);
  const int8_t *rbase =
      ep.add.res ? ep.add.res + (long long)m0 * ep.ldc + n_base + n0 : nullptr;
  // WAVE_ROWS: a wave copies out the rows it staged itself (first, step, end)
  const int first = WAVE_ROWS ? lane : tid;
  constexpr int STEP = WAVE_ROWS ? 64 : THREADS;
  const int row_lo = WAVE_ROWS ? wm * WM : 0;
  const int row_n = WAVE_ROWS ? max(0, min(WM, rows_here - row_lo)) : rows_here;
  if (vec_ok && (!rbase || ((((uintptr_t)rbase) & 15) == 0))) {
    const int segs = cols_here / 16;
    // every scale small and no pre-shift in the stages that run
    const bool fast = fused_out_is_fast(ep);
    const FusedAddConsts fc = fused_add_consts(ep.add);
    // (the residual is read where it is used, a piece at a time: asking for
    // four pieces ahead costs the tiled kernels twenty registers and a wave per
    // SIMD)
    for (int c = first; c < row_n * segs; c += STEP) {
      const int r = row_lo + c / segs, s = c % segs;
      int4 v = *reinterpret_cast<const int4 *>(s_out + r * OUT_STRIDE + s * 16);
      v = fused_out_words(v, rbase ? rbase + (long long)r * ep.ldc + s * 16 : nullptr, ep, fc, fast);
      *reinterpret_cast<int4 *>(obase + (long long)r * ep.ldc + s * 16) = v;
    }
  } else {
    for (int c = first; c < row_n * cols_here; c += STEP) {
      const int r = row_lo + c / cols_here, s = c % cols_here;
      int32_t v = s_out[r * OUT_STRIDE + s];
      if (rbase) v = fused_add_one<false>(v, rbase[(long long)r * ep.ldc + s], ep.add);
      else if (ep.add.relu) v = (int32_t)(int8_t)fused_relu_word_t<false>((uint32_t)v & 0xff, ep.add);
      obase[(long long)r * ep.ldc + s] = (int8_t)v;
    }
  }
}

// f(std::integral_constant<int, I>) for I in [I0, N): a loop whose index is a
// compile-time constant in the body whatever the unroller decides.
template <int I, int N, class F> __device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// ---- requantisation from transposed accumulators ---------------------------------
// With the weights as the first matrix-core operand, lane l of a 32x32 result
// holds output row (pixel) l % 32 and, in register r, weight row
// 8 (r / 4) + 4 (l / 32) + r % 4 of the 32-row sub-tile. When the weight row that
// feeds matrix-core row rho is perm_row16(rho), register r of lane half h is
// output column 16 h + r: the sixteen accumulators of a lane are sixteen
// consecutive output bytes, requantised, packed and written with one 16-byte
// store straight from registers (no staging in LDS, no barrier).
__device__ __forceinline__ int perm_row16(int rho) {
  return 16 * ((rho >> 2) & 1) + 4 * (rho >> 3) + (rho & 3);
}

// The slot (row position in LDS) of weight row c when slots are read in
// order: the inverse of perm_row16 within each group of 32 rows.
__device__ __forceinline__ int perm_slot16(int c) {
  return (c & ~31) + 8 * ((c >> 2) & 3) + 4 * ((c >> 4) & 1) + (c & 3);
}

// A lane then needs the constants of 16 columns per sub-tile instead of one
// column's: they are kept in LDS as kParArrays arrays of BN ints (four
// consecutive columns per ds_read_b128, one address per half wave).
enum { kParColc = 0, kParPre = 1, kParScale = 2, kParPost = 3, kParFold = 4, kParArrays = 5 };

// Requantisation variants: 0 scale_i32; 1 the 24-bit multiply with pre-shift;
// 3 the 24-bit multiply without pre-shift and with the column constant folded
// (the caller's requantisation hints); LEAKY_RELU always takes 0.
__device__ __forceinline__ int requant_mode(const Epilogue &ep) {
  return ep.act == 5 ? 0 : ((ep.fast & 3) == 3 ? 3 : (ep.fast & 1));
}

// Column c's constants from its raw parameters (the arithmetic of the shared
// epilogue below).
template <int BN>
__device__ __forceinline__ void par_table_store(int32_t *s_par, int c, const ColRaw &r,
                                                const Epilogue &ep, int K, int mode) {
  uint32_t colc = (uint32_t)K * (uint32_t)ep.a_off * (uint32_t)r.woff;
  if (ep.sum_b) colc -= (uint32_t)ep.a_off * (uint32_t)r.sumb;
  if (ep.bias)
    colc += (uint32_t)scale_i32((int32_t)((uint32_t)r.bias - (uint32_t)r.boff), r.bpre, r.bpost,
                                r.bscale, 0);
  // the rounding term of the post-shift, with what the variant may fold into
  // it: the output offset (modes 1 and 3) and the column constant (mode 3)
  uint32_t fold = r.opost > 0 ? (1u << (r.opost - 1)) : 0u;
  if (mode != 0) fold += (uint32_t)ep.out_off << r.opost;
  if (mode == 3) fold += colc * (uint32_t)r.oscale;
  s_par[kParColc * BN + c] = (int32_t)colc;
  s_par[kParPre * BN + c] = r.opre;
  s_par[kParScale * BN + c] = r.oscale;
  s_par[kParPost * BN + c] = r.opost;
  s_par[kParFold * BN + c] = (int32_t)fold;
}

// Sixteen accumulators -> sixteen output bytes (before the fused add); par
// points at the first of the sixteen columns in the table.
template <int MODE, bool LEAKY, int BN>
__device__ __forceinline__ int4 requant_pack16(const v16i &acc, const int32_t *par,
                                               const Epilogue &ep, int32_t lo, int32_t hi) {
  uint32_t w[4];
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const v4i scale = *reinterpret_cast<const v4i *>(par + kParScale * BN + 4 * q);
    const v4i post = *reinterpret_cast<const v4i *>(par + kParPost * BN + 4 * q);
    v4i colc, pre;
    if constexpr (MODE != 3) {
      colc = *reinterpret_cast<const v4i *>(par + kParColc * BN + 4 * q);
      pre = *reinterpret_cast<const v4i *>(par + kParPre * BN + 4 * q);
    }
    const v4i fold = *reinterpret_cast<const v4i *>(par + kParFold * BN + 4 * q);
    uint32_t b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t x = (uint32_t)acc[4 * q + i];
      int32_t y;
      if constexpr (MODE == 3) {
        y = (int32_t)((uint32_t)__mul24((int32_t)x, scale[i]) + (uint32_t)fold[i]) >> post[i];
      } else if constexpr (MODE == 1) {
        y = (int32_t)((uint32_t)__mul24((int32_t)(x + (uint32_t)colc[i]) >> pre[i], scale[i]) +
                      (uint32_t)fold[i]) >> post[i];
      } else {
        // scale_i32 with the rounding term from the table: in this layout every
        // accumulator has its own column, so nothing per column is amortised
        const uint32_t m = (uint32_t)((int32_t)(x + (uint32_t)colc[i]) >> pre[i]) *
                               (uint32_t)scale[i] + (uint32_t)fold[i];
        y = (int32_t)((uint32_t)((int32_t)m >> post[i]) + (uint32_t)ep.out_off);
      }
      if constexpr (LEAKY) {
        if (y < ep.out_off)
          y = scale_i32((int32_t)((uint32_t)y - (uint32_t)ep.out_off), ep.a0, ep.a1, ep.a2,
                        ep.out_off);
      }
      b[i] = (uint32_t)med3_i32(y, lo, hi);
    }
    // low bytes of four registers -> one word
    const uint32_t w01 = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
    const uint32_t w23 = __builtin_amdgcn_perm(b[3], b[2], 0x0c0c0400u);
    w[q] = __builtin_amdgcn_perm(w23, w01, 0x05040100u);
  }
  return make_int4((int)w[0], (int)w[1], (int)w[2], (int)w[3]);
}

// Activation and the final int8 clip as one clamp to [lo, hi]:
// clip(min(max(y, a0), a1)) == min(max(y, clip(a0)), clip(a1)), RELU being
// the clamp [out_off, +inf) and NONE the clamp (-inf, +inf).
__device__ __forceinline__ void activation_clamp(const Epilogue &ep, int32_t &lo, int32_t &hi) {
  lo = -128;
  hi = 127;
  if (ep.act == 1) lo = clip_i8(ep.out_off);
  if (ep.act == 2) {
    lo = clip_i8(ep.a0);
    hi = clip_i8(ep.a1);
    if (lo > hi) lo = hi; // min(max(y, lo), hi) is hi then; so is the median
  }
}

// Writes sixteen requantised bytes of output row `out_row` (and residual row
// res_row, or NULL) at column n of N: one 16-byte store where the addresses
// allow it (vec) and the columns all exist, bytes otherwise.
__device__ __forceinline__ void store16(int4 v, int8_t *out_row, const int8_t *res_row, int n,
                                        int N, bool vec, const Epilogue &ep,
                                        const FusedAddConsts &fc, bool fast) {
  if (vec && n + 16 <= N) {
    v = fused_out_words(v, res_row ? res_row + n : nullptr, ep, fc, fast);
    *reinterpret_cast<int4 *>(out_row + n) = v;
    return;
  }
  // (rare: kept as a rolled loop so that it stays small next to the fast path)
#pragma unroll 1
  for (int b = 0; b < 16; b++) {
    if (n + b < N) {
      const uint32_t word = (uint32_t)(b < 4 ? v.x : b < 8 ? v.y : b < 12 ? v.z : v.w);
      int32_t x = (int32_t)(int8_t)(word >> (8 * (b & 3)));
      if (res_row) x = fused_add_one<false>(x, res_row[n + b], ep.add);
      else if (ep.add.relu) x = (int32_t)(int8_t)fused_relu_word_t<false>((uint32_t)x & 0xff, ep.add);
      out_row[n + b] = (int8_t)x;
    }
  }
}

// A wave holds the requantised results of 32 output rows as 16-byte pieces, one
// row per lane pair, staged in a wave-private LDS tile (rows `stride` bytes
// apart, `group` bytes per row: 32 to 128). Stores straight from registers
// would reach memory as 16-byte pieces of many lines (measured: 1.5 to 1.85 x
// the output bytes written at the memory side); here the tile is read back with
// group / 16 lanes per row, so that a store instruction writes whole rows of
// the group (whole 128-byte lines for a 128-byte group), with the fused residual
// add / Relu applied to words read the same way. `lane` is the lane index in
// the wave; output row r of the tile is row m0 + r of the output (rows at and
// past M are not written), its first byte of the group is column col0.
__device__ __forceinline__ void wave_fence() {
  // a wave reads back only what its own lanes wrote: LDS serves one wave's
  // accesses in order, so the compiler is all that has to be held back
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ void wave_rows_copy_out(const int8_t *s_stage, int stride, int group,
                                                   int lane, int m0, int M, int col0,
                                                   const Epilogue &ep, const FusedAddConsts &fc,
                                                   bool fast) {
  const int lpr = group / 16;                  // lanes per row
  const int rpp = 64 / lpr;                    // rows per pass
  const int rb_row = lane / lpr, rb_seg = lane - rb_row * lpr;
  for (int r0 = 0; r0 < 32; r0 += rpp) {
    const int row = r0 + rb_row, m = m0 + row;
    if (row < 32 && m < M) {
      int4 v = *reinterpret_cast<const int4 *>(s_stage + row * stride + rb_seg * 16);
      const long long at = (long long)m * ep.ldc + col0 + rb_seg * 16;
      v = fused_out_words(v, ep.add.res ? ep.add.res + at : nullptr, ep, fc, fast);
      *reinterpret_cast<int4 *>(ep.out + at) = v;
    }
  }
}

template <int BN, int WM, int WN, int MODE, bool LEAKY>
__device__ __forceinline__ void gemm_epilogue_direct_impl(
    v16i (&acc)[WM / 32][WN / 32], const int32_t *s_par, const Epilogue &ep, int M, int N,
    int m0, int n0, int n_base, int wm, int wn, int l32, int lhi) {
  constexpr int TM = WM / 32, TN = WN / 32;
  int32_t lo, hi;
  activation_clamp(ep, lo, hi);
  const bool fast = fused_out_is_fast(ep);
  const FusedAddConsts fc = fused_add_consts(ep.add);
  const bool vec = (ep.ldc % 16 == 0) && ((n_base + n0) % 16 == 0) &&
                   (((((uintptr_t)ep.out) | ((uintptr_t)ep.add.res)) & 15) == 0);
  // (compile-time indices: the accumulators must stay in registers however
  // large the unrolled body gets)
  static_for<0, TM>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
    const int m = m0 + wm * WM + i * 32 + l32;
    int8_t *out_row = ep.out + (long long)m * ep.ldc + n_base;
    const int8_t *res_row = ep.add.res ? ep.add.res + (long long)m * ep.ldc + n_base : nullptr;
    static_for<0, TN>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      const int cl = wn * WN + j * 32 + 16 * lhi;   // column within the tile
      const int4 v = requant_pack16<MODE, LEAKY, BN>(acc[i][j], s_par + cl, ep, lo, hi);
      if (m < M) store16(v, out_row, res_row, n0 + cl, N, vec, ep, fc, fast);
      // one sub-tile at a time: hoisting the next ones' table reads over this
      // one's arithmetic costs more registers than the kernels have
      __builtin_amdgcn_sched_barrier(0);
    });
  });
}

template <int BN, int WM, int WN>
__device__ __forceinline__ void gemm_epilogue_direct(
    v16i (&acc)[WM / 32][WN / 32], const int32_t *s_par, const Epilogue &ep, int M, int N,
    int m0, int n0, int n_base, int wm, int wn, int l32, int lhi) {
  const int mode = requant_mode(ep);
  if (ep.act == 5)
    gemm_epilogue_direct_impl<BN, WM, WN, 0, true>(acc, s_par, ep, M, N, m0, n0, n_base, wm, wn,
                                                   l32, lhi);
  else if (mode == 3)
    gemm_epilogue_direct_impl<BN, WM, WN, 3, false>(acc, s_par, ep, M, N, m0, n0, n_base, wm, wn,
                                                    l32, lhi);
  else if (mode == 1)
    gemm_epilogue_direct_impl<BN, WM, WN, 1, false>(acc, s_par, ep, M, N, m0, n0, n_base, wm, wn,
                                                    l32, lhi);
  else
    gemm_epilogue_direct_impl<BN, WM, WN, 0, false>(acc, s_par, ep, M, N, m0, n0, n_base, wm, wn,
                                                    l32, lhi);
}

// Shared epilogue. Accumulator layout of v_mfma_i32_32x32x32_i8: lane l holds
// column l % 32 and, in register r, row 8*(r/4) + 4*(l/32) + r%4 of the tile.
// Must be entered after a block barrier (LDS is reused).
template <int BM, int BN, int WM, int WN, bool NEED_SA, bool NEED_SB,
          bool LEAKY, int FAST = 0, bool WAVE_ROWS = false>
__device__ __forceinline__ void gemm_epilogue_impl(
    v16i (&acc)[WM / 32][WN / 32], int (&sa)[WM / 32], int (&sb)[WN / 32],
    int8_t *lds, const Epilogue &ep, int M, int N, int K, int m0, int n0,
    int n_base, const ColRaw (&col)[WN / 32]) {
  constexpr int WAVES_N = BN / WN;
  constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int OUT_STRIDE = BN + 16;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, lhi = lane >> 5;

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

  // Activation and the final int8 clip as one clamp to [lo, hi]:
  // clip(min(max(y, a0), a1)) == min(max(y, clip(a0)), clip(a1)), RELU being
  // the clamp [out_off, +inf) and NONE the clamp (-inf, +inf).
  int32_t lo = -128, hi = 127;
  if (ep.act == 1) lo = clip_i8(ep.out_off);
  if (ep.act == 2) {
    lo = clip_i8(ep.a0);
    hi = clip_i8(ep.a1);
    if (lo > hi) lo = hi; // min(max(y, lo), hi) is hi then; so is the median
  }

#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int32_t woff = col[j].woff;
    const int32_t opre = col[j].opre, opost = col[j].opost;
    const int32_t oscale = col[j].oscale;
    uint32_t colc = (uint32_t)K * (uint32_t)ep.a_off * (uint32_t)woff;
    if constexpr (NEED_SB) {
      colc -= (uint32_t)ep.a_off * (uint32_t)sb[j];
    } else if (ep.sum_b) {
      colc -= (uint32_t)ep.a_off * (uint32_t)col[j].sumb;
    }
    if (ep.bias)
      colc += (uint32_t)scale_i32((int32_t)((uint32_t)col[j].bias - (uint32_t)col[j].boff),
                                  col[j].bpre, col[j].bpost, col[j].bscale, 0);
    // FAST: the caller vouches for 24-bit operands and for room for the
    // output offset below the post-shift, so that
    //   ((x * s + rtn) >> post) + off == (x * s + (rtn + (off << post))) >> post
    // with a 24-bit multiply-add; with no pre-shift anywhere the column
    // constant goes through the multiply once per column as well. Same bits as
    // scale_i32 in half (a third) of the instruction slots: the 32-bit multiply
    // alone takes four.
    uint32_t fold = 0;
    if constexpr (FAST != 0) {
      fold = (opost > 0 ? (1u << (opost - 1)) : 0u) + ((uint32_t)ep.out_off << opost);
      if constexpr (FAST == 2) fold += colc * (uint32_t)oscale;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ml = wm * WM + i * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
        int32_t y;
        if constexpr (FAST == 2) {
          uint32_t x = (uint32_t)acc[i][j][r];
          if constexpr (NEED_SA) x -= (uint32_t)woff * (uint32_t)s_sumA[ml];
          y = (int32_t)((uint32_t)__mul24((int32_t)x, oscale) + fold) >> opost;
        } else if constexpr (FAST == 1) {
          uint32_t x = (uint32_t)acc[i][j][r] + colc;
          if constexpr (NEED_SA) x -= (uint32_t)woff * (uint32_t)s_sumA[ml];
          y = (int32_t)((uint32_t)__mul24((int32_t)x >> opre, oscale) + fold) >> opost;
        } else {
          uint32_t v = (uint32_t)acc[i][j][r] + colc;
          if constexpr (NEED_SA) v -= (uint32_t)woff * (uint32_t)s_sumA[ml];
          y = scale_i32((int32_t)v, opre, opost, oscale, ep.out_off);
        }
        if constexpr (LEAKY) {
          if (y < ep.out_off)
            y = scale_i32((int32_t)((uint32_t)y - (uint32_t)ep.out_off), ep.a0,
                          ep.a1, ep.a2, ep.out_off);
        }
        s_out[ml * OUT_STRIDE + wn * WN + j * 32 + l32] = (int8_t)med3_i32(y, lo, hi);
      }
    }
  }
  if constexpr (WAVE_ROWS) {
    // a wave reads back only what its own lanes wrote: LDS serves one wave's
    // accesses in order, so the compiler is all that has to be held back
    static_assert(BN == WN && !NEED_SA, "a wave must own whole rows of the tile");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  } else {
    __syncthreads();
  }

  epilogue_copy_out<BM, BN, WM, THREADS, WAVE_ROWS>(s_out, ep, M, N, m0, n0, n_base, wm);
}

template <int BM, int BN, int WM, int WN, bool NEED_SA, bool NEED_SB, bool WAVE_ROWS = false>
__device__ __forceinline__ void gemm_epilogue(
    v16i (&acc)[WM / 32][WN / 32], int (&sa)[WM / 32], int (&sb)[WN / 32],
    int8_t *lds, const Epilogue &ep, int M, int N, int K, int m0, int n0,
    int n_base, const ColRaw (&col)[WN / 32]) {
  if (ep.act == 5) // LEAKY_RELU: rare, kept out of the common instruction stream
    gemm_epilogue_impl<BM, BN, WM, WN, NEED_SA, NEED_SB, true, 0, WAVE_ROWS>(
        acc, sa, sb, lds, ep, M, N, K, m0, n0, n_base, col);
  else if ((ep.fast & 3) == 3)
    gemm_epilogue_impl<BM, BN, WM, WN, NEED_SA, NEED_SB, false, 2, WAVE_ROWS>(
        acc, sa, sb, lds, ep, M, N, K, m0, n0, n_base, col);
  else if (ep.fast & 1)
    gemm_epilogue_impl<BM, BN, WM, WN, NEED_SA, NEED_SB, false, 1, WAVE_ROWS>(
        acc, sa, sb, lds, ep, M, N, K, m0, n0, n_base, col);
  else
    gemm_epilogue_impl<BM, BN, WM, WN, NEED_SA, NEED_SB, false, 0, WAVE_ROWS>(
        acc, sa, sb, lds, ep, M, N, K, m0, n0, n_base, col);
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
  // Tiles are fetched into registers D K-steps ahead of their use (small tiles
  // have the registers for it): a step of this loop is short, so with one tile
  // in flight every step would wait out a full memory round trip.
  constexpr int D = (A_CH + B_CH <= 2) ? 3 : (A_CH + B_CH <= 4) ? 2 : 1;
  int4 ra[D][A_CH], rb[D][B_CH];
  auto fetch = [&](int slot, int kt) {
    const int k0 = kt * kBK;
#pragma unroll
    for (int i = 0; i < A_CH; i++) ra[slot][i] = A.template load<AL_A>(arow[i], k0 + a_k[i], K);
#pragma unroll
    for (int i = 0; i < B_CH; i++) rb[slot][i] = B.template load<AL_B>(brow[i], k0 + b_k[i], K);
  };
  auto park = [&](int slot, int8_t *stage) {
#pragma unroll
    for (int i = 0; i < A_CH; i++) *reinterpret_cast<int4 *>(stage + a_lds[i]) = ra[slot][i];
#pragma unroll
    for (int i = 0; i < B_CH; i++) *reinterpret_cast<int4 *>(stage + b_lds[i]) = rb[slot][i];
  };
  // the first tile is requested ahead of the epilogue's per-column parameters
  // (two hundred instructions of address arithmetic and null checks over ten
  // optional arrays, which then run while the tile is on its way)
  fetch(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  ColRaw col[TN];
  load_col_raw<TN, WN>(col, ep, N, n0, n_base, wn, l32);
  __builtin_amdgcn_sched_barrier(0);
  park(0, lds);
  // tiles 1..D on their way; tile t lives in register slot (t - 1) % D
#pragma unroll
  for (int t = 1; t <= D; t++)
    if (t < KT) fetch((t - 1) % D, t);
  __syncthreads();

  const int a_frag = (wm * WM + l32) * kLdsStride + lhi * 16;
  const int b_frag = (BM + wn * WN + l32) * kLdsStride + lhi * 16;

  for (int kb = 0; kb < KT; kb += D) {
#pragma unroll
    for (int u = 0; u < D; u++) {
      const int kt = kb + u;
      if (kt >= KT) break;
      const int8_t *cur = lds + (kt & 1) * STAGE;
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
      if (kt + 1 < KT) {
        // tile kt+1 sits in slot u (it was fetched D steps ago); the slot then
        // takes tile kt+1+D
        park(u, lds + ((kt + 1) & 1) * STAGE);
        if (kt + 1 + D < KT) fetch(u, kt + 1 + D);
      }
      __syncthreads();
    }
  }

  gemm_epilogue<BM, BN, WM, WN, NEED_SA, NEED_SB>(acc, sa, sb, lds, ep, M, N, K,
                                                  m0, n0, n_base, col);
}

// ---- direct-to-LDS main loop ---------------------------------------------------

// 16 bytes per lane from global memory straight into LDS at
// lds_addr + 16 * lane (M0 carries the wave-uniform LDS address). Issued
// through inline assembly so that the compiler's own wait-count insertion
// does not serialise later LDS reads against loads still in flight; the
// kernel below waits explicitly with dma_wait<N>().
// The same with the LDS address given as the sum of two wave-uniform parts
// (a ring slot's offset and the load's place in the slot): the scalar add
// writes M0 itself.
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_a, uint32_t lds_b) {
  asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off"
               :
               : "s"(lds_a), "s"(lds_b), "v"(gptr)
               : "memory", "scc");
}

__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr), "v"(gptr)
               : "memory");
}

// Waits until at most N of this wave's vector-memory operations are pending.
template <int N> __device__ __forceinline__ void dma_wait() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Bytes whose value equals their row index: row v of this table is a 16-byte
// chunk filled with the byte v. Out-of-image convolution taps are loaded from
// it (a direct-to-LDS load cannot synthesise a constant).
struct FillTable {
  uint8_t b[256 * 16];
  constexpr FillTable() : b{} {
    for (int i = 0; i < 256 * 16; i++) b[i] = (uint8_t)(i / 16);
  }
};
__device__ __attribute__((aligned(16))) const FillTable g_fill_table{};

__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(
      (const __attribute__((address_space(3))) void *)p);
}

// SHORT: the K loop has fewer steps than the ring has slots and the launch
// provides LDS for those KT slots only, so that more workgroups share a CU
// (what such a layer needs: it is all load latency and epilogue). Re-reads
// past the end then go to the last tile's own slot (the same bytes again)
// instead of slots nobody consumes. Only the 128x128 tile without in-kernel
// row sums has this variant; it is compiled for four waves per SIMD.
// K split over workgroups (blockIdx.z = the split): every workgroup of an
// output tile multiplies its share of the K steps and leaves its int32
// accumulators in the caller's workspace; the one that arrives last at the
// tile's counter adds the others' to its own (int32 sums wrap, so the order
// does not matter: the reference's sum, libjit_matmul.cpp:284-316) and runs the
// epilogue. Nobody waits for anybody. Counters are zero before a launch and
// are left zero by it.
struct SplitK {
  int32_t *partials = nullptr;   // [group][tile][split][BM * BN], in the accumulators' own order
  uint32_t *counters = nullptr;  // [group][tile]
  int splits = 1;
};

template <int BM, int BN, int WM, int WN, int STAGES, bool NEED_SA,
          bool NEED_SB, class ARows, bool SHORT = false, bool SPLITK = false>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64,
                             ((BM / WM) * (BN / WN) == 8 && BM * BN <= 256 * 128)
                                 ? (BM * BN == 256 * 128 ? 1 : 2)
                             : (BM * BN == 256 * 128) ? 2
                             : SHORT                  ? 4
                             : (BM * BN == 128 * 128) ? 3
                                                      : 1) void gemm_i8_dma_kernel(
    ARows A, DenseRows B, Epilogue ep, int M, int N, int K, int tiles_m,
    int tiles_n, long long b_group_stride, int n_per_group, SplitK sk) {
  static_assert(!SPLITK || (!NEED_SA && !NEED_SB && !SHORT), "split K: no in-kernel row sums");
  constexpr int WAVES_N = BN / WN;
  constexpr int WAVES = (BM / WM) * (BN / WN);
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int STAGE = (BM + BN) * kBK;             // bytes per ring slot
  // one load instruction moves a group of 16 rows x 64 bytes
  constexpr int A_LOADS = BM / 16 / WAVES, B_LOADS = BN / 16 / WAVES;
  constexpr int LOADS = A_LOADS + B_LOADS;
  static_assert(BM / 16 % WAVES == 0 && BN / 16 % WAVES == 0, "tile vs waves");
  static_assert(STAGES >= 3 && (STAGES - 1) * LOADS < 64, "ring depth");

  extern __shared__ __attribute__((aligned(16))) int8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, lhi = lane >> 5;

  const int grp = blockIdx.y;
  A.set_group(grp);
  B.p += (long long)grp * b_group_stride;
  const int n_base = grp * n_per_group;

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // Load plan. Lane i of a group load owns row (i >> 2) of the group and the
  // LDS chunk position (i & 3); the chunk stored there is kc = pos ^ swizzle.
  const int row_in_grp = lane >> 2;
  const int kc_lane = ((lane & 3) ^ ((lane >> 4) & 3)) * 16;
  typename ARows::Row arow[A_LOADS];
  const int8_t *bptr[B_LOADS];
  uint32_t a_dst[A_LOADS], b_dst[B_LOADS];
  const uint32_t lds0 = lds_address(lds);
#pragma unroll
  for (int i = 0; i < A_LOADS; i++) {
    const int g = i * WAVES + wave;
    arow[i] = A.row(min(m0 + g * 16 + row_in_grp, M - 1));
    a_dst[i] = lds0 + g * 1024;
  }
#pragma unroll
  for (int i = 0; i < B_LOADS; i++) {
    const int g = i * WAVES + wave;
    bptr[i] = B.p + (long long)min(n0 + g * 16 + row_in_grp, N - 1) * B.ld + kc_lane;
    b_dst[i] = lds0 + BM * kBK + g * 1024;
  }

  // this workgroup's K steps: all of them, or its share (every split has at
  // least one: the launch sees to that)
  int KT = K / kBK, k_begin = 0;
  if constexpr (SPLITK) {
    const int per = (KT + sk.splits - 1) / sk.splits;
    k_begin = (int)blockIdx.z * per * kBK;
    KT = min(per, KT - (int)blockIdx.z * per);
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) bptr[i] += k_begin;
  }
  // A tile's loads are issued in two halves, H0 then H1, so that the memory
  // pipeline sees a steady trickle instead of one burst per K step.
  constexpr int H0 = LOADS / 2;
  // `loc` is A.locate() of this lane's chunk of tile nk (one locate serves
  // every row of the tile and both halves of its loads)
  // Tiles are located in order, one K step at a time (nk never decreases and
  // grows by at most one between calls; past the end the last tile stays).
  typename ARows::Loc run_loc = A.locate(kc_lane + k_begin);
  int run_tile = 0;
  auto locate_tile = [&](int nk) {
    const int t = min(nk, KT - 1);
    if (t != run_tile) {
      A.advance(run_loc);
      run_tile = t;
    }
    return run_loc;
  };
  // `ring` is the byte offset of the ring slot tile nk goes to (slot nk %
  // STAGES, carried by the caller instead of divided out for every load) and
  // k0 the tile's K offset, already clamped to the last tile
  auto issue_load = [&](int nk, uint32_t ring, int k0, int i, const typename ARows::Loc &loc) {
    const uint32_t slot = SHORT ? (uint32_t)min(nk, KT - 1) * STAGE : ring;
    if (i < A_LOADS)
      dma16(A.chunk_ptr(arow[i], loc), slot, a_dst[i]);
    else
      dma16(bptr[i - A_LOADS] + k0, slot, b_dst[i - A_LOADS]);
  };
  // prologue: tiles 0..STAGES-2 and the first half of tile STAGES-1 in flight
  // (tiles past the end are re-reads of the last one into slots nobody
  // consumes, which keeps the counts uniform). The columns' constants, which
  // the epilogue consumes, are requested behind tile 0: the first multiply
  // waits for that tile, and the constants' address arithmetic (ten optional
  // arrays) then runs while it is on its way.
  ColRaw col[TN];
#pragma unroll
  for (int s = 0; s < STAGES - 1; s++) {
    const typename ARows::Loc loc = locate_tile(s);
#pragma unroll
    for (int i = 0; i < LOADS; i++) issue_load(s, s * STAGE, min(s, KT - 1) * kBK, i, loc);
    if (s == 0) {
      __builtin_amdgcn_sched_barrier(0);
      load_col_raw<TN, WN>(col, ep, N, n0, n_base, wn, l32);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // the tile whose second half is still to be requested
  typename ARows::Loc half_loc = locate_tile(STAGES - 1);
#pragma unroll
  for (int i = 0; i < H0; i++)
    issue_load(STAGES - 1, (STAGES - 1) * STAGE, min(STAGES - 1, KT - 1) * kBK, i, half_loc);

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

  // fragment addresses: row (l & 31) of a 32-row sub-tile, chunk ks*2 + (l>>5)
  const int swz = (lane >> 2) & 3;
  int frag_off[kBK / 32];
#pragma unroll
  for (int ks = 0; ks < kBK / 32; ks++)
    frag_off[ks] = l32 * kBK + (((ks * 2 + lhi) ^ swz) << 4);
  const int a_base = wm * WM * kBK;
  const int b_base = BM * kBK + wn * WN * kBK;

  static_assert(kBK == 64 && STAGES >= 3, "two 32-byte k slices per stage");
  v4i af[2][TM], bf[2][TN];
  // fragment f of a k slice: the TM A fragments, then the TN B fragments
  auto read_frag = [&](const int8_t *stage, int ks, int buf, int f) {
    if (f < TM)
      af[buf][f] = *reinterpret_cast<const v4i *>(stage + a_base + f * 32 * kBK + frag_off[ks]);
    else
      bf[buf][f - TM] = *reinterpret_cast<const v4i *>(stage + b_base + (f - TM) * 32 * kBK + frag_off[ks]);
  };
  // The MFMAs of one k slice with the memory operations of the next slice
  // spread between them: a wave issues in order, so a burst of loads that
  // fills the memory queues would hold back the MFMAs queued behind it.
  auto multiply = [&](int buf, auto &&between) {
    if constexpr (NEED_SA) {
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int q = 0; q < 4; q++)
          sa[i] = __builtin_amdgcn_sdot4(af[buf][i][q], 0x01010101, sa[i], false);
    }
    if constexpr (NEED_SB) {
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int q = 0; q < 4; q++)
          sb[j] = __builtin_amdgcn_sdot4(bf[buf][j][q], 0x01010101, sb[j], false);
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[buf][i], bf[buf][j],
                                                          acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        between(i * TN + j);
        __builtin_amdgcn_sched_barrier(0);
      }
  };
  constexpr int MFMAS = TM * TN;
  constexpr int FRAGS = TM + TN;
  // Fragment read f is slotted in after MFMA t when f is in
  // [t*FRAGS/MFMAS, (t+1)*FRAGS/MFMAS): spread evenly, each in the last slot
  // of its interval. Load x of n goes to the middle of its interval, which are
  // the slots the reads leave empty when there are fewer operations than
  // MFMAs (a read and a load behind the same MFMA take longer to issue than
  // the MFMA runs, which stalls the next one).
  auto frags_in_slot = [&](int t, const int8_t *stage, int ks, int buf) {
#pragma unroll
    for (int f = t * FRAGS / MFMAS; f < (t + 1) * FRAGS / MFMAS; f++)
      read_frag(stage, ks, buf, f);
  };
  auto loads_in_slot = [&](int t, int nk, uint32_t ring, int k0, int first, int n,
                           const typename ARows::Loc &loc) {
#pragma unroll
    for (int x = 0; x < n; x++)
      if (min(MFMAS - 1, (2 * x + 1) * MFMAS / (2 * n)) == t)
        issue_load(nk, ring, k0, first + x, loc);
  };

  // tile 0 has landed once only the newer requests are pending
  dma_wait<(STAGES - 2) * LOADS + H0>();
  __syncthreads();
#pragma unroll
  for (int f = 0; f < FRAGS; f++) read_frag(lds, 0, 0, f);
  // Ring positions and K offsets are carried from step to step: the slot of
  // tile kt, of tile kt-1 (which tile kt+STAGES-1 takes over) and the clamped K
  // offsets of the two tiles a step requests. One wave per SIMD issues an
  // instruction every four cycles at best, so every scalar instruction of this
  // bookkeeping is time the matrix cores idle when workgroups are few.
  uint32_t ring_cur = 0, ring_prev = (STAGES - 1) * STAGE; // byte offsets
  const int k_last = (KT - 1) * kBK;
  int k_far0 = min(STAGES - 1, KT - 1) * kBK; // tile kt+STAGES-1
  int k_far1 = min(STAGES, KT - 1) * kBK;     // tile kt+STAGES
  for (int kt = 0; kt < KT; kt++) {
    const uint32_t ring_next = ring_cur + STAGE == STAGES * STAGE ? 0u : ring_cur + STAGE;
    const int8_t *cur = lds + (SHORT ? (uint32_t)kt * STAGE : ring_cur);
    // (the fragments read past the end are not used)
    const int8_t *nxt = lds + (SHORT ? (uint32_t)min(kt + 1, KT - 1) * STAGE : ring_next);
    // slice 0 runs while the fragments of slice 1 arrive and the second half
    // of tile kt+STAGES-1 is requested (its slot held tile kt-1, which every
    // wave had read before the previous barrier)
    multiply(0, [&](int t) {
      frags_in_slot(t, cur, 1, 1);
      loads_in_slot(t, kt + STAGES - 1, ring_prev, k_far0, H0, LOADS - H0, half_loc);
    });
    // tile kt+1 has landed once only tiles kt+2..kt+STAGES-1 are pending; past
    // the barrier every wave holds tile kt in registers, so its slot is free
    dma_wait<(STAGES - 2) * LOADS>();
    __syncthreads();
    // slice 1 runs while slice 0 of the next tile is read and the first half
    // of tile kt+STAGES is requested into the slot of tile kt
    half_loc = locate_tile(kt + STAGES);
    multiply(1, [&](int t) {
      frags_in_slot(t, nxt, 0, 0);
      loads_in_slot(t, kt + STAGES, ring_cur, k_far1, 0, H0, half_loc);
    });
    ring_prev = ring_cur;
    ring_cur = ring_next;
    k_far0 = min(k_far0 + kBK, k_last);
    k_far1 = min(k_far1 + kBK, k_last);
  }
  dma_wait<0>(); // drain the re-reads before LDS is reused
  __syncthreads();
  if constexpr (SPLITK) {
    constexpr int THREADS = WAVES * 64;
    const size_t tile_id = (size_t)grp * ((size_t)tiles_m * tiles_n) + blockIdx.x;
    int32_t *mine = sk.partials + (tile_id * sk.splits + blockIdx.z) * (size_t)(BM * BN);
    // Accumulators as they lie in the registers: value v of a lane at
    // [v][thread]. The sums pass between workgroups that may sit on different
    // dies, each with an L2 of its own: they are stored and loaded as
    // device-scope accesses (written through to, and read from, the memory
    // side), which costs nothing beyond the access itself. A device-scope
    // fence would write back and invalidate the whole L2 once per workgroup
    // (measured: 65 us on top of a 20 us launch).
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          __hip_atomic_store(mine + ((i * TN + j) * 16 + r) * THREADS + tid, acc[i][j][r],
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // Every store of this workgroup has been acknowledged before its arrival
    // is counted: each wave waits for its own stores (a workgroup-scope
    // release fence does not: it orders the waves of a CU through their
    // shared cache, which these stores pass by), then the waves meet.
    dma_wait<0>();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    uint32_t *s_arrived = reinterpret_cast<uint32_t *>(lds);
    if (tid == 0)
      *s_arrived = __hip_atomic_fetch_add(sk.counters + tile_id, 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const uint32_t arrived = *s_arrived;
    __syncthreads();                  // LDS is the epilogue's from here on
    if (arrived != (uint32_t)sk.splits - 1) return;   // the whole workgroup leaves
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    for (int s = 0; s < sk.splits; s++) {
      if (s == (int)blockIdx.z) continue;
      const int32_t *theirs = sk.partials + (tile_id * sk.splits + s) * (size_t)(BM * BN);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int r = 0; r < 16; r++)
            acc[i][j][r] += __hip_atomic_load(theirs + ((i * TN + j) * 16 + r) * THREADS + tid,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (tid == 0)                     // as the next launch expects it
      __hip_atomic_store(sk.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  gemm_epilogue<BM, BN, WM, WN, NEED_SA, NEED_SB>(acc, sa, sb, lds, ep, M, N, K,
                                                  m0, n0, n_base, col);
}

template <int BM, int BN> constexpr size_t gemm_epilogue_lds_bytes() {
  return (size_t)BM * 4 + (size_t)BM * (BN + 16);
}

template <int BM, int BN> constexpr size_t gemm_lds_bytes() {
  constexpr size_t stages = 2 * (size_t)(BM + BN) * kLdsStride;
  constexpr size_t epi = gemm_epilogue_lds_bytes<BM, BN>();
  return stages > epi ? stages : epi;
}

template <int BM, int BN, int STAGES> constexpr size_t gemm_dma_lds_bytes() {
  constexpr size_t ring = (size_t)STAGES * (BM + BN) * kBK;
  constexpr size_t epi = gemm_epilogue_lds_bytes<BM, BN>();
  return ring > epi ? ring : epi;
}

// LDS a block may use on the current device (cached per process).
static size_t lds_limit() {
  static std::atomic<size_t> limit{0};
  size_t v = limit.load(std::memory_order_relaxed);
  if (!v) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipGetDeviceProperties(&p, dev) == hipSuccess)
      v = p.sharedMemPerBlock;
    else
      v = 64 * 1024;
    limit.store(v, std::memory_order_relaxed);
  }
  return v;
}

// Kernels that want more than 48 KiB of dynamic LDS have to say so once per
// device; `done` holds one bit per device (any host thread may get here first,
// setting the attribute twice is harmless).
template <class Kern>
static int set_lds_attr(Kern kern, size_t lds, std::atomic<uint64_t> &done) {
  if (lds <= 48 * 1024) return MI355X_OK;
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  const uint64_t bit = 1ull << (dev & 63);
  if (!(done.load(std::memory_order_acquire) & bit)) {
    MI355X_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)lds));
    done.fetch_or(bit, std::memory_order_release);
  }
  return MI355X_OK;
}

struct GemmShape {
  int M, N, K, groups;
  long long b_group_stride;
};

// Launches one tile configuration of the register-staged kernel. `groups` > 1
// is the grouped convolution.
template <int BM, int BN, int WM, int WN, bool AL_A, bool AL_B, class ARows>
static int gemm_launch(const ARows &A, const DenseRows &B, const Epilogue &ep,
                       const GemmShape &g, hipStream_t st) {
  constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
  constexpr size_t lds = gemm_lds_bytes<BM, BN>();
  auto kern = gemm_i8_kernel<BM, BN, WM, WN, true, true, AL_A, AL_B, ARows>;
  static std::atomic<uint64_t> attr_set{0}; // per instantiation, one bit per device
  int rc = set_lds_attr(kern, lds, attr_set);
  if (rc != MI355X_OK) return rc;
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  const long long total = (long long)tiles_m * tiles_n;
  MI355X_REQUIRE(total < 0x7fffffffLL && g.groups < 65536, "problem too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)g.groups),
                     dim3(THREADS), lds, st, A, B, ep, g.M, g.N, g.K, tiles_m,
                     tiles_n, g.b_group_stride, g.N);
  return check_launch("gemm_i8");
}

// Same for the direct-to-LDS kernel.
template <int BM, int BN, int WM, int WN, int STAGES, bool SA, bool SB,
          class ARows>
static int gemm_dma_launch(const ARows &A, const DenseRows &B,
                           const Epilogue &ep, const GemmShape &g,
                           hipStream_t st) {
  constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
  constexpr size_t lds = gemm_dma_lds_bytes<BM, BN, STAGES>();
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  const long long total = (long long)tiles_m * tiles_n;
  MI355X_REQUIRE(total < 0x7fffffffLL && g.groups < 65536, "problem too large");
  if constexpr (BM == 128 && BN == 128 && !SA && !SB) {
    const int KT = g.K / kBK;
    if (KT < STAGES) {
      // KT ring slots (or the epilogue's staging area if that is larger): under
      // 48 KiB, so no attribute is needed
      const size_t ring = (size_t)KT * (BM + BN) * kBK;
      const size_t epi = gemm_epilogue_lds_bytes<BM, BN>();
      hipLaunchKernelGGL((gemm_i8_dma_kernel<BM, BN, WM, WN, STAGES, SA, SB, ARows, true>),
                         dim3((unsigned)total, (unsigned)g.groups), dim3(THREADS),
                         ring > epi ? ring : epi, st, A, B, ep, g.M, g.N, g.K, tiles_m,
                         tiles_n, g.b_group_stride, g.N, SplitK{});
      return check_launch("gemm_i8_dma");
    }
  }
  auto kern = gemm_i8_dma_kernel<BM, BN, WM, WN, STAGES, SA, SB, ARows>;
  static std::atomic<uint64_t> attr_set{0}; // per instantiation, one bit per device
  int rc = set_lds_attr(kern, lds, attr_set);
  if (rc != MI355X_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)g.groups),
                     dim3(THREADS), lds, st, A, B, ep, g.M, g.N, g.K, tiles_m,
                     tiles_n, g.b_group_stride, g.N, SplitK{});
  return check_launch("gemm_i8_dma");
}

// The 128x128 tile of eight waves with K split over `splits` workgroups per
// output tile (see SplitK). The workspace holds the tiles' counters (zero
// before the launch, zero after it), then the partial sums.
constexpr size_t kSplitTile = 128;
static size_t splitk_counter_bytes(const GemmShape &g) {
  const size_t tiles = ((g.M + kSplitTile - 1) / kSplitTile) * ((g.N + kSplitTile - 1) / kSplitTile);
  return (tiles * (size_t)g.groups * sizeof(uint32_t) + 255) & ~(size_t)255;
}
static size_t splitk_workspace_bytes(const GemmShape &g, int splits) {
  const size_t tiles = ((g.M + kSplitTile - 1) / kSplitTile) * ((g.N + kSplitTile - 1) / kSplitTile);
  return splitk_counter_bytes(g) +
         tiles * (size_t)g.groups * (size_t)splits * kSplitTile * kSplitTile * sizeof(int32_t);
}
// How many workgroups share an output tile's K loop: enough to give every CU
// one, at most four, each with at least 32 K steps (handing the sums over costs
// about what 24 steps take: measured, K of 4608 over 100 tiles 22.5 -> 19.8 us,
// K of 2048 9.9 -> 13.3 us); 1 = not split (the grid already fills half the
// chip, or K is short).
// forced (the caller named the tile): at least two whenever K has two steps.
static int splitk_choice(const GemmShape &g, int cus, bool forced) {
  const long long tiles = (long long)((g.M + kSplitTile - 1) / kSplitTile) *
                          ((g.N + kSplitTile - 1) / kSplitTile) * g.groups;
  const int KT = g.K / kBK;
  int s = 1;
  if (tiles > 0 && tiles * 2 <= cus) {
    s = (int)std::min<long long>(4, cus / tiles);
    while (s > 1 && KT / s < 32) s--;
  }
  if (forced && s < 2 && KT >= 2) s = 2;
  return s;
}

static int gemm_cus() {
  static std::atomic<int> cached{0};
  int v = cached.load(std::memory_order_relaxed);
  if (v > 0) return v;
  int dev = 0;
  v = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
    v = 256;
  cached.store(v, std::memory_order_relaxed);
  return v;
}

template <class ARows>
static int gemm_dma_launch_splitk(const ARows &A, const DenseRows &B, const Epilogue &ep,
                                  const GemmShape &g, int splits, void *workspace,
                                  hipStream_t st) {
  constexpr int BM = 128, BN = 128, WM = 64, WN = 32, STAGES = 3;
  constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
  constexpr size_t lds = gemm_dma_lds_bytes<BM, BN, STAGES>();
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  const long long total = (long long)tiles_m * tiles_n;
  MI355X_REQUIRE(total < 0x7fffffffLL && g.groups < 65536 && splits >= 2 && splits <= 64,
                 "problem too large");
  // every split has at least one K step (the kernel counts on it)
  const int KT = g.K / kBK, per = (KT + splits - 1) / splits;
  MI355X_REQUIRE(g.K % kBK == 0 && (splits - 1) * per < KT, "K of %d cannot be split %d ways",
                 g.K, splits);
  auto kern = gemm_i8_dma_kernel<BM, BN, WM, WN, STAGES, false, false, ARows, false, true>;
  static std::atomic<uint64_t> attr_set{0}; // per instantiation, one bit per device
  int rc = set_lds_attr(kern, lds, attr_set);
  if (rc != MI355X_OK) return rc;
  SplitK sk;
  sk.counters = reinterpret_cast<uint32_t *>(workspace);
  sk.partials = reinterpret_cast<int32_t *>(reinterpret_cast<uint8_t *>(workspace) +
                                            splitk_counter_bytes(g));
  sk.splits = splits;
  hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)g.groups, (unsigned)splits),
                     dim3(THREADS), lds, st, A, B, ep, g.M, g.N, g.K, tiles_m, tiles_n,
                     g.b_group_stride, g.N, sk);
  return check_launch("gemm_i8_dma_splitk");
}

// Tile choice from the problem size: 256x256 for large problems (a wave owns
// 128x128, which halves LDS traffic per MFMA), smaller tiles when the grid
// would otherwise not fill 256 CUs.
enum class Tile { T256, T128, T128x64, T64, T256x128, T128x256, T128w8 = 9, T256x128w8 = 10, T256w8 = 11 };
// g_tile_override (common.h) in [0, 5] or [9, 11] forces that tile for the launch
// being issued (w8: eight waves per workgroup instead of four).
static Tile pick_tile(const GemmShape &g, size_t lds_256) {
  auto tiles = [&](int bm, int bn) {
    return (long long)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * g.groups;
  };
  if (((g_tile_override >= 0 && g_tile_override <= 5) ||
       (g_tile_override >= 9 && g_tile_override <= 11)) &&
      ((g_tile_override != 0 && g_tile_override != 11) || lds_256 <= lds_limit()))
    return (Tile)g_tile_override;
  // Measured on the convolution shapes of ResNet-50 and on large FCs. The big
  // tiles run with eight waves (two per SIMD: one wave's fragment reads and
  // bookkeeping hide behind the other's matrix-core work), which beat their
  // four-wave forms on every large shape tried (us, four waves / eight):
  // M8192 K4096 N4096 137.8 / 130.4, M16384 K2048 N4096 161.2 / 144.3,
  // M16384 K1024 N1024 30.4 / 25.9, M32768 K2048 N1024 83.7 / 74.9. 256x256
  // needs a grid that fills the chip; below that 256x128, then 128x128, then
  // many small resident workgroups; few-row problems want 64x64.
  if (tiles(256, 256) >= 256 && g.N >= 256 && g.K >= 1024 && lds_256 <= lds_limit())
    return Tile::T256w8;
  // two workgroups per CU, so one workgroup's epilogue overlaps the other's loads
  if (tiles(256, 128) >= 256 && g.N >= 256) return Tile::T256x128;
  if (tiles(128, 128) >= 256 && g.N >= 128 && g.K >= 512) return Tile::T128w8;
  if (tiles(128, 64) >= 256) return Tile::T128x64;
  if (tiles(64, 64) >= 256 || g.M < 1024) return Tile::T64;
  return Tile::T128x64;
}

constexpr int kTileSplitK = 12;   // tile number of the K-split launch

template <bool SA, bool SB, class ARows>
static int gemm_dma_tiles(const ARows &A, const DenseRows &B, const Epilogue &ep,
                          const GemmShape &g, hipStream_t st) {
  // K split over workgroups: when the call brings a workspace and the grid
  // would leave half the chip idle, or when the call names the tile
  const bool named = g_tile_override == kTileSplitK;
  if (named || (g_tile_override < 0 && g_workspace)) {
    if constexpr (!SA && !SB) {
      const int splits = splitk_choice(g, gemm_cus(), named);
      if (splits >= 2 && g_workspace && (((uintptr_t)g_workspace) & 255) == 0 &&
          g_workspace_bytes >= splitk_workspace_bytes(g, splits))
        return gemm_dma_launch_splitk(A, B, ep, g, splits, g_workspace, st);
      if (named)
        return fail(MI355X_ERR_NOT_SUPPORTED,
                    "tile %d (K split over workgroups) needs two K steps and a 256-byte "
                    "aligned workspace of %zu bytes in the launch's options",
                    kTileSplitK, splitk_workspace_bytes(g, splits < 2 ? 2 : splits));
    } else if (named) {
      return fail(MI355X_ERR_NOT_SUPPORTED,
                  "tile %d (K split over workgroups) needs precomputed weight row sums and "
                  "zero weight offsets", kTileSplitK);
    }
  }
  switch (pick_tile(g, gemm_dma_lds_bytes<256, 256, 4>())) {
  case Tile::T256:
    return gemm_dma_launch<256, 256, 128, 128, 4, SA, SB>(A, B, ep, g, st);
  case Tile::T128:
    return gemm_dma_launch<128, 128, 64, 64, 3, SA, SB>(A, B, ep, g, st);
  case Tile::T128x64:
    return gemm_dma_launch<128, 64, 32, 64, 3, SA, SB>(A, B, ep, g, st);
  case Tile::T256x128:
    return gemm_dma_launch<256, 128, 128, 64, 3, SA, SB>(A, B, ep, g, st);
  case Tile::T128x256:
    return gemm_dma_launch<128, 256, 64, 128, 3, SA, SB>(A, B, ep, g, st);
  case Tile::T128w8:
    return gemm_dma_launch<128, 128, 64, 32, 3, SA, SB>(A, B, ep, g, st);
  case Tile::T256x128w8:
    return gemm_dma_launch<256, 128, 64, 64, 3, SA, SB>(A, B, ep, g, st);
  case Tile::T256w8:
    return gemm_dma_launch<256, 256, 128, 64, 4, SA, SB>(A, B, ep, g, st);
  default:
    return gemm_dma_launch<64, 64, 32, 32, 4, SA, SB>(A, B, ep, g, st);
  }
}

template <bool AL_A, bool AL_B, class ARows>
static int gemm_staged_tiles(const ARows &A, const DenseRows &B,
                             const Epilogue &ep, const GemmShape &g,
                             hipStream_t st) {
  switch (pick_tile(g, gemm_lds_bytes<256, 256>())) {
  case Tile::T256:
    return gemm_launch<256, 256, 128, 128, AL_A, AL_B>(A, B, ep, g, st);
  case Tile::T128:
    return gemm_launch<128, 128, 64, 64, AL_A, AL_B>(A, B, ep, g, st);
  case Tile::T128x64:
    return gemm_launch<128, 64, 32, 64, AL_A, AL_B>(A, B, ep, g, st);
  case Tile::T256x128:
  case Tile::T128x256:
  case Tile::T128w8:
  case Tile::T256x128w8:
  case Tile::T256w8:
    return gemm_launch<128, 128, 64, 64, AL_A, AL_B>(A, B, ep, g, st);
  default:
    return gemm_launch<64, 64, 32, 32, AL_A, AL_B>(A, B, ep, g, st);
  }
}

// need_sa / need_sb: whether the row sums of A / B have to be formed inside
// the kernel (a non-zero B offset; a non-zero A offset without precomputed
// ep.sum_b). aligned: both operands allow 16-byte chunk
// loads (16-byte aligned rows; for convolutions also IC/group % 16 == 0).
template <class ARows>
static int gemm_dispatch(const ARows &A, const DenseRows &B, const Epilogue &ep_in,
                         int M, int N, int K, int groups,
                         long long b_group_stride, bool need_sa, bool need_sb,
                         bool aligned, hipStream_t st) {
  const GemmShape g{M, N, K, groups, b_group_stride};
  Epilogue ep = ep_in;
  ep.fast = g_requant_hint & 3;
  if (aligned && K >= kBK && K % kBK == 0) {
    if (need_sa && need_sb) return gemm_dma_tiles<true, true>(A, B, ep, g, st);
    if (need_sa) return gemm_dma_tiles<true, false>(A, B, ep, g, st);
    if (need_sb) return gemm_dma_tiles<false, true>(A, B, ep, g, st);
    return gemm_dma_tiles<false, false>(A, B, ep, g, st);
  }
  if (g_tile_override == kTileSplitK)
    return fail(MI355X_ERR_NOT_SUPPORTED,
                "tile %d (K split over workgroups) needs K a multiple of 64 and 16-byte "
                "aligned operands", kTileSplitK);
  // K tails and unaligned operands: register-staged loop, both row sums kept
  if (aligned) return gemm_staged_tiles<true, true>(A, B, ep, g, st);
  return gemm_staged_tiles<false, false>(A, B, ep, g, st);
}

} // namespace mi355x
#endif
