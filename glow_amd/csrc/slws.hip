// FusedRowwiseQuantizedSparseLengthsWeightedSum / Sum and the offsets-based
// EmbeddingBag twin, for 8-bit and 4-bit fused rows with fp32 or fp16
// scale/offset (reference lib/LLVMIRCodeGen/libjit/libjit.cpp:1253-1276,
// 2454-2481; lib/Backends/Interpreter/InterpreterNodes.cpp:5764-5889).
//
// One bag per group of LPB lanes (a whole 64-lane wavefront for rows of 64+
// data bytes, so every row read is one coalesced request). A lane owns BPL
// consecutive data bytes of the row and keeps their running sums in
// registers. For each batch of up to 64 lookups lane j first fetches index j,
// weight j and the (scale, offset) pair of row j; then all row reads of the
// batch are issued back to back before the first one is consumed, so a bag
// costs three dependent memory round trips however long it is. The sums are
// formed in bag order with separately rounded multiply and add, which
// reproduces the CPU loop bit for bit.
//
// In the wavefront-per-bag kernel the per-lookup values (row byte offset,
// weight, scale, offset) are handed from lane j to the whole wave through a
// wave-private LDS slot read back at a uniform address (a broadcast), which
// keeps the vector ALU for the five operations per element the arithmetic
// needs (convert, multiply, add, multiply, add).
//
// That is the strict form of the arithmetic (slws_kernel, slws_wave_kernel;
// MI355X_SLWS_MATH_STRICT). By default rows of 32, 64, 128 or 256 data bytes
// with fp32 accumulation run the fused kernels further down (slws_rows_kernel,
// slws_groups_kernel): the CPU loop's own expression per element in bag order,
// with two fused multiply-adds (MI355X_SLWS_MATH_ELEMENT), or on request the
// sum regrouped into one fused multiply-add per element (_REGROUPED). A call
// names its arithmetic in mi355x_launch_opts; mi355x_slws_set_fused_math sets
// what the calls that name none get.
//
// The start of a bag in the index list is the exclusive prefix sum of the
// lengths. A block sums the lengths in front of it itself (from the start of
// its chunk of kChunkBags bags, plus one pre-summed value per earlier chunk),
// which keeps the common small-batch case at a single launch.
#include "common.h"

// Every multiply and add below must round on its own (the CPU code this
// reproduces has no fused multiply-add). The pragma covers contraction in the
// front end; the build must also pass -ffp-contract=off (the Makefile does),
// because HIP's default "fast" mode fuses in the back end regardless.
#pragma clang fp contract(off)

#include <hip/hip_fp16.h>

#include <atomic>
#include <type_traits>
#include <mutex>
#include <vector>

namespace mi355x {

constexpr int kSlwsThreads = 256;
constexpr int kBatch = 64;         // lookups fetched per round
constexpr int kChunkBags = 4096;   // bags per pre-summed chunk
constexpr int kMaxChunks = 32768;  // workspace entries (int64 each)
// Bags per block of slws_rows_kernel: sixteen (one block of 1024 threads per CU
// at 4096 bags: the lengths in front of a block are summed once per CU) up to
// kRowsWideBags bags per launch, eight beyond (measured: 3 % faster at 4096
// bags, level at 16 384, 6 % slower at 65 536).
constexpr int kRowsWaves = 16, kRowsWavesMany = 8;
constexpr size_t kRowsWideBags = 16384;
__host__ __device__ constexpr int rows_waves(size_t bags) {
  return bags < kRowsWideBags ? kRowsWaves : kRowsWavesMany;
}

struct SlwsArgs {
  void *dest;
  const uint8_t *data;
  const void *weights;     // fp32 / fp16 / NULL
  const void *indices;     // int64 / int32
  const int32_t *lengths;  // lengths mode
  const int32_t *offsets;  // offsets mode (NULL in lengths mode)
  const int64_t *chunk_sums; // lengths mode with more than one chunk
  int64_t data_rows;
  int64_t num_indices;
  int64_t segments;        // number of output rows
  int32_t offsets_have_end;
  int32_t in_line;         // bytes per fused row
  int32_t data_bytes;      // quantized bytes per row (before scale/offset)
  int32_t out_cols;
  int32_t out16, w16, idx64;
  // rowwise (not fused) tables: scale and offset of row r are sep_scales[r],
  // sep_offsets[r] (fp32) and rows hold data bytes only
  const float *sep_scales, *sep_offsets;
  // multi-table launches: blockIdx.y selects the table whose pointers replace
  // the ones above
  const mi355x_sls_table *tables;
  // output transform: 0 = fp32 / fp16 rows as above; 1 = round to fp16 when
  // out16 (what the operator stores), then Quantize to int8 with (q_scale,
  // q_offset), rows q_stride bytes apart (ConvertTo + Quantize + InsertTensor
  // behind the lookup)
  int32_t out_q8;
  float q_scale, q_offset;
  int64_t q_stride;
};

__device__ __forceinline__ void select_table(SlwsArgs &a) {
  if (a.tables) {
    const mi355x_sls_table t = a.tables[blockIdx.y];
    a.data = t.data;
    a.indices = t.indices;
    a.lengths = t.lengths;
    a.offsets = t.bag_offsets;
    a.offsets_have_end = 1;
    a.dest = t.dest;
    a.data_rows = (int64_t)t.data_rows;
    a.num_indices = (int64_t)t.num_indices;
  }
}

// Stores the columns [col0, col0 + N) of output row `bag`.
template <int N>
__device__ __forceinline__ void store_columns(const SlwsArgs &a, long long bag, int col0,
                                              const float (&acc)[N]) {
  if (a.out_q8) {
    int8_t *d = reinterpret_cast<int8_t *>(a.dest) + bag * a.q_stride + col0;
#pragma unroll
    for (int c = 0; c < N; c++) {
      if (col0 + c < a.out_cols) {
        const float v = a.out16 ? __half2float(__float2half_rn(acc[c])) : acc[c];
        // the Quantize kernel's expression (the conversion saturates)
        const float r = rintf(__fadd_rn(__fdiv_rn(v, a.q_scale), a.q_offset));
        d[c] = (int8_t)min(max((int32_t)r, -128), 127);
      }
    }
    return;
  }
  const long long o0 = bag * (long long)a.out_cols + col0;
  if (a.out16) {
    __half *d = reinterpret_cast<__half *>(a.dest) + o0;
#pragma unroll
    for (int c = 0; c < N; c++)
      if (col0 + c < a.out_cols) d[c] = __float2half_rn(acc[c]);
  } else {
    float *d = reinterpret_cast<float *>(a.dest) + o0;
    if (N == 2 && col0 + 1 < a.out_cols && ((((uintptr_t)d) & 7) == 0)) {
      *reinterpret_cast<float2 *>(d) = make_float2(acc[0], acc[N - 1]);
    } else {
#pragma unroll
      for (int c = 0; c < N; c++)
        if (col0 + c < a.out_cols) d[c] = acc[c];
    }
  }
}

typedef uint8_t __attribute__((address_space(1))) global_u8;
typedef unsigned short __attribute__((address_space(1))) global_u16;

template <int LPB> __device__ __forceinline__ int bcast_i(int v, int j) {
  if constexpr (LPB == 64) {
    return __builtin_amdgcn_readlane(v, j);
  } else {
    return __shfl(v, j, LPB);
  }
}
template <int LPB> __device__ __forceinline__ float bcast_f(float v, int j) {
  return __int_as_float(bcast_i<LPB>(__float_as_int(v), j));
}

__device__ __forceinline__ uint32_t load_u32_any(const uint8_t *p) {
  if ((((uintptr_t)p) & 3) == 0) return *reinterpret_cast<const uint32_t *>(p);
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) |
         ((uint32_t)p[3] << 24);
}

__device__ __forceinline__ float f16round(float v) {
  return __half2float(__float2half_rn(v));
}

// acc += w * (scale * q + offset), each operation rounded on its own; with
// fp16 accumulation the product and the sum are rounded to binary16 the way
// glow::float16's operator+= does (reference include/glow/Support/Float16.h).
template <bool ACC16>
__device__ __forceinline__ float accumulate(float acc, float w, float s,
                                            float o, uint32_t q) {
  float d = __fadd_rn(__fmul_rn(s, (float)q), o);
  float t = __fmul_rn(d, w);
  if constexpr (ACC16) {
    // The product must be rounded to binary32 before it is rounded to
    // binary16, as on the CPU. Left to itself the compiler merges multiply and
    // conversion into one mixed-precision operation that rounds once, which
    // differs in the last place now and then; the empty statement keeps the
    // binary32 product as a value of its own.
    asm volatile("" : "+v"(t));
    return f16round(__fadd_rn(acc, f16round(t)));
  } else {
    return __fadd_rn(acc, t);
  }
}

// Sum of v over the 64 lanes of the wave, returned wave-uniform. Lanes are
// combined inside each row of 16 with DPP moves (no LDS round trip), the four
// row totals are read out as scalars.
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
  int x = (int)v;
  x += __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  x += __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  x += __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, true); // row_half_mirror
  x += __builtin_amdgcn_update_dpp(0, x, 0x140, 0xf, 0xf, true); // row_mirror
  return (uint32_t)__builtin_amdgcn_readlane(x, 0) +
         (uint32_t)__builtin_amdgcn_readlane(x, 16) +
         (uint32_t)__builtin_amdgcn_readlane(x, 32) +
         (uint32_t)__builtin_amdgcn_readlane(x, 48);
}

__device__ __forceinline__ uint32_t clamp_len(int v) {
  return v > 0 ? (uint32_t)v : 0u;
}

// Position of the first lookup of `bag` in the index list and its length.
// Lengths mode: exclusive prefix sum of the clamped lengths in front of the
// block (summed by the block itself, all loads in one memory round trip) plus
// the lengths of the block's earlier bags. Sums inside a chunk are 32-bit:
// positions are checked against num_indices before any use, so absurd lengths
// cannot cause an out-of-range read. Offsets mode: read off the offsets vector.
// Offsets mode: span of `bag` read off the offsets vector.
__device__ __forceinline__ void bag_span_offsets(const SlwsArgs &a,
                                                 long long bag,
                                                 long long &start, int &len) {
  start = 0;
  len = 0;
  if (bag < a.segments) {
    // both ends are clamped into the index list, so that offsets that make no
    // sense (negative, decreasing, past the end) give short or empty bags and
    // never a position outside the list
    start = min(max((long long)a.offsets[bag], 0LL), (long long)a.num_indices);
    long long end = (!a.offsets_have_end && bag == a.segments - 1)
                        ? a.num_indices
                        : (long long)a.offsets[bag + 1];
    end = min(max(end, start), (long long)a.num_indices);
    len = (int)min(end - start, 0x7fffffffLL);
  }
}

// Lengths mode, first half: every wave leaves the sum of the clamped lengths
// it has seen in front of the block in s_part[wave], and the block's own
// clamped lengths go to s_own[]. Ends with a block barrier.
template <int kGroups, int kThreads = kSlwsThreads>
__device__ __forceinline__ void block_prefix(const SlwsArgs &a, int tid,
                                             long long first_bag,
                                             long long *s_part, int *s_own) {
  const long long chunk = first_bag / kChunkBags;
  const long long lo = chunk * kChunkBags;
  const int32_t *lbase = a.lengths + lo;
  const int n_before = (int)(first_bag - lo); // < kChunkBags, multiple of 4
  uint32_t part = 0;
  if ((((uintptr_t)lbase) & 15) == 0) {
    constexpr int kVecTrips = (kChunkBags / 4 + kThreads - 1) / kThreads;
    const int4 *l4 = reinterpret_cast<const int4 *>(lbase);
    const int nvec = n_before / 4;
    if (nvec > 0) {
      // every trip loads (indices past the end re-read the last vector and
      // are masked out), so all loads are in flight together
      int4 x[kVecTrips];
#pragma unroll
      for (int u = 0; u < kVecTrips; u++)
        x[u] = l4[min(tid + u * kThreads, nvec - 1)];
#pragma unroll
      for (int u = 0; u < kVecTrips; u++) {
        const uint32_t t = clamp_len(x[u].x) + clamp_len(x[u].y) +
                           clamp_len(x[u].z) + clamp_len(x[u].w);
        part += (tid + u * kThreads < nvec) ? t : 0u;
      }
    }
  } else {
    for (int i = tid; i < n_before; i += kThreads) part += clamp_len(lbase[i]);
  }
  long long below = 0;
  if (a.chunk_sums) {
    for (long long c = tid; c < chunk; c += kThreads) below += a.chunk_sums[c];
    below = (long long)wave_sum_u32((uint32_t)below) +
            ((long long)wave_sum_u32((uint32_t)(below >> 32)) << 32);
  }
  if (tid < kGroups) {
    const long long b = first_bag + tid;
    s_own[tid] = (int)min(clamp_len(b < a.segments ? a.lengths[b] : 0),
                          0x7fffffffu);
  }
  below += wave_sum_u32(part);
  if ((tid & 63) == 0) s_part[tid >> 6] = below;
  __syncthreads();
}

// Position of the first lookup of `bag` in the index list and its length.
// Lengths mode: exclusive prefix sum of the clamped lengths in front of the
// block (summed by the block itself, all loads in one memory round trip) plus
// the lengths of the block's earlier bags. Sums inside a chunk are 32-bit:
// positions are checked against num_indices before any use, so absurd lengths
// cannot cause an out-of-range read.
template <int kGroups>
__device__ __forceinline__ void bag_span(const SlwsArgs &a, int tid, int grp,
                                         long long bag, long long first_bag,
                                         long long *s_part, int *s_own,
                                         long long &start, int &len) {
  if (a.offsets) {
    bag_span_offsets(a, bag, start, len);
    return;
  }
  block_prefix<kGroups>(a, tid, first_bag, s_part, s_own);
  start = 0;
#pragma unroll
  for (int w = 0; w < kSlwsThreads / 64; w++) start += s_part[w];
  for (int g = 0; g < grp; g++) start += s_own[g];
  len = bag < a.segments ? s_own[grp] : 0;
}

template <int LPB, int BPL, bool IS4, bool SO16, bool ACC16>
__global__ __launch_bounds__(kSlwsThreads) void slws_kernel(SlwsArgs a) {
  select_table(a);
  constexpr int kGroups = kSlwsThreads / LPB;      // bags per block
  constexpr int kColsPerByte = IS4 ? 2 : 1;
  constexpr int kColsPerLane = BPL * kColsPerByte;
  __shared__ long long s_part[kSlwsThreads / 64];
  __shared__ int s_own[kGroups];

  const int tid = threadIdx.x;
  const int sub = tid % LPB;                        // lane within the bag group
  const int grp = tid / LPB;
  const long long first_bag = (long long)blockIdx.x * kGroups;
  const long long bag = first_bag + grp;

  long long start = 0;
  int len = 0;
  bag_span<kGroups>(a, tid, grp, bag, first_bag, s_part, s_own, start, len);
  // a bag cannot use more lookups than the index list holds: bounds the loop
  // below whatever the lengths say
  {
    const long long room = a.num_indices - start;
    len = room <= 0 ? 0 : (int)min((long long)len, room);
  }

  const int n_passes = (a.data_bytes + LPB * BPL - 1) / (LPB * BPL);
  for (int pass = 0; pass < n_passes; pass++) {
    const int byte0 = (pass * LPB + sub) * BPL;       // first data byte of lane
    const bool lane_live = byte0 < a.data_bytes;
    float acc[kColsPerLane];
#pragma unroll
    for (int c = 0; c < kColsPerLane; c++) acc[c] = 0.0f;

    for (int base = 0; base < len; base += kBatch) {
      const int cnt = min(kBatch, len - base);
      // first pass: lookup `sub + k*LPB` of the batch is fetched by lane `sub`
      constexpr int kPerLane = kBatch / LPB;
      int row_lo[kPerLane];
      float wgt[kPerLane], scl[kPerLane], ofs[kPerLane];
#pragma unroll
      for (int k = 0; k < kPerLane; k++) {
        const int j = sub + k * LPB;
        long long pos = start + base + j;
        long long row = -1;
        float w = 0.0f;
        if (j < cnt && pos < a.num_indices) {
          row = a.idx64 ? reinterpret_cast<const long long *>(a.indices)[pos]
                        : (long long)reinterpret_cast<const int *>(a.indices)[pos];
          if (!a.weights) {
            w = 1.0f;
          } else if (a.w16) {
            w = __half2float(reinterpret_cast<const __half *>(a.weights)[pos]);
          } else {
            w = reinterpret_cast<const float *>(a.weights)[pos];
          }
        }
        float s = 0.0f, o = 0.0f;
        if (row >= 0 && row < a.data_rows) {
          const uint8_t *so = a.data + row * a.in_line + a.data_bytes;
          if constexpr (SO16) {
            uint32_t v = load_u32_any(so);
            s = __half2float(__ushort_as_half((unsigned short)(v & 0xffff)));
            o = __half2float(__ushort_as_half((unsigned short)(v >> 16)));
          } else if (a.sep_scales) {
            s = a.sep_scales[row];
            o = a.sep_offsets[row];
          } else {
            s = __uint_as_float(load_u32_any(so));
            o = __uint_as_float(load_u32_any(so + 4));
          }
        } else {
          row = 0; // skipped lookup: reads row 0, contributes w * 0
          w = 0.0f;
        }
        row_lo[k] = (int)row; // data_rows * in_line is checked to fit 2^31 rows
        wgt[k] = w;
        scl[k] = s;
        ofs[k] = o;
      }
      // second pass: all row reads of the batch in flight before the first use
      uint32_t q[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; j++) {
        q[j] = 0;
        if (j < cnt) {
          const int row = bcast_i<LPB>(row_lo[j / LPB], j % LPB);
          if (lane_live) {
            const uint8_t *p = a.data + (long long)row * a.in_line + byte0;
            if constexpr (BPL == 2) {
              q[j] = *reinterpret_cast<const unsigned short *>(p);
            } else {
              q[j] = *p;
            }
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kBatch; j++) {
        if (j < cnt) {
          const float w = bcast_f<LPB>(wgt[j / LPB], j % LPB);
          const float s = bcast_f<LPB>(scl[j / LPB], j % LPB);
          const float o = bcast_f<LPB>(ofs[j / LPB], j % LPB);
#pragma unroll
          for (int b = 0; b < BPL; b++) {
            const uint32_t byte = (q[j] >> (8 * b)) & 0xff;
            if constexpr (IS4) {
              acc[2 * b] = accumulate<ACC16>(acc[2 * b], w, s, o, byte & 15);
              acc[2 * b + 1] = accumulate<ACC16>(acc[2 * b + 1], w, s, o, byte >> 4);
            } else {
              acc[b] = accumulate<ACC16>(acc[b], w, s, o, byte);
            }
          }
        }
      }
    }

    if (bag < a.segments && lane_live)
      store_columns<kColsPerLane>(a, bag, byte0 * kColsPerByte, acc);
  }
}

// Orders this wave's LDS writes before its later LDS reads of other lanes'
// slots. LDS operations of one wave execute in order; the fences keep the
// compiler from moving them across.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Span of the bag of one wavefront (4 waves, 4 consecutive bags per block),
// returned wave-uniform so that it stays in scalar registers. Lengths mode
// ends with a block barrier. A bag cannot use more lookups than the index list
// holds, which bounds the callers' loops whatever the lengths say.
__device__ __forceinline__ void wave_bag_span(const SlwsArgs &a, int tid, int wave,
                                              long long bag, long long first_bag,
                                              long long *s_part, int *s_own,
                                              long long &start, int &len) {
  constexpr int kGroups = 4;
  if (a.offsets) {
    long long start_v;
    int len_v;
    bag_span_offsets(a, bag, start_v, len_v);
    len = __builtin_amdgcn_readfirstlane(len_v);
    start = ((long long)__builtin_amdgcn_readfirstlane((int)(start_v >> 32)) << 32) |
            (unsigned int)__builtin_amdgcn_readfirstlane((int)start_v);
  } else {
    block_prefix<kGroups>(a, tid, first_bag, s_part, s_own);
    const long long block_start = s_part[0] + s_part[1] + s_part[2] + s_part[3];
    const int4 own = *reinterpret_cast<const int4 *>(s_own);
    const int w = __builtin_amdgcn_readfirstlane(wave);
    const int o0 = __builtin_amdgcn_readfirstlane(own.x);
    const int o1 = __builtin_amdgcn_readfirstlane(own.y);
    const int o2 = __builtin_amdgcn_readfirstlane(own.z);
    const int o3 = __builtin_amdgcn_readfirstlane(own.w);
    const long long bs =
        ((long long)__builtin_amdgcn_readfirstlane((int)(block_start >> 32)) << 32) |
        (unsigned int)__builtin_amdgcn_readfirstlane((int)block_start);
    start = bs + (w > 0 ? o0 : 0) + (w > 1 ? o1 : 0) + (w > 2 ? o2 : 0);
    len = w == 0 ? o0 : (w == 1 ? o1 : (w == 2 ? o2 : o3));
    if (bag >= a.segments) len = 0;
  }
  const long long room = a.num_indices - start;
  len = room <= 0 ? 0 : (int)min((long long)len, room);
}

// One bag per wavefront. OFF32: every row's byte offset fits 32 bits, so row
// addresses are formed as a uniform base plus a 32-bit per-lane offset.
template <int BPL, bool IS4, bool SO16, bool ACC16, bool OFF32>
__global__ __launch_bounds__(kSlwsThreads) void slws_wave_kernel(SlwsArgs a) {
  select_table(a);
  constexpr int kGroups = kSlwsThreads / 64;
  constexpr int kColsPerByte = IS4 ? 2 : 1;
  constexpr int kColsPerLane = BPL * kColsPerByte;
  constexpr int kGroup = 4;   // lookups handled under one uniform branch
  __shared__ long long s_part[kGroups];
  __shared__ __attribute__((aligned(16))) int s_own[kGroups];
  // per wave, per lookup of the batch: {row offset or row, weight, scale, offset}
  __shared__ int4 s_look[kGroups][kBatch];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const long long first_bag = (long long)blockIdx.x * kGroups;
  const long long bag = first_bag + wave;

  long long start;
  int len;
  wave_bag_span(a, tid, wave, bag, first_bag, s_part, s_own, start, len);
  int4 *look = s_look[wave];

  const int n_passes = (a.data_bytes + 64 * BPL - 1) / (64 * BPL);
  for (int pass = 0; pass < n_passes; pass++) {
    const int byte0 = (pass * 64 + lane) * BPL;
    const bool lane_live = byte0 < a.data_bytes;
    // lanes past the end of the row read its first bytes and store nothing
    const uint32_t lane_off = lane_live ? (uint32_t)byte0 : 0u;
    float acc[kColsPerLane];
#pragma unroll
    for (int c = 0; c < kColsPerLane; c++) acc[c] = 0.0f;

    for (int base = 0; base < len; base += kBatch) {
      const int cnt = min(kBatch, len - base);
      // first pass: lane j fetches lookup j of the batch
      int my_key;
      uint32_t so_lo = 0, so_hi = 0;
      float my_w;
      bool my_valid;
      {
        const long long pos = start + base + lane;
        long long row = -1;
        float w = 0.0f;
        if (lane < cnt && pos < a.num_indices) {
          row = a.idx64 ? reinterpret_cast<const long long *>(a.indices)[pos]
                        : (long long)reinterpret_cast<const int *>(a.indices)[pos];
          if (!a.weights) {
            w = 1.0f;
          } else if (a.w16) {
            w = __half2float(reinterpret_cast<const __half *>(a.weights)[pos]);
          } else {
            w = reinterpret_cast<const float *>(a.weights)[pos];
          }
        }
        // a skipped lookup reads row 0 and contributes w * 0
        my_valid = row >= 0 && row < a.data_rows;
        if (!my_valid) {
          row = 0;
          w = 0.0f;
        }
        my_w = w;
        my_key = OFF32 ? (int)(uint32_t)(row * a.in_line) : (int)row;
        // The row's scale and offset are requested here and consumed only
        // after the row reads below have been issued, so that the two
        // dependent round trips (index -> scale/offset, index -> row bytes)
        // overlap instead of following each other.
        if (!SO16 && a.sep_scales) {
          so_lo = __float_as_uint(a.sep_scales[row]);
          so_hi = __float_as_uint(a.sep_offsets[row]);
        } else {
          const uint8_t *so = a.data + row * a.in_line + a.data_bytes;
          so_lo = load_u32_any(so);
          if constexpr (!SO16) so_hi = load_u32_any(so + 4);
        }
      }
      // second pass: all row reads of the batch in flight before the first use.
      // Lookups are taken four at a time under one uniform branch; slots
      // beyond cnt hold {row 0, w 0, scale 0, offset 0} and add exactly +0.
      uint32_t q[kBatch];
#pragma unroll
      for (int g = 0; g < kBatch / kGroup; g++) {
        if (g * kGroup < cnt) {
          // An opaque copy of the 32-bit lane offset keeps its widening next
          // to the loads, which lets them use the scalar-base + 32-bit
          // vector-offset addressing form (global address space).
          uint32_t off = lane_off;
          asm volatile("" : "+v"(off));
#pragma unroll
          for (int u = 0; u < kGroup; u++) {
            const int j = g * kGroup + u;
            const int key = __builtin_amdgcn_readlane(my_key, j);
            // uniform row base (kept in scalar registers) + per-lane offset
            const uint8_t *rowp;
            if constexpr (OFF32) {
              rowp = a.data + (uint32_t)key;
            } else {
              rowp = a.data + (long long)key * a.in_line;
            }
            asm volatile("" : "+s"(rowp));
            const global_u8 *p = (const global_u8 *)rowp + off;
            if constexpr (BPL == 2) {
              q[j] = *(const global_u16 *)p;
            } else {
              q[j] = *p;
            }
          }
        }
      }
      {
        float s, o;
        if constexpr (SO16) {
          s = __half2float(__ushort_as_half((unsigned short)(so_lo & 0xffff)));
          o = __half2float(__ushort_as_half((unsigned short)(so_lo >> 16)));
        } else {
          s = __uint_as_float(so_lo);
          o = __uint_as_float(so_hi);
        }
        if (!my_valid) s = o = 0.0f;
        look[lane] = make_int4(my_key, __float_as_int(my_w), __float_as_int(s),
                               __float_as_int(o));
      }
      wave_lds_sync();
#pragma unroll
      for (int g = 0; g < kBatch / kGroup; g++) {
        if (g * kGroup < cnt) {
          int4 r[kGroup];
#pragma unroll
          for (int u = 0; u < kGroup; u++) r[u] = look[g * kGroup + u];
#pragma unroll
          for (int u = 0; u < kGroup; u++) {
            const int j = g * kGroup + u;
            const float w = __int_as_float(r[u].y), s = __int_as_float(r[u].z),
                        o = __int_as_float(r[u].w);
#pragma unroll
            for (int b = 0; b < BPL; b++) {
              const uint32_t byte = (q[j] >> (8 * b)) & 0xff;
              if constexpr (IS4) {
                acc[2 * b] = accumulate<ACC16>(acc[2 * b], w, s, o, byte & 15);
                acc[2 * b + 1] = accumulate<ACC16>(acc[2 * b + 1], w, s, o, byte >> 4);
              } else {
                acc[b] = accumulate<ACC16>(acc[b], w, s, o, byte);
              }
            }
          }
        }
      }
      wave_lds_sync(); // slots are rewritten by the next batch
    }

    if (bag < a.segments && lane_live)
      store_columns<kColsPerLane>(a, bag, byte0 * kColsPerByte, acc);
  }
}


// ---- fused-arithmetic variants ---------------------------------------------------
//
// Same operator with fused multiply-adds, for rows of 32, 64, 128 or 256 data
// bytes with fp32 accumulation.
//
// kMathElement (the default):
//   v = fma(s_j, q_jk, o_j);  dest[k] = fma(w_j, v, dest[k])
// the CPU loop's own expression w*(s*q+o) per element, with the two roundings
// of its products left out: three vector instructions per element (convert,
// fma, fma) instead of five. Each term differs from the CPU loop's by at most
// half a unit in the last place of s*q and of w*v, and nothing is regrouped,
// so a sum that cancels cancels here exactly where it does on the CPU.
//
// kMathRegrouped (on request only):
//   dest[k] = sum_j (w_j*s_j) * q_jk  +  sum_j (w_j*o_j)
// two instructions per element, but the two partial sums are large and of
// opposite sign for tables with a negative offset, so the error is relative to
// the magnitude a bag adds up and not to the result.
//
// One bag per wavefront; a lane reads 4 consecutive data bytes, so a row takes
// LPR = data_bytes/4 lanes and one load instruction fetches 64/LPR rows. The
// partial sums of the row groups are added across lanes at the end of the bag.
constexpr int kMathStrict = MI355X_SLWS_MATH_STRICT, kMathElement = MI355X_SLWS_MATH_ELEMENT,
              kMathRegrouped = MI355X_SLWS_MATH_REGROUPED;

// Cut points of the measurement entry point mi355x_frwq_slws_probe: the kernel
// stops after the named stage and stores a value that depends on what it read.
constexpr int kProbeOff = 0, kProbeSpan = 1, kProbeIndex = 2, kProbeScaleOffset = 3,
              kProbeRows = 4;

template <int MATH>
__device__ __forceinline__ float fused_term(const float4 &f, float q, float acc) {
  if constexpr (MATH == kMathElement) {
    return __fmaf_rn(f.x, __fmaf_rn(f.y, q, f.z), acc);   // f = {w, s, o}
  } else {
    return __fmaf_rn(f.x, q, acc);                        // f = {w*s, w*o}
  }
}

typedef uint32_t __attribute__((address_space(1))) global_u32;
typedef int32_t __attribute__((address_space(1))) global_i32;
typedef long long __attribute__((address_space(1))) global_i64;

// Sum of v over each row of 16 lanes, left in all 16 lanes of the row.
__device__ __forceinline__ uint32_t row16_sum_u32(uint32_t v) {
  int x = (int)v;
  x += __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  x += __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  x += __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, true); // row_half_mirror
  x += __builtin_amdgcn_update_dpp(0, x, 0x140, 0xf, 0xf, true); // row_mirror
  return (uint32_t)x;
}

typedef int __attribute__((ext_vector_type(4))) i32x4;
typedef i32x4 __attribute__((address_space(1))) global_i32x4;

// Span of the bag of wavefront `wave` of a block of WAVES wavefronts (WAVES
// consecutive bags per block), wave-uniform. Lengths mode: the block sums the
// clamped lengths in front of it (from the start of its chunk of kChunkBags
// bags, one 16-byte load per thread and trip, trips beyond the block's position
// skipped), one barrier, then lane g of every wave takes wave g's partial sum
// and bag g's length and a 16-lane sum gives the wave its start. The whole of
// it is about fifty vector instructions: with four waves on a SIMD every
// instruction a wave issues costs the launch sixteen cycles.
template <int WAVES>
__device__ __forceinline__ void rows_bag_span(const SlwsArgs &a, int tid, int lane, int wave,
                                              long long first_bag, uint32_t *s_part,
                                              long long *s_below, int *s_own,
                                              long long &start, int &len) {
  static_assert(WAVES % 4 == 0 && WAVES <= 16, "4, 8, 12 or 16 waves per block");
  constexpr int T = WAVES * 64;
  const long long bag = first_bag + wave;
  if (a.offsets) {
    long long start_v;
    int len_v;
    bag_span_offsets(a, bag, start_v, len_v);
    len = __builtin_amdgcn_readfirstlane(len_v);
    start = ((long long)__builtin_amdgcn_readfirstlane((int)(start_v >> 32)) << 32) |
            (unsigned int)__builtin_amdgcn_readfirstlane((int)start_v);
  } else {
    const long long chunk = first_bag / kChunkBags;
    const long long lo = chunk * kChunkBags;
    const int32_t *lbase = a.lengths + lo;
    const int n_before = (int)(first_bag - lo);   // < kChunkBags, a multiple of WAVES
    uint32_t part = 0;
    if ((((uintptr_t)lbase) & 15) == 0) {
      constexpr int kTrips = (kChunkBags / 4 + T - 1) / T;
      const global_i32x4 *l4 = (const global_i32x4 *)lbase;
      const int nvec = n_before >> 2;
      i32x4 x[kTrips];
#pragma unroll
      for (int u = 0; u < kTrips; u++)
        if (u * T < nvec) x[u] = l4[min(tid + u * T, nvec - 1)];
#pragma unroll
      for (int u = 0; u < kTrips; u++) {
        if (u * T < nvec) {
          const uint32_t t = clamp_len(x[u].x) + clamp_len(x[u].y) + clamp_len(x[u].z) +
                             clamp_len(x[u].w);
          part += (tid + u * T < nvec) ? t : 0u;
        }
      }
    } else {
      for (int i = tid; i < n_before; i += T) part += clamp_len(lbase[i]);
    }
    if (tid < WAVES) {
      const long long b = first_bag + tid;
      s_own[tid] = (int)min(clamp_len(b < a.segments ? a.lengths[b] : 0), 0x7fffffffu);
    }
    if (a.chunk_sums) {
      long long below = 0;
      for (long long c = tid; c < chunk; c += T) below += a.chunk_sums[c];
      below = (long long)wave_sum_u32((uint32_t)below) +
              ((long long)wave_sum_u32((uint32_t)(below >> 32)) << 32);
      if (lane == 0) s_below[wave] = below;
    }
    part = wave_sum_u32(part);
    if (lane == 0) s_part[wave] = part;
    __syncthreads();
    const uint32_t p = lane < WAVES ? s_part[lane] : 0u;
    const int own = lane < WAVES ? s_own[lane] : 0;
    const uint32_t before = row16_sum_u32(p + (lane < wave ? (uint32_t)own : 0u));
    start = (long long)(uint32_t)__builtin_amdgcn_readlane((int)before, 0);
    if (a.chunk_sums) {
      long long below = 0;
#pragma unroll
      for (int g = 0; g < WAVES; g++) below += s_below[g];
      start += ((long long)__builtin_amdgcn_readfirstlane((int)(below >> 32)) << 32) |
               (unsigned int)__builtin_amdgcn_readfirstlane((int)below);
    }
    len = bag < a.segments ? __builtin_amdgcn_readlane(own, wave) : 0;
  }
  const long long room = a.num_indices - start;
  len = room <= 0 ? 0 : (int)min((long long)len, room);
}

// One bag per wavefront, WAVES bags per block; whole rows of LPR * 4 data bytes.
// The caller guarantees a 4-byte aligned table and row pitch.
template <bool IS4, bool SO16, int LPR, bool OFF32, int MATH, int WAVES,
          int PROBE = kProbeOff>
__global__ __launch_bounds__(WAVES * 64) void slws_rows_kernel(SlwsArgs a) {
  select_table(a);
  constexpr int RPI = 64 / LPR;           // rows per load instruction
  constexpr int kCols = IS4 ? 8 : 4;      // output columns per lane
  constexpr int kLoads = kBatch / RPI;    // load instructions of a full batch
  constexpr int kChunk = kLoads < 4 ? kLoads : 4; // loads under one uniform branch
  constexpr int kDataBytes = LPR * 4;
  __shared__ uint32_t s_part[WAVES];
  __shared__ long long s_below[WAVES];
  __shared__ int s_own[WAVES];
  // per wave, per lookup of the batch: row byte offset (or row) and
  // {w, s, o} (kMathElement) or {w*s, w*o} (kMathRegrouped)
  __shared__ uint32_t s_key[WAVES][kBatch];
  __shared__ float4 s_ws[WAVES][kBatch];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long long first_bag = (long long)blockIdx.x * WAVES;
  const long long bag = first_bag + wave;

  long long start;
  int len;
  rows_bag_span<WAVES>(a, tid, lane, wave, first_bag, s_part, s_below, s_own, start, len);
  uint32_t *keys = s_key[wave];
  float4 *wso = s_ws[wave];

  const int sub = lane / LPR;             // which row of a load this lane reads
  const int lir = lane % LPR;
  const uint32_t lane_off = (uint32_t)lir * 4u;
  float acc[kCols];
  float acc_o = 0.0f;
#pragma unroll
  for (int c = 0; c < kCols; c++) acc[c] = 0.0f;
  if constexpr (PROBE == kProbeSpan) {
    // measurement only: the launch up to the bags' positions
    if (bag < a.segments && lane == 0)
      reinterpret_cast<float *>(a.dest)[bag * a.out_cols] = (float)(start + len);
    return;
  }
  const bool sep = !SO16 && a.sep_scales != nullptr;   // uniform

  for (int base = 0; base < len; base += kBatch) {
    const int cnt = min(kBatch, len - base);
    // first pass: lane j fetches lookup j of the batch. len never reaches past
    // the index list (see rows_bag_span), so lane < cnt is the only check.
    uint32_t so_lo = 0, so_hi = 0;
    float my_w = 0.0f;
    bool my_valid = false;
    {
      const long long at = start + base;   // uniform: scalar base + lane offset
      uint32_t row = 0;
      if (lane < cnt) {
        if (a.idx64) {
          const long long r = ((const global_i64 *)a.indices + at)[lane];
          my_valid = (unsigned long long)r < (unsigned long long)a.data_rows;
          row = (uint32_t)r;
        } else {
          row = (uint32_t)((const global_i32 *)a.indices + at)[lane];
          my_valid = row < (uint32_t)a.data_rows;
        }
        if (!a.weights) {
          my_w = 1.0f;
        } else if (a.w16) {
          my_w = __half2float(
              __ushort_as_half(((const global_u16 *)a.weights + at)[lane]));
        } else {
          my_w = __uint_as_float(((const global_u32 *)a.weights + at)[lane]);
        }
      }
      // a skipped lookup reads row 0 and contributes exactly +0
      if (!my_valid) row = 0;
      // The row's scale and offset are requested here and consumed only after
      // the row reads below have been issued, so that the two round trips that
      // depend on the index (scale/offset, row bytes) overlap.
      // (Loads through global-address pointers: a generic-address load also
      // counts as an LDS operation, and the wait for the keys below would then
      // wait for it.)
      if (sep) {
        so_lo = ((const global_u32 *)a.sep_scales)[row];
        so_hi = ((const global_u32 *)a.sep_offsets)[row];
      } else if constexpr (OFF32) {
        const uint32_t key = row * (uint32_t)a.in_line;
        const global_u32 *so =
            (const global_u32 *)((const global_u8 *)a.data + kDataBytes) ;
        so_lo = *(const global_u32 *)((const global_u8 *)so + key);
        if constexpr (!SO16) so_hi = *(const global_u32 *)((const global_u8 *)so + key + 4u);
      } else {
        const global_u32 *so = (const global_u32 *)((const global_u8 *)a.data +
                                                    ((long long)row * a.in_line + kDataBytes));
        so_lo = so[0];
        if constexpr (!SO16) so_hi = so[1];
      }
      keys[lane] = OFF32 ? row * (uint32_t)a.in_line : row;
      if constexpr (PROBE == kProbeIndex) {
        // measurement only: up to the index and weight of every lookup
        acc_o += my_w + (float)row;
        continue;
      }
    }
    if constexpr (PROBE == kProbeScaleOffset) {
      // measurement only: up to the scale and offset of every lookup
      acc_o += my_valid ? my_w * __uint_as_float(so_lo) + __uint_as_float(so_hi) : 0.0f;
      continue;
    }
    wave_lds_sync();
    // second pass: all row reads of the batch in flight before the first use,
    // kChunk load instructions per chunk, as many chunks as the batch has
    // lookups for. The chunk count is wave-uniform and picks one straight-line
    // body (loads of N chunks, the park of {w, s, o}, arithmetic of N chunks):
    // with the chunks under separate branches the loaded words become values
    // carried around the loop and cost a register copy each per batch. Slots
    // beyond cnt hold {row 0, 0, 0, 0} and add exactly +0.
    auto second_pass = [&](auto nc) {
      constexpr int N = decltype(nc)::value;   // chunks
      uint32_t q[N * kChunk];
#pragma unroll
      for (int g = 0; g < N * kChunk; g++) {
        const uint32_t key = keys[g * RPI + sub];
        if constexpr (OFF32) {
          q[g] = *(const global_u32 *)((const global_u8 *)a.data + (key + lane_off));
        } else {
          q[g] = *reinterpret_cast<const uint32_t *>(
              a.data + (long long)key * a.in_line + lane_off);
        }
      }
      {
        float sc, of;
        if constexpr (SO16) {
          sc = __half2float(__ushort_as_half((unsigned short)(so_lo & 0xffff)));
          of = __half2float(__ushort_as_half((unsigned short)(so_lo >> 16)));
        } else {
          sc = __uint_as_float(so_lo);
          of = __uint_as_float(so_hi);
        }
        if constexpr (MATH == kMathElement)
          wso[lane] = my_valid ? make_float4(my_w, sc, of, 0.0f)
                               : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        else
          wso[lane] = my_valid ? make_float4(my_w * sc, my_w * of, 0.0f, 0.0f)
                               : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
      wave_lds_sync();
#pragma unroll
      for (int g = 0; g < N * kChunk; g++) {
        if constexpr (PROBE == kProbeRows) {
          // measurement only: every row read, no arithmetic
          acc_o = __uint_as_float(__float_as_uint(acc_o) ^ q[g]);
          continue;
        }
        const float4 f = wso[g * RPI + sub];
        if constexpr (MATH == kMathRegrouped) acc_o += f.y;
        if constexpr (IS4) {
          const uint32_t lo = q[g] & 0x0f0f0f0fu, hi = (q[g] >> 4) & 0x0f0f0f0fu;
#pragma unroll
          for (int b = 0; b < 4; b++) {
            acc[2 * b] = fused_term<MATH>(f, (float)((lo >> (8 * b)) & 0xff), acc[2 * b]);
            acc[2 * b + 1] =
                fused_term<MATH>(f, (float)((hi >> (8 * b)) & 0xff), acc[2 * b + 1]);
          }
        } else {
#pragma unroll
          for (int b = 0; b < 4; b++)
            acc[b] = fused_term<MATH>(f, (float)((q[g] >> (8 * b)) & 0xff), acc[b]);
        }
      }
    };
    constexpr int kChunks = kLoads / kChunk;
    static_assert(kChunks <= 16, "one case per chunk count");
    const int chunks = (cnt + kChunk * RPI - 1) / (kChunk * RPI);   // 1..kChunks, uniform
#define MI355X_SECOND_PASS(n)                                                  \
  case n:                                                                      \
    if constexpr (n <= kChunks) second_pass(std::integral_constant<int, (n <= kChunks ? n : 1)>()); \
    break;
    switch (chunks) {
      MI355X_SECOND_PASS(1) MI355X_SECOND_PASS(2) MI355X_SECOND_PASS(3) MI355X_SECOND_PASS(4)
      MI355X_SECOND_PASS(5) MI355X_SECOND_PASS(6) MI355X_SECOND_PASS(7) MI355X_SECOND_PASS(8)
      MI355X_SECOND_PASS(9) MI355X_SECOND_PASS(10) MI355X_SECOND_PASS(11) MI355X_SECOND_PASS(12)
      MI355X_SECOND_PASS(13) MI355X_SECOND_PASS(14) MI355X_SECOND_PASS(15) MI355X_SECOND_PASS(16)
    default:
      break;
    }
#undef MI355X_SECOND_PASS
    wave_lds_sync(); // slots are rewritten by the next batch
  }
  if constexpr (PROBE == kProbeRows) acc_o = (float)(__float_as_uint(acc_o) & 0xffu);

  // partial sums of the RPI row groups -> lanes of group 0
#pragma unroll
  for (int c = 0; c < kCols; c++) {
    float v = MATH == kMathRegrouped || PROBE != kProbeOff ? acc[c] + acc_o : acc[c];
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
    acc[c] = v;
  }
  if (bag < a.segments && sub == 0) {
    float *d = reinterpret_cast<float *>(a.dest) + (bag * (long long)(LPR * kCols) + lir * kCols);
    if (!a.out_q8 && !a.out16 && ((((uintptr_t)a.dest) & 15) == 0)) {
      // dense fp32 rows of exactly LPR * kCols columns: 16-byte stores
#pragma unroll
      for (int c = 0; c < kCols; c += 4)
        *reinterpret_cast<float4 *>(d + c) = make_float4(acc[c], acc[c + 1], acc[c + 2], acc[c + 3]);
    } else {
      store_columns<kCols>(a, bag, lir * kCols, acc);
    }
  }
}

// The same arithmetic for short rows (32 or 64 data bytes): a row takes only
// LPR = 8 or 16 lanes, so a wavefront works on 64/LPR bags side by side, one
// per lane group, and nothing has to be added across lanes at the end. A
// group's lanes fetch its lookups (index, weight, scale, offset) kGB at a
// time and hand them to each other through a wave-private LDS table.
template <bool IS4, bool SO16, int LPR, bool OFF32, int MATH>
__global__ __launch_bounds__(kSlwsThreads) void slws_groups_kernel(SlwsArgs a) {
  select_table(a);
  constexpr int kGroups = kSlwsThreads / LPR; // bags per block
  constexpr int kCols = IS4 ? 8 : 4;          // output columns per lane
  constexpr int kGB = 32;                     // lookups of a bag per round
  constexpr int kPer = kGB / LPR;             // lookups one lane fetches per round
  constexpr int kChunk = 8;                   // row reads under one uniform branch
  __shared__ long long s_part[kSlwsThreads / 64];
  __shared__ int s_own[kGroups];
  __shared__ uint32_t s_key[kGroups][kGB];
  __shared__ float4 s_ws[kGroups][kGB];

  const int tid = threadIdx.x;
  const int grp = tid / LPR, lir = tid % LPR;
  const long long first_bag = (long long)blockIdx.x * kGroups;
  const long long bag = first_bag + grp;

  long long start = 0;
  int len = 0;
  bag_span<kGroups>(a, tid, grp, bag, first_bag, s_part, s_own, start, len);
  {
    const long long room = a.num_indices - start;
    len = room <= 0 ? 0 : (int)min((long long)len, room);
  }
  // the loops below run as long as the longest bag of the wavefront needs
  int wave_len = len;
#pragma unroll
  for (int off = LPR; off < 64; off <<= 1) wave_len = max(wave_len, __shfl_xor(wave_len, off, 64));
  wave_len = __builtin_amdgcn_readfirstlane(wave_len);

  uint32_t *keys = s_key[grp];
  float4 *wso = s_ws[grp];
  const uint32_t lane_off = (uint32_t)lir * 4u;
  float acc[kCols];
  float acc_o = 0.0f;
#pragma unroll
  for (int c = 0; c < kCols; c++) acc[c] = 0.0f;

  for (int base = 0; base < wave_len; base += kGB) {
    const int cnt = min(kGB, len - base);           // this bag's share (may be <= 0)
    const int wave_cnt = min(kGB, wave_len - base); // uniform
    // scale and offset are requested with the index in hand and consumed after
    // the row reads have been issued (global-address loads: see slws_rows_kernel)
    uint32_t so_lo[kPer], so_hi[kPer];
    float my_w[kPer];
    bool my_valid[kPer];
#pragma unroll
    for (int k = 0; k < kPer; k++) {
      const int j = lir + k * LPR;
      const long long pos = start + base + j;
      long long row = -1;
      float w = 0.0f;
      if (j < cnt && pos < a.num_indices) {
        row = a.idx64 ? ((const global_i64 *)a.indices)[pos]
                      : (long long)((const global_i32 *)a.indices)[pos];
        if (!a.weights) {
          w = 1.0f;
        } else if (a.w16) {
          w = __half2float(reinterpret_cast<const __half *>(a.weights)[pos]);
        } else {
          w = reinterpret_cast<const float *>(a.weights)[pos];
        }
      }
      // a skipped lookup reads row 0 and contributes exactly +0
      my_valid[k] = row >= 0 && row < a.data_rows;
      if (!my_valid[k]) row = 0;
      my_w[k] = w;
      so_hi[k] = 0;
      if (!SO16 && a.sep_scales) {
        so_lo[k] = ((const global_u32 *)a.sep_scales)[row];
        so_hi[k] = ((const global_u32 *)a.sep_offsets)[row];
      } else {
        const global_u32 *so = (const global_u32 *)((const global_u8 *)a.data +
                                                    (row * a.in_line + a.data_bytes));
        so_lo[k] = so[0];
        if constexpr (!SO16) so_hi[k] = so[1];
      }
      keys[j] = OFF32 ? (uint32_t)(row * a.in_line) : (uint32_t)row;
    }
    wave_lds_sync();
    uint32_t q[kGB];
#pragma unroll
    for (int c = 0; c < kGB / kChunk; c++) {
      if (c * kChunk < wave_cnt) {
#pragma unroll
        for (int u = 0; u < kChunk; u++) {
          const int j = c * kChunk + u;
          const uint32_t key = keys[j];
          if constexpr (OFF32) {
            q[j] = *(const global_u32 *)((const global_u8 *)a.data + (key + lane_off));
          } else {
            q[j] = *reinterpret_cast<const uint32_t *>(
                a.data + (long long)key * a.in_line + lane_off);
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kPer; k++) {
      float sc, of;
      if constexpr (SO16) {
        sc = __half2float(__ushort_as_half((unsigned short)(so_lo[k] & 0xffff)));
        of = __half2float(__ushort_as_half((unsigned short)(so_lo[k] >> 16)));
      } else {
        sc = __uint_as_float(so_lo[k]);
        of = __uint_as_float(so_hi[k]);
      }
      if constexpr (MATH == kMathElement)
        wso[lir + k * LPR] = my_valid[k] ? make_float4(my_w[k], sc, of, 0.0f)
                                         : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      else
        wso[lir + k * LPR] = my_valid[k] ? make_float4(my_w[k] * sc, my_w[k] * of, 0.0f, 0.0f)
                                         : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    wave_lds_sync();
#pragma unroll
    for (int c = 0; c < kGB / kChunk; c++) {
      if (c * kChunk < wave_cnt) {
#pragma unroll
        for (int u = 0; u < kChunk; u++) {
          const int j = c * kChunk + u;
          const float4 f = wso[j];
          if constexpr (MATH == kMathRegrouped) acc_o += f.y;
          if constexpr (IS4) {
            const uint32_t lo = q[j] & 0x0f0f0f0fu, hi = (q[j] >> 4) & 0x0f0f0f0fu;
#pragma unroll
            for (int b = 0; b < 4; b++) {
              acc[2 * b] = fused_term<MATH>(f, (float)((lo >> (8 * b)) & 0xff), acc[2 * b]);
              acc[2 * b + 1] =
                  fused_term<MATH>(f, (float)((hi >> (8 * b)) & 0xff), acc[2 * b + 1]);
            }
          } else {
#pragma unroll
            for (int b = 0; b < 4; b++)
              acc[b] = fused_term<MATH>(f, (float)((q[j] >> (8 * b)) & 0xff), acc[b]);
          }
        }
      }
    }
    wave_lds_sync(); // slots are rewritten by the next round
  }
#pragma unroll
  for (int c = 0; c < kCols; c++) acc[c] += acc_o;
  if (bag < a.segments) store_columns<kCols>(a, bag, lir * kCols, acc);
}

// A launch that does nothing (measurement: what any launch of this shape costs).
__global__ __launch_bounds__(kRowsWaves * 64) void slws_empty_kernel(float *dest) {
  if (dest == nullptr && threadIdx.x == 12345) dest[0] = 0.0f; // never taken
}

// Sum of the clamped lengths of each chunk of kChunkBags bags.
__global__ __launch_bounds__(256) void slws_chunk_sums_kernel(
    const int32_t *lengths, long long segments, int64_t *chunk_sums) {
  __shared__ long long s_part[4];
  const long long lo = (long long)blockIdx.x * kChunkBags;
  const long long hi = min(lo + (long long)kChunkBags, segments);
  long long sum = 0;
  for (long long i = lo + threadIdx.x; i < hi; i += 256) {
    int v = lengths[i];
    sum += v > 0 ? v : 0;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0)
    chunk_sums[blockIdx.x] = s_part[0] + s_part[1] + s_part[2] + s_part[3];
}

// Scratch for the chunk sums (lengths mode with more than kChunkBags bags):
// one int64 per chunk, written by slws_chunk_sums_kernel and read by the
// lookup kernel behind it on the same stream.
//
// The ordinary entry points take it from a registry keyed by (device, stream):
// launches on one stream are ordered, so they may share a buffer; launches on
// different streams never do. A buffer is allocated when the stream is made
// known to the library (mi355x_init for the device's default stream,
// mi355x_stream_create, mi355x_slws_reserve_stream), never inside a launch.
struct StreamScratch {
  int dev;
  hipStream_t stream;
  int64_t *ws;
};
static std::mutex g_ws_mutex;
static std::vector<StreamScratch> g_ws;

int slws_reserve_stream(hipStream_t st) {
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  for (const StreamScratch &e : g_ws)
    if (e.dev == dev && e.stream == st) return MI355X_OK;
  int64_t *ws = nullptr;
  MI355X_HIP(hipMalloc((void **)&ws, kMaxChunks * sizeof(int64_t)));
  g_ws.push_back(StreamScratch{dev, st, ws});
  return MI355X_OK;
}

int slws_release_stream(hipStream_t st) {
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  int64_t *ws = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (size_t i = 0; i < g_ws.size(); i++)
      if (g_ws[i].dev == dev && g_ws[i].stream == st) {
        ws = g_ws[i].ws;
        g_ws.erase(g_ws.begin() + (long)i);
        break;
      }
  }
  if (ws) MI355X_HIP(hipFree(ws));
  return MI355X_OK;
}

static int stream_scratch(hipStream_t st, int64_t **ws) {
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  for (const StreamScratch &e : g_ws)
    if (e.dev == dev && e.stream == st) {
      *ws = e.ws;
      return MI355X_OK;
    }
  return fail(MI355X_ERR_INVALID_ARGUMENT,
              "more than %d bags on a stream without scratch for the bag offsets: "
              "use a stream from mi355x_stream_create (or the default stream after "
              "mi355x_init), or call mi355x_slws_reserve_stream(stream) once before",
              kChunkBags);
}

// The same scratch for callers that must not allocate: a fixed array in the
// code object, one copy per device, found once per device with
// hipGetSymbolAddress. Host code never uses the array's name as an address.
constexpr int kStaticChunks = 4096;   // 32 KiB; 4096 * 4096 = 16.7M bags
static __device__ __align__(256) int64_t scratch[kStaticChunks];
static std::mutex g_static_mutex;
static int64_t *g_static_ptr[64] = {nullptr};

int slws_init_device() {
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  MI355X_REQUIRE(dev >= 0 && dev < 64, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[dev]) {
    int64_t *ptr = nullptr;
    MI355X_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
    MI355X_REQUIRE(ptr, "hipGetSymbolAddress returned a NULL address");
    g_static_ptr[dev] = ptr;
  }
  return MI355X_OK;
}

static int static_scratch(int64_t **ws) {
  int dev = 0;
  MI355X_HIP(hipGetDevice(&dev));
  MI355X_REQUIRE(dev >= 0 && dev < 64, "device index %d out of range", dev);
  {
    std::lock_guard<std::mutex> lock(g_static_mutex);
    *ws = g_static_ptr[dev];
  }
  if (*ws) return MI355X_OK;
  int rc = slws_init_device();   // first call on this device
  if (rc != MI355X_OK) return rc;
  std::lock_guard<std::mutex> lock(g_static_mutex);
  *ws = g_static_ptr[dev];
  return MI355X_OK;
}

template <int LPB, int BPL>
static void launch_kind(int kind, bool acc16, dim3 grid, hipStream_t st,
                        const SlwsArgs &a) {
#define MI355X_SLWS_LAUNCH(IS4, SO16, ACC16)                                   \
  hipLaunchKernelGGL((slws_kernel<LPB, BPL, IS4, SO16, ACC16>), grid,          \
                     dim3(kSlwsThreads), 0, st, a)
  switch (kind) {
  case MI355X_FUSED_U8_F32:
    MI355X_SLWS_LAUNCH(false, false, false);
    break;
  case MI355X_FUSED_U8_F16:
    if (acc16) MI355X_SLWS_LAUNCH(false, true, true);
    else MI355X_SLWS_LAUNCH(false, true, false);
    break;
  case MI355X_FUSED_U4_F16:
    if (acc16) MI355X_SLWS_LAUNCH(true, true, true);
    else MI355X_SLWS_LAUNCH(true, true, false);
    break;
  default:
    MI355X_SLWS_LAUNCH(true, false, false);
    break;
  }
#undef MI355X_SLWS_LAUNCH
}

template <int BPL, bool OFF32>
static void launch_wave_kind(int kind, bool acc16, dim3 grid, hipStream_t st,
                             const SlwsArgs &a) {
#define MI355X_SLWS_WAVE(IS4, SO16, ACC16)                                     \
  hipLaunchKernelGGL((slws_wave_kernel<BPL, IS4, SO16, ACC16, OFF32>), grid,   \
                     dim3(kSlwsThreads), 0, st, a)
  switch (kind) {
  case MI355X_FUSED_U8_F32:
    MI355X_SLWS_WAVE(false, false, false);
    break;
  case MI355X_FUSED_U8_F16:
    if (acc16) MI355X_SLWS_WAVE(false, true, true);
    else MI355X_SLWS_WAVE(false, true, false);
    break;
  case MI355X_FUSED_U4_F16:
    if (acc16) MI355X_SLWS_WAVE(true, true, true);
    else MI355X_SLWS_WAVE(true, true, false);
    break;
  default:
    MI355X_SLWS_WAVE(true, false, false);
    break;
  }
#undef MI355X_SLWS_WAVE
}

template <int LPR, bool OFF32, int MATH, int WAVES>
static void launch_rows_kind(int kind, dim3 grid, hipStream_t st, const SlwsArgs &a) {
#define MI355X_SLWS_ROWS(IS4, SO16)                                            \
  hipLaunchKernelGGL((slws_rows_kernel<IS4, SO16, LPR, OFF32, MATH, WAVES>), grid, \
                     dim3(WAVES * 64), 0, st, a)
  switch (kind) {
  case MI355X_FUSED_U8_F32:
    MI355X_SLWS_ROWS(false, false);
    break;
  case MI355X_FUSED_U8_F16:
    MI355X_SLWS_ROWS(false, true);
    break;
  case MI355X_FUSED_U4_F16:
    MI355X_SLWS_ROWS(true, true);
    break;
  default:
    MI355X_SLWS_ROWS(true, false);
    break;
  }
#undef MI355X_SLWS_ROWS
}

template <int LPR, bool OFF32, int MATH>
static void launch_groups_kind(int kind, dim3 grid, hipStream_t st, const SlwsArgs &a) {
#define MI355X_SLWS_GROUPS(IS4, SO16)                                          \
  hipLaunchKernelGGL((slws_groups_kernel<IS4, SO16, LPR, OFF32, MATH>), grid,  \
                     dim3(kSlwsThreads), 0, st, a)
  switch (kind) {
  case MI355X_FUSED_U8_F32:
    MI355X_SLWS_GROUPS(false, false);
    break;
  case MI355X_FUSED_U8_F16:
    MI355X_SLWS_GROUPS(false, true);
    break;
  case MI355X_FUSED_U4_F16:
    MI355X_SLWS_GROUPS(true, true);
    break;
  default:
    MI355X_SLWS_GROUPS(true, false);
    break;
  }
#undef MI355X_SLWS_GROUPS
}

// Arithmetic of the launches that do not name one (process-wide default).
static std::atomic<int> g_fused_math{kMathElement};
// Arithmetic named by the call being issued on this thread (OptsScope); -1: none.
thread_local int g_slws_math = -1;

// Several tables in one launch and/or the int8 output transform.
struct SlwsExtra {
  const float *sep_scales = nullptr, *sep_offsets = nullptr; // rowwise tables
  const mi355x_sls_table *tables = nullptr; // device array
  size_t n_tables = 1;
  int out_q8 = 0;
  float q_scale = 1.0f;
  int32_t q_offset = 0;
  size_t q_stride = 0;
  bool static_scratch = false; // chunk sums in the code object's fixed array
  int math = -1;               // kMath*; -1 = the process-wide default
  int probe = kProbeOff;       // measurement cut point (mi355x_frwq_slws_probe)
};

static int slws_dispatch(void *dest, int out_is_f16, const uint8_t *data,
                         size_t data_rows, int kind, const void *weights,
                         int weights_are_f16, const void *indices,
                         int idx_is_64, size_t num_indices,
                         const int32_t *lengths, const int32_t *offsets,
                         int has_end_offset, size_t out_rows,
                         size_t in_line_size, size_t out_line_size,
                         int fp16_accum, void *stream,
                         const SlwsExtra &x = SlwsExtra()) {
  if (out_rows == 0 || x.n_tables == 0) return MI355X_OK;
  MI355X_REQUIRE(kind >= 0 && kind <= 3, "unknown fused kind %d", kind);
  MI355X_REQUIRE(x.tables || (dest && (lengths || offsets)), "NULL tensor");
  MI355X_REQUIRE(x.n_tables <= 65535, "more than 65535 tables");
  const bool is4 = kind == MI355X_FUSED_U4_F16 || kind == MI355X_FUSED_U4_F32;
  const bool so16 = kind == MI355X_FUSED_U8_F16 || kind == MI355X_FUSED_U4_F16;
  const size_t so_bytes = x.sep_scales ? 0 : (so16 ? 4 : 8);
  // in_line_size is the distance between rows: the fused row's own size, or
  // more when the table has been laid out with padded rows
  MI355X_REQUIRE(out_line_size > 0 && (!is4 || out_line_size % 2 == 0),
                 "out_line_size %zu is not a row of this kind", out_line_size);
  const size_t cols = out_line_size;
  const size_t data_bytes = is4 ? cols / 2 : cols;
  MI355X_REQUIRE(in_line_size >= data_bytes + so_bytes,
                 "in_line_size %zu does not hold %zu columns of the fused row",
                 in_line_size, cols);
  MI355X_REQUIRE(in_line_size < (1u << 20) && data_rows < (1ull << 31) &&
                     out_rows < (1ull << 40),
                 "table or batch too large");
  MI355X_REQUIRE(x.tables || num_indices == 0 || (indices && data),
                 "NULL indices or data with num_indices > 0");
  MI355X_REQUIRE(!x.tables || out_rows <= (size_t)kChunkBags,
                 "a multi-table launch takes at most %d bags per table", kChunkBags);
  MI355X_REQUIRE(!x.out_q8 || x.q_stride >= cols, "output rows overlap");
  hipStream_t st = as_stream(stream);

  SlwsArgs a;
  a.dest = dest;
  a.data = data;
  a.weights = weights;
  a.indices = indices;
  a.lengths = lengths;
  a.offsets = offsets;
  a.chunk_sums = nullptr;
  a.data_rows = (int64_t)data_rows;
  a.num_indices = (int64_t)num_indices;
  a.segments = (int64_t)out_rows;
  a.offsets_have_end = has_end_offset;
  a.in_line = (int32_t)in_line_size;
  a.data_bytes = (int32_t)data_bytes;
  a.out_cols = (int32_t)cols;
  a.out16 = out_is_f16;
  a.w16 = weights_are_f16;
  a.idx64 = idx_is_64;
  a.sep_scales = x.sep_scales;
  a.sep_offsets = x.sep_offsets;
  a.tables = x.tables;
  a.out_q8 = x.out_q8;
  a.q_scale = x.q_scale;
  a.q_offset = (float)x.q_offset;
  a.q_stride = (int64_t)x.q_stride;

  if (!offsets) {
    const size_t chunks = (out_rows + kChunkBags - 1) / kChunkBags;
    if (chunks > 1) {
      int64_t *ws = nullptr;
      int rc;
      if (x.static_scratch) {
        MI355X_REQUIRE(chunks <= (size_t)kStaticChunks,
                       "%zu bags: the entry point that allocates nothing takes at "
                       "most %d", out_rows, kStaticChunks * kChunkBags);
        rc = static_scratch(&ws);
      } else {
        MI355X_REQUIRE(chunks <= (size_t)kMaxChunks, "more than %d bags",
                       kMaxChunks * kChunkBags);
        rc = stream_scratch(st, &ws);
      }
      if (rc != MI355X_OK) return rc;
      hipLaunchKernelGGL(slws_chunk_sums_kernel, dim3((unsigned)chunks),
                         dim3(256), 0, st, lengths, (long long)out_rows, ws);
      rc = check_launch("slws_chunk_sums");
      if (rc != MI355X_OK) return rc;
      a.chunk_sums = ws;
    }
  }

  const bool acc16 = out_is_f16 && fp16_accum && so16;
  const bool even = (in_line_size % 2 == 0) && (((uintptr_t)data) % 2 == 0);
  int lpb = 64;
  if (even && data_bytes <= 32) lpb = 16;
  else if (even && data_bytes <= 64) lpb = 32;
  const size_t groups = kSlwsThreads / lpb;
  const size_t blocks = (out_rows + groups - 1) / groups;
  MI355X_REQUIRE(blocks < 0x7fffffffu, "too many bags");
  dim3 grid((unsigned)blocks, (unsigned)x.n_tables);
  const bool off32 = (unsigned long long)data_rows * in_line_size <= 0xffffffffull;
  // fused arithmetic: whole rows of 32, 64, 128 or 256 data bytes, 4-byte
  // aligned, fp32 accumulation. A multi-table launch cannot check the
  // alignment of each table here; its tables must be 4-byte aligned.
  const int math = x.math >= 0     ? x.math
                   : g_slws_math >= 0 ? g_slws_math
                                      : g_fused_math.load(std::memory_order_relaxed);
  MI355X_REQUIRE(math >= kMathStrict && math <= kMathRegrouped,
                 "unknown SparseLengths arithmetic %d", math);
  const bool rows_ok = math != kMathStrict && !acc16 &&
                       in_line_size % 4 == 0 && (((uintptr_t)data) % 4 == 0) &&
                       (data_bytes == 32 || data_bytes == 64 ||
                        data_bytes == 128 || data_bytes == 256);
  if (x.probe != kProbeOff) {
    MI355X_REQUIRE(rows_ok && kind == MI355X_FUSED_U8_F32 && data_bytes == 128 && off32 &&
                       !x.tables && !x.out_q8 && math == kMathElement,
                   "the probe covers uint8 rows of 128 columns with fp32 scale and offset");
    const size_t pw = (size_t)rows_waves(out_rows);
    const size_t rblocks = (out_rows + pw - 1) / pw;
    MI355X_REQUIRE(rblocks < 0x7fffffffu, "too many bags");
    dim3 rgrid((unsigned)rblocks);
#define MI355X_PROBE_CASE(P)                                                   \
  case P:                                                                      \
    if (pw == (size_t)kRowsWaves)                                              \
      hipLaunchKernelGGL(                                                      \
          (slws_rows_kernel<false, false, 32, true, kMathElement, kRowsWaves, P>), rgrid, \
          dim3(kRowsWaves * 64), 0, st, a);                                    \
    else                                                                       \
      hipLaunchKernelGGL(                                                      \
          (slws_rows_kernel<false, false, 32, true, kMathElement, kRowsWavesMany, P>), rgrid, \
          dim3(kRowsWavesMany * 64), 0, st, a);                                \
    break;
    switch (x.probe) {
      MI355X_PROBE_CASE(kProbeSpan)
      MI355X_PROBE_CASE(kProbeIndex)
      MI355X_PROBE_CASE(kProbeScaleOffset)
      MI355X_PROBE_CASE(kProbeRows)
    default:
      return fail(MI355X_ERR_INVALID_ARGUMENT, "unknown probe stage %d", x.probe);
    }
#undef MI355X_PROBE_CASE
    return check_launch("frwq_slws_probe");
  }
  if (rows_ok && data_bytes <= 64) {
    // short rows: several bags per wavefront
    const size_t per_block = kSlwsThreads / (data_bytes / 4);
    const size_t gblocks = (out_rows + per_block - 1) / per_block;
    MI355X_REQUIRE(gblocks < 0x7fffffffu, "too many bags");
    dim3 ggrid((unsigned)gblocks, (unsigned)x.n_tables);
#define MI355X_GROUPS_CASE(LPR)                                                \
  if (math == kMathElement) {                                                  \
    if (off32) launch_groups_kind<LPR, true, kMathElement>(kind, ggrid, st, a);  \
    else launch_groups_kind<LPR, false, kMathElement>(kind, ggrid, st, a);     \
  } else {                                                                     \
    if (off32) launch_groups_kind<LPR, true, kMathRegrouped>(kind, ggrid, st, a); \
    else launch_groups_kind<LPR, false, kMathRegrouped>(kind, ggrid, st, a);   \
  }
    if (data_bytes == 32) {
      MI355X_GROUPS_CASE(8)
    } else {
      MI355X_GROUPS_CASE(16)
    }
#undef MI355X_GROUPS_CASE
    return check_launch("frwq_slws");
  }
  if (rows_ok) {
    const size_t rw = (size_t)rows_waves(out_rows);
    const size_t rblocks = (out_rows + rw - 1) / rw;
    MI355X_REQUIRE(rblocks < 0x7fffffffu, "too many bags");
    dim3 rgrid((unsigned)rblocks, (unsigned)x.n_tables);
#define MI355X_ROWS_MATH(BYTES, MATH)                                          \
  if (rw == (size_t)kRowsWaves) {                                              \
    if (off32) launch_rows_kind<BYTES / 4, true, MATH, kRowsWaves>(kind, rgrid, st, a); \
    else launch_rows_kind<BYTES / 4, false, MATH, kRowsWaves>(kind, rgrid, st, a); \
  } else {                                                                     \
    if (off32) launch_rows_kind<BYTES / 4, true, MATH, kRowsWavesMany>(kind, rgrid, st, a); \
    else launch_rows_kind<BYTES / 4, false, MATH, kRowsWavesMany>(kind, rgrid, st, a); \
  }
#define MI355X_ROWS_CASE(BYTES)                                                \
  case BYTES:                                                                  \
    if (math == kMathElement) {                                                \
      MI355X_ROWS_MATH(BYTES, kMathElement)                                    \
    } else {                                                                   \
      MI355X_ROWS_MATH(BYTES, kMathRegrouped)                                  \
    }                                                                          \
    break;
    switch (data_bytes) {
      MI355X_ROWS_CASE(32)
      MI355X_ROWS_CASE(64)
      MI355X_ROWS_CASE(128)
      MI355X_ROWS_CASE(256)
    }
#undef MI355X_ROWS_CASE
#undef MI355X_ROWS_MATH
    return check_launch("frwq_slws");
  }
  if (lpb == 16) launch_kind<16, 2>(kind, acc16, grid, st, a);
  else if (lpb == 32) launch_kind<32, 2>(kind, acc16, grid, st, a);
  else if (!even && off32) launch_wave_kind<1, true>(kind, acc16, grid, st, a);
  else if (!even) launch_wave_kind<1, false>(kind, acc16, grid, st, a);
  else if (off32) launch_wave_kind<2, true>(kind, acc16, grid, st, a);
  else launch_wave_kind<2, false>(kind, acc16, grid, st, a);
  return check_launch("frwq_slws");
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

int mi355x_slws_set_fused_math(int on) {  // on: MI355X_SLWS_MATH_*
  MI355X_REQUIRE(on >= kMathStrict && on <= kMathRegrouped,
                 "unknown SparseLengths arithmetic %d", on);
  g_fused_math.store(on, std::memory_order_relaxed);
  return MI355X_OK;
}

int mi355x_frwq_slws_probe(int stage, float *dest, const uint8_t *data, size_t data_rows,
                           const float *weights, const int64_t *indices,
                           size_t num_indices, const int32_t *lengths, size_t segments,
                           size_t in_line_size, void *stream) {
  MI355X_REQUIRE(segments == 0 || lengths, "lengths is NULL");
  if (stage == 0) {
    // a launch of the same shape that does nothing
    if (segments == 0) return MI355X_OK;
    const size_t w = (size_t)rows_waves(segments);
    hipLaunchKernelGGL(slws_empty_kernel, dim3((unsigned)((segments + w - 1) / w)),
                       dim3((unsigned)w * 64), 0, as_stream(stream), dest);
    return check_launch("slws_empty");
  }
  SlwsExtra x;
  x.math = kMathElement;
  x.probe = stage;
  return slws_dispatch(dest, 0, data, data_rows, MI355X_FUSED_U8_F32, weights, 0, indices, 1,
                       num_indices, lengths, nullptr, 0, segments, in_line_size, 128, 0,
                       stream, x);
}

static int mi355x_frwq_sls_multi_impl(const mi355x_sls_table *tables, size_t n_tables,
                          size_t max_data_rows, int kind, int idx_is_64,
                          size_t segments, size_t in_line_size,
                          size_t out_line_size, int out_kind, float out_scale,
                          int32_t out_offset, size_t dest_row_stride,
                          int fp16_accum, void *stream) {
  if (n_tables == 0 || segments == 0) return MI355X_OK;
  MI355X_REQUIRE(tables, "tables is NULL");
  MI355X_REQUIRE(out_kind >= 0 && out_kind <= 3, "unknown output kind %d", out_kind);
  SlwsExtra x;
  x.tables = tables;
  x.n_tables = n_tables;
  x.out_q8 = out_kind >= 2;
  x.q_scale = out_scale;
  x.q_offset = out_offset;
  x.q_stride = dest_row_stride;
  const int out16 = out_kind == MI355X_SLS_OUT_F16 || out_kind == MI355X_SLS_OUT_I8_VIA_F16;
  return slws_dispatch(nullptr, out16, nullptr, max_data_rows, kind, nullptr, 0, nullptr,
                       idx_is_64, 0, nullptr, nullptr, 0, segments, in_line_size,
                       out_line_size, fp16_accum, stream, x);
}

int mi355x_frwq_sls_multi(const mi355x_sls_table *tables, size_t n_tables,
                          size_t max_data_rows, int kind, int idx_is_64,
                          size_t segments, size_t in_line_size,
                          size_t out_line_size, int out_kind, float out_scale,
                          int32_t out_offset, size_t dest_row_stride,
                          int fp16_accum, void *stream) {
  return mi355x_frwq_sls_multi_impl(tables, n_tables, max_data_rows, kind, idx_is_64, segments, in_line_size, out_line_size, out_kind, out_scale, out_offset, dest_row_stride, fp16_accum, stream);
}

int mi355x_frwq_sls_multi_opts(const mi355x_sls_table *tables, size_t n_tables,
                          size_t max_data_rows, int kind, int idx_is_64,
                          size_t segments, size_t in_line_size,
                          size_t out_line_size, int out_kind, float out_scale,
                          int32_t out_offset, size_t dest_row_stride,
                          int fp16_accum, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_frwq_sls_multi_impl(tables, n_tables, max_data_rows, kind, idx_is_64, segments, in_line_size, out_line_size, out_kind, out_scale, out_offset, dest_row_stride, fp16_accum, stream);
}

static int mi355x_rwq_slws_impl(float *dest, const uint8_t *data, size_t data_rows,
                    const float *scales, const float *offsets, const float *weights,
                    const void *indices, int idx_is_64, size_t num_indices,
                    const int32_t *lengths, size_t segments, size_t line_size,
                    void *stream) {
  MI355X_REQUIRE(segments == 0 || lengths, "lengths is NULL");
  MI355X_REQUIRE(segments == 0 || (scales && offsets), "NULL scales or offsets");
  SlwsExtra x;
  x.sep_scales = scales;
  x.sep_offsets = offsets;
  return slws_dispatch(dest, 0, data, data_rows, MI355X_FUSED_U8_F32, weights, 0, indices,
                       idx_is_64, num_indices, lengths, nullptr, 0, segments, line_size,
                       line_size, 0, stream, x);
}

int mi355x_rwq_slws(float *dest, const uint8_t *data, size_t data_rows,
                    const float *scales, const float *offsets, const float *weights,
                    const void *indices, int idx_is_64, size_t num_indices,
                    const int32_t *lengths, size_t segments, size_t line_size,
                    void *stream) {
  return mi355x_rwq_slws_impl(dest, data, data_rows, scales, offsets, weights, indices, idx_is_64, num_indices, lengths, segments, line_size, stream);
}

int mi355x_rwq_slws_opts(float *dest, const uint8_t *data, size_t data_rows,
                    const float *scales, const float *offsets, const float *weights,
                    const void *indices, int idx_is_64, size_t num_indices,
                    const int32_t *lengths, size_t segments, size_t line_size,
                    void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_rwq_slws_impl(dest, data, data_rows, scales, offsets, weights, indices, idx_is_64, num_indices, lengths, segments, line_size, stream);
}

static int mi355x_frwq_slws_impl(void *dest, int out_is_f16, const uint8_t *data,
                     size_t data_rows, int kind, const void *weights,
                     int weights_are_f16, const void *indices, int idx_is_64,
                     size_t num_indices, const int32_t *lengths,
                     size_t segments, size_t in_line_size,
                     size_t out_line_size, int fp16_accum, void *stream) {
  MI355X_REQUIRE(segments == 0 || lengths, "lengths is NULL");
  return slws_dispatch(dest, out_is_f16, data, data_rows, kind, weights,
                       weights_are_f16, indices, idx_is_64, num_indices,
                       lengths, nullptr, 0, segments, in_line_size,
                       out_line_size, fp16_accum, stream);
}

int mi355x_frwq_slws(void *dest, int out_is_f16, const uint8_t *data,
                     size_t data_rows, int kind, const void *weights,
                     int weights_are_f16, const void *indices, int idx_is_64,
                     size_t num_indices, const int32_t *lengths,
                     size_t segments, size_t in_line_size,
                     size_t out_line_size, int fp16_accum, void *stream) {
  return mi355x_frwq_slws_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, idx_is_64, num_indices, lengths, segments, in_line_size, out_line_size, fp16_accum, stream);
}

int mi355x_frwq_slws_opts(void *dest, int out_is_f16, const uint8_t *data,
                     size_t data_rows, int kind, const void *weights,
                     int weights_are_f16, const void *indices, int idx_is_64,
                     size_t num_indices, const int32_t *lengths,
                     size_t segments, size_t in_line_size,
                     size_t out_line_size, int fp16_accum, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_frwq_slws_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, idx_is_64, num_indices, lengths, segments, in_line_size, out_line_size, fp16_accum, stream);
}

static int mi355x_frwq_slws_noalloc_impl(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *lengths,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream) {
  MI355X_REQUIRE(segments == 0 || lengths, "lengths is NULL");
  MI355X_REQUIRE(segments <= (size_t)kStaticChunks * kChunkBags,
                 "%zu bags: mi355x_frwq_slws_noalloc takes at most %d", segments,
                 kStaticChunks * kChunkBags);
  SlwsExtra x;
  x.static_scratch = true;
  return slws_dispatch(dest, out_is_f16, data, data_rows, kind, weights,
                       weights_are_f16, indices, idx_is_64, num_indices,
                       lengths, nullptr, 0, segments, in_line_size,
                       out_line_size, fp16_accum, stream, x);
}

int mi355x_frwq_slws_noalloc(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *lengths,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream) {
  return mi355x_frwq_slws_noalloc_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, idx_is_64, num_indices, lengths, segments, in_line_size, out_line_size, fp16_accum, stream);
}

int mi355x_frwq_slws_noalloc_opts(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *lengths,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_frwq_slws_noalloc_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, idx_is_64, num_indices, lengths, segments, in_line_size, out_line_size, fp16_accum, stream);
}

static int mi355x_frwq_slws_offsets_impl(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *bag_offsets,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream) {
  MI355X_REQUIRE(segments == 0 || bag_offsets, "bag_offsets is NULL");
  // segments + 1 offsets: every bag reads its two ends, no prefix sum, no
  // scratch and no second launch whatever the number of bags
  return slws_dispatch(dest, out_is_f16, data, data_rows, kind, weights,
                       weights_are_f16, indices, idx_is_64, num_indices, nullptr,
                       bag_offsets, 1, segments, in_line_size, out_line_size,
                       fp16_accum, stream);
}

int mi355x_frwq_slws_offsets(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *bag_offsets,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream) {
  return mi355x_frwq_slws_offsets_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, idx_is_64, num_indices, bag_offsets, segments, in_line_size, out_line_size, fp16_accum, stream);
}

int mi355x_frwq_slws_offsets_opts(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *bag_offsets,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_frwq_slws_offsets_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, idx_is_64, num_indices, bag_offsets, segments, in_line_size, out_line_size, fp16_accum, stream);
}

int mi355x_slws_bag_offsets_host(const int32_t *lengths, size_t segments,
                                 int32_t *bag_offsets) {
  MI355X_REQUIRE(bag_offsets && (segments == 0 || lengths), "NULL vector");
  uint64_t sum = 0;
  bag_offsets[0] = 0;
  for (size_t i = 0; i < segments; i++) {
    sum += lengths[i] > 0 ? (uint64_t)lengths[i] : 0u;   // as the kernels clamp
    MI355X_REQUIRE(sum <= 0x7fffffffull,
                   "the lengths sum past 2^31 - 1 at bag %zu: use the lengths entry point", i);
    bag_offsets[i + 1] = (int32_t)sum;
  }
  return MI355X_OK;
}

int mi355x_slws_reserve_stream(void *stream) {
  return slws_reserve_stream(as_stream(stream));
}

static int mi355x_embedding_bag_rowwise_offsets_impl(
    void *dest, int out_is_f16, const uint8_t *data, size_t data_rows,
    int kind, const void *weights, int weights_are_f16, const int32_t *indices,
    size_t num_indices, const int32_t *offsets, size_t segments,
    int has_end_offset, size_t in_line_size, size_t out_line_size,
    int fp16_accum, void *stream) {
  MI355X_REQUIRE(segments == 0 || offsets, "offsets is NULL");
  if (has_end_offset) {
    MI355X_REQUIRE(segments >= 1, "has_end_offset needs at least one offset");
    segments -= 1;
  }
  return slws_dispatch(dest, out_is_f16, data, data_rows, kind, weights,
                       weights_are_f16, indices, 0, num_indices, nullptr,
                       offsets, has_end_offset, segments, in_line_size,
                       out_line_size, fp16_accum, stream);
}

int mi355x_embedding_bag_rowwise_offsets(
    void *dest, int out_is_f16, const uint8_t *data, size_t data_rows,
    int kind, const void *weights, int weights_are_f16, const int32_t *indices,
    size_t num_indices, const int32_t *offsets, size_t segments,
    int has_end_offset, size_t in_line_size, size_t out_line_size,
    int fp16_accum, void *stream) {
  return mi355x_embedding_bag_rowwise_offsets_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, num_indices, offsets, segments, has_end_offset, in_line_size, out_line_size, fp16_accum, stream);
}

int mi355x_embedding_bag_rowwise_offsets_opts(
    void *dest, int out_is_f16, const uint8_t *data, size_t data_rows,
    int kind, const void *weights, int weights_are_f16, const int32_t *indices,
    size_t num_indices, const int32_t *offsets, size_t segments,
    int has_end_offset, size_t in_line_size, size_t out_line_size,
    int fp16_accum, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_embedding_bag_rowwise_offsets_impl(dest, out_is_f16, data, data_rows, kind, weights, weights_are_f16, indices, num_indices, offsets, segments, has_end_offset, in_line_size, out_line_size, fp16_accum, stream);
}

} // extern "C"
