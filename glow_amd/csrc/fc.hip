// RowwiseQuantizedFullyConnected, FullyConnected and MatMul for int8 tensors
// on the int8 matrix cores (reference
// lib/LLVMIRCodeGen/libjit/libjit_matmul.cpp:254-316, 353-371, 395-450).
// All three are the same contraction with different parameter shapes:
// per-row weight offsets and requantisation vectors for the rowwise form,
// scalars for the other two.
#include "gemm_i8.h"
#include "gemm_skinny.h"
#include "gemm_stream.h"

namespace mi355x {

thread_local int g_tile_override = -1;
thread_local void *g_workspace = nullptr;
thread_local size_t g_workspace_bytes = 0;
thread_local int g_requant_hint = 0;

// dst [cols x rows] = src [rows x cols]^T through a 64x64 LDS tile.
__global__ __launch_bounds__(256) void transpose2d_i8_kernel(
    int8_t *__restrict__ dst, const int8_t *__restrict__ src, int rows,
    int cols) {
  __shared__ int8_t tile[64][64 + 4];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    const int rr = r0 + r, cc = c0 + tx;
    tile[r][tx] = (rr < rows && cc < cols) ? src[(long long)rr * cols + cc] : 0;
  }
  __syncthreads();
  for (int c = ty; c < 64; c += 4) {
    const int cc = c0 + c, rr = r0 + tx;
    if (cc < cols && rr < rows) dst[(long long)cc * rows + rr] = tile[tx][c];
  }
}

// sums[r] = sum_k rows[r][k]; one wavefront per row, 16 bytes per lane and trip.
__global__ __launch_bounds__(256) void rowsum_i8_kernel(
    int32_t *__restrict__ sums, const int8_t *__restrict__ rows, long long n_rows,
    int K, int vec_ok) {
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  const int lane = threadIdx.x & 63;
  const int8_t *p = rows + r * K;
  int acc = 0;
  int k = 0;
  if (vec_ok) {
    for (; k + 1024 <= K; k += 1024) {
      const int4 v = *reinterpret_cast<const int4 *>(p + k + lane * 16);
      acc = __builtin_amdgcn_sdot4(v.x, 0x01010101, acc, false);
      acc = __builtin_amdgcn_sdot4(v.y, 0x01010101, acc, false);
      acc = __builtin_amdgcn_sdot4(v.z, 0x01010101, acc, false);
      acc = __builtin_amdgcn_sdot4(v.w, 0x01010101, acc, false);
    }
  }
  for (int i = k + lane; i < K; i += 64) acc += p[i];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
  if (lane == 0) sums[r] = acc;
}

static bool aligned_rows(const void *p, size_t ld) {
  return ((((uintptr_t)p) & 15) == 0) && (ld % 16 == 0);
}

static int check_dims(size_t M, size_t K, size_t N) {
  MI355X_REQUIRE(M < (1u << 30) && N < (1u << 30) && K < (1u << 30) &&
                     M * K < (1ull << 40) && N * K < (1ull << 40),
                 "matrix dimensions too large");
  return MI355X_OK;
}

// Shared launch path. `w_nk` is [N x K].
static int fc_common(int8_t *out, const int8_t *in, const int8_t *w_nk,
                     const Epilogue &ep_in, size_t M, size_t K, size_t N,
                     bool need_sa, void *stream) {
  if (M == 0 || N == 0) return MI355X_OK;
  DenseRows A{in, (long long)K, (int)M};
  DenseRows B{w_nk, (long long)K, (int)N};
  Epilogue ep = ep_in;
  ep.out = out;
  ep.ldc = (long long)N;
  const bool aligned = aligned_rows(in, K) && aligned_rows(w_nk, K);
  const bool need_sb = ep.a_off != 0 && !ep.sum_b;
  // few output tiles: 32x32 tiles with the K loop split over the waves (tile 6
  // forces it wherever the kernel can run at all, for tuning)
  const GemmShape g{(int)M, (int)N, (int)K, 1, 0};
  const bool can_skinny = aligned && !need_sa && !need_sb && !ep.add.res && K >= 32 &&
                          K % 32 == 0 && (long long)((M + 31) / 32) * ((N + 31) / 32) < (1 << 22);
  if ((g_tile_override == 6 && can_skinny) ||
      (g_tile_override < 0 && skinny_applies(g, ep, need_sa, need_sb, aligned))) {
    ep.fast = g_requant_hint & 3;
    return gemm_skinny_launch(A, B, ep, g, as_stream(stream));
  }
  // many rows over 64, 128 or 256 inputs: the streaming kernel (by its shape
  // rule, or tile 8)
  if ((g_tile_override == 8 || (g_tile_override < 0 && stream_applies((int)M, (int)N))) &&
      stream_can_run((int)M, (int)N, (int)K, need_sa, need_sb, aligned, ep)) {
    StreamRows R{};
    R.in = in; R.ld = (long long)K; R.dense = 1; R.seg_chunks = (int)(K / 32);
    ep.fast = g_requant_hint & 3;
    return gemm_stream_launch(R, w_nk, ep, (int)M, (int)N, (int)K, as_stream(stream));
  }
  // Tiles 6..8 name one special kernel each; a launch that kernel cannot serve
  // says so instead of running another kernel under the asked-for number.
  if (g_tile_override >= 6 && g_tile_override <= 8)
    return fail(MI355X_ERR_NOT_SUPPORTED,
                "tile %d does not apply to this product (shape, alignment or offsets)",
                g_tile_override);
  return gemm_dispatch(A, B, ep, (int)M, (int)N, (int)K, 1, 0, need_sa, need_sb,
                       aligned, as_stream(stream));
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

int mi355x_gemm_tile_override(int tile) {
  MI355X_REQUIRE(tile >= -1 && tile <= 12, "tile %d outside [-1, 12]", tile);
  g_tile_override = tile;
  return MI355X_OK;
}

int mi355x_gemm_splitk_workspace_bytes(size_t M, size_t N, size_t K, size_t groups, int named,
                                       size_t *bytes) {
  MI355X_REQUIRE(bytes, "NULL result");
  *bytes = 0;
  if (M == 0 || N == 0 || K < 2 * (size_t)kBK || K % kBK != 0 || groups == 0) return MI355X_OK;
  MI355X_REQUIRE(M < (1ull << 31) && N < (1ull << 31) && K < (1ull << 31) && groups < 65536,
                 "problem too large");
  const GemmShape g{(int)M, (int)N, (int)K, (int)groups, 0};
  const int splits = splitk_choice(g, gemm_cus(), named != 0);
  if (splits >= 2) *bytes = splitk_workspace_bytes(g, splits);
  return MI355X_OK;
}

int mi355x_gemm_requant_hint(int flags) {
  MI355X_REQUIRE(flags >= 0 && flags <= 3 && flags != 2,
                 "hint %d: bit 1 (no pre-shifts) needs bit 0 (24-bit operands)", flags);
  g_requant_hint = flags;
  return MI355X_OK;
}

int mi355x_transpose2d_i8(int8_t *dst, const int8_t *src, size_t rows,
                          size_t cols, void *stream) {
  if (rows == 0 || cols == 0) return MI355X_OK;
  MI355X_REQUIRE(dst && src, "NULL tensor");
  MI355X_REQUIRE(rows < (1u << 30) && cols < (1u << 30) &&
                     (rows + 63) / 64 < 65536,
                 "matrix too large");
  dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  hipLaunchKernelGGL(transpose2d_i8_kernel, grid, dim3(256), 0,
                     as_stream(stream), dst, src, (int)rows, (int)cols);
  return check_launch("transpose2d_i8");
}

int mi355x_rowsum_i8(int32_t *sums, const int8_t *rows, size_t n_rows, size_t K,
                     void *stream) {
  if (n_rows == 0) return MI355X_OK;
  MI355X_REQUIRE(sums && (rows || K == 0), "NULL tensor");
  MI355X_REQUIRE(K < (1u << 30) && (n_rows + 3) / 4 < 0x7fffffffu,
                 "matrix too large");
  hipLaunchKernelGGL(rowsum_i8_kernel, dim3((unsigned)((n_rows + 3) / 4)),
                     dim3(256), 0, as_stream(stream), sums, rows,
                     (long long)n_rows, (int)K, (int)aligned_rows(rows, K));
  return check_launch("rowsum_i8");
}

static int mi355x_rwq_fc_i8_impl(int8_t *out, const int8_t *in, const int8_t *weights,
                     const void *bias, int bias_is_i8,
                     const int32_t *weights_offsets, const int32_t *bias_pre,
                     const int32_t *bias_post, const int32_t *bias_scale,
                     const int32_t *out_pre, const int32_t *out_post,
                     const int32_t *out_scale, size_t M, size_t K, size_t N,
                     int32_t out_offset, int32_t in_offset,
                     int32_t bias_offset, int weights_offsets_all_zero,
                     const int32_t *weights_row_sums, void *stream) {
  if (M == 0 || N == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in && weights && bias, "NULL tensor");
  MI355X_REQUIRE(weights_offsets && bias_pre && bias_post && bias_scale &&
                     out_pre && out_post && out_scale,
                 "NULL per-row parameter vector");
  int rc = check_dims(M, K, N);
  if (rc != MI355X_OK) return rc;
  Epilogue ep{};
  ep.bias = bias;
  ep.bias_is_i8 = bias_is_i8;
  ep.b_off = ColParam{nullptr, bias_offset};
  ep.bias_pre = ColParam{bias_pre, 0};
  ep.bias_post = ColParam{bias_post, 0};
  ep.bias_scale = ColParam{bias_scale, 0};
  ep.w_off = ColParam{weights_offsets, 0};
  ep.out_pre = ColParam{out_pre, 0};
  ep.out_post = ColParam{out_post, 0};
  ep.out_scale = ColParam{out_scale, 0};
  ep.a_off = in_offset;
  ep.out_off = out_offset;
  ep.act = MI355X_ACT_NONE;
  ep.sum_b = weights_row_sums;
  return fc_common(out, in, weights, ep, M, K, N, !weights_offsets_all_zero,
                   stream);
}

int mi355x_rwq_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                     const void *bias, int bias_is_i8,
                     const int32_t *weights_offsets, const int32_t *bias_pre,
                     const int32_t *bias_post, const int32_t *bias_scale,
                     const int32_t *out_pre, const int32_t *out_post,
                     const int32_t *out_scale, size_t M, size_t K, size_t N,
                     int32_t out_offset, int32_t in_offset,
                     int32_t bias_offset, int weights_offsets_all_zero,
                     const int32_t *weights_row_sums, void *stream) {
  return mi355x_rwq_fc_i8_impl(out, in, weights, bias, bias_is_i8, weights_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, M, K, N, out_offset, in_offset, bias_offset, weights_offsets_all_zero, weights_row_sums, stream);
}

int mi355x_rwq_fc_i8_opts(int8_t *out, const int8_t *in, const int8_t *weights,
                     const void *bias, int bias_is_i8,
                     const int32_t *weights_offsets, const int32_t *bias_pre,
                     const int32_t *bias_post, const int32_t *bias_scale,
                     const int32_t *out_pre, const int32_t *out_post,
                     const int32_t *out_scale, size_t M, size_t K, size_t N,
                     int32_t out_offset, int32_t in_offset,
                     int32_t bias_offset, int weights_offsets_all_zero,
                     const int32_t *weights_row_sums, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_rwq_fc_i8_impl(out, in, weights, bias, bias_is_i8, weights_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, M, K, N, out_offset, in_offset, bias_offset, weights_offsets_all_zero, weights_row_sums, stream);
}

static int mi355x_rwq_fc_relu_i8_impl(int8_t *out, const int8_t *in, const int8_t *weights,
                          const void *bias, int bias_is_i8,
                          const int32_t *weights_offsets, const int32_t *bias_pre,
                          const int32_t *bias_post, const int32_t *bias_scale,
                          const int32_t *out_pre, const int32_t *out_post,
                          const int32_t *out_scale, size_t M, size_t K, size_t N,
                          int32_t fc_offset, int32_t in_offset, int32_t bias_offset,
                          int weights_offsets_all_zero, const int32_t *weights_row_sums,
                          int32_t relu_offset, int32_t relu_pre, int32_t relu_post,
                          int32_t relu_scale, void *stream) {
  if (M == 0 || N == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in && weights && bias, "NULL tensor");
  MI355X_REQUIRE(weights_offsets && bias_pre && bias_post && bias_scale &&
                     out_pre && out_post && out_scale,
                 "NULL per-row parameter vector");
  MI355X_REQUIRE(shift_ok(relu_pre) && shift_ok(relu_post), "relu pre/post shift outside [0, 31]");
  MI355X_REQUIRE(fc_offset >= -128 && fc_offset <= 127,
                 "offset %d of the FullyConnected result outside the int8 range", fc_offset);
  int rc = check_dims(M, K, N);
  if (rc != MI355X_OK) return rc;
  Epilogue ep{};
  ep.bias = bias;
  ep.bias_is_i8 = bias_is_i8;
  ep.b_off = ColParam{nullptr, bias_offset};
  ep.bias_pre = ColParam{bias_pre, 0};
  ep.bias_post = ColParam{bias_post, 0};
  ep.bias_scale = ColParam{bias_scale, 0};
  ep.w_off = ColParam{weights_offsets, 0};
  ep.out_pre = ColParam{out_pre, 0};
  ep.out_post = ColParam{out_post, 0};
  ep.out_scale = ColParam{out_scale, 0};
  ep.a_off = in_offset;
  ep.out_off = fc_offset;
  ep.act = MI355X_ACT_NONE;
  ep.sum_b = weights_row_sums;
  ep.add.res = nullptr;
  ep.add.relu = 1;
  ep.add.sum_off = fc_offset;
  ep.add.dest_off = relu_offset;
  ep.add.dest_pre = relu_pre;
  ep.add.dest_post = relu_post;
  ep.add.dest_scale = relu_scale;
  ep.add.small = relu_scale > -(1 << 23) && relu_scale < (1 << 23);
  return fc_common(out, in, weights, ep, M, K, N, !weights_offsets_all_zero,
                   stream);
}

int mi355x_rwq_fc_relu_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                          const void *bias, int bias_is_i8,
                          const int32_t *weights_offsets, const int32_t *bias_pre,
                          const int32_t *bias_post, const int32_t *bias_scale,
                          const int32_t *out_pre, const int32_t *out_post,
                          const int32_t *out_scale, size_t M, size_t K, size_t N,
                          int32_t fc_offset, int32_t in_offset, int32_t bias_offset,
                          int weights_offsets_all_zero, const int32_t *weights_row_sums,
                          int32_t relu_offset, int32_t relu_pre, int32_t relu_post,
                          int32_t relu_scale, void *stream) {
  return mi355x_rwq_fc_relu_i8_impl(out, in, weights, bias, bias_is_i8, weights_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, M, K, N, fc_offset, in_offset, bias_offset, weights_offsets_all_zero, weights_row_sums, relu_offset, relu_pre, relu_post, relu_scale, stream);
}

int mi355x_rwq_fc_relu_i8_opts(int8_t *out, const int8_t *in, const int8_t *weights,
                          const void *bias, int bias_is_i8,
                          const int32_t *weights_offsets, const int32_t *bias_pre,
                          const int32_t *bias_post, const int32_t *bias_scale,
                          const int32_t *out_pre, const int32_t *out_post,
                          const int32_t *out_scale, size_t M, size_t K, size_t N,
                          int32_t fc_offset, int32_t in_offset, int32_t bias_offset,
                          int weights_offsets_all_zero, const int32_t *weights_row_sums,
                          int32_t relu_offset, int32_t relu_pre, int32_t relu_post,
                          int32_t relu_scale, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_rwq_fc_relu_i8_impl(out, in, weights, bias, bias_is_i8, weights_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, M, K, N, fc_offset, in_offset, bias_offset, weights_offsets_all_zero, weights_row_sums, relu_offset, relu_pre, relu_post, relu_scale, stream);
}

static int mi355x_fc_i8_impl(int8_t *out, const int8_t *in, const int8_t *weights_kn,
                 int8_t *weights_nk_workspace, int repack, const void *bias,
                 int bias_is_i8, size_t M, size_t K, size_t N,
                 int32_t out_offset, int32_t in_offset, int32_t weights_offset,
                 int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                 int32_t bias_scale, int32_t out_pre, int32_t out_post,
                 int32_t out_scale, const int32_t *weights_row_sums,
                 void *stream) {
  if (M == 0 || N == 0) return MI355X_OK;
  MI355X_REQUIRE(out && in && weights_nk_workspace && bias, "NULL tensor");
  MI355X_REQUIRE(shift_ok(bias_pre) && shift_ok(bias_post) &&
                     shift_ok(out_pre) && shift_ok(out_post),
                 "pre/post shift outside [0, 31]");
  int rc = check_dims(M, K, N);
  if (rc != MI355X_OK) return rc;
  if (repack) {
    MI355X_REQUIRE(weights_kn, "weights_kn is NULL with repack set");
    rc = mi355x_transpose2d_i8(weights_nk_workspace, weights_kn, K, N, stream);
    if (rc != MI355X_OK) return rc;
  }
  Epilogue ep{};
  ep.bias = bias;
  ep.bias_is_i8 = bias_is_i8;
  ep.b_off = ColParam{nullptr, bias_offset};
  ep.bias_pre = ColParam{nullptr, bias_pre};
  ep.bias_post = ColParam{nullptr, bias_post};
  ep.bias_scale = ColParam{nullptr, bias_scale};
  ep.w_off = ColParam{nullptr, weights_offset};
  ep.out_pre = ColParam{nullptr, out_pre};
  ep.out_post = ColParam{nullptr, out_post};
  ep.out_scale = ColParam{nullptr, out_scale};
  ep.a_off = in_offset;
  ep.out_off = out_offset;
  ep.act = MI355X_ACT_NONE;
  ep.sum_b = weights_row_sums;
  return fc_common(out, in, weights_nk_workspace, ep, M, K, N,
                   weights_offset != 0, stream);
}

int mi355x_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights_kn,
                 int8_t *weights_nk_workspace, int repack, const void *bias,
                 int bias_is_i8, size_t M, size_t K, size_t N,
                 int32_t out_offset, int32_t in_offset, int32_t weights_offset,
                 int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                 int32_t bias_scale, int32_t out_pre, int32_t out_post,
                 int32_t out_scale, const int32_t *weights_row_sums,
                 void *stream) {
  return mi355x_fc_i8_impl(out, in, weights_kn, weights_nk_workspace, repack, bias, bias_is_i8, M, K, N, out_offset, in_offset, weights_offset, bias_offset, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, weights_row_sums, stream);
}

int mi355x_fc_i8_opts(int8_t *out, const int8_t *in, const int8_t *weights_kn,
                 int8_t *weights_nk_workspace, int repack, const void *bias,
                 int bias_is_i8, size_t M, size_t K, size_t N,
                 int32_t out_offset, int32_t in_offset, int32_t weights_offset,
                 int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                 int32_t bias_scale, int32_t out_pre, int32_t out_post,
                 int32_t out_scale, const int32_t *weights_row_sums,
                 void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_fc_i8_impl(out, in, weights_kn, weights_nk_workspace, repack, bias, bias_is_i8, M, K, N, out_offset, in_offset, weights_offset, bias_offset, bias_pre, bias_post, bias_scale, out_pre, out_post, out_scale, weights_row_sums, stream);
}

static int mi355x_matmul_i8_impl(int8_t *out, const int8_t *lhs, const int8_t *rhs_kn,
                     int8_t *rhs_nk_workspace, int repack, size_t M, size_t K,
                     size_t N, int32_t out_offset, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, void *stream) {
  if (M == 0 || N == 0) return MI355X_OK;
  MI355X_REQUIRE(out && lhs && rhs_nk_workspace, "NULL tensor");
  MI355X_REQUIRE(shift_ok(out_pre) && shift_ok(out_post),
                 "pre/post shift outside [0, 31]");
  int rc = check_dims(M, K, N);
  if (rc != MI355X_OK) return rc;
  if (repack) {
    MI355X_REQUIRE(rhs_kn, "rhs_kn is NULL with repack set");
    rc = mi355x_transpose2d_i8(rhs_nk_workspace, rhs_kn, K, N, stream);
    if (rc != MI355X_OK) return rc;
  }
  Epilogue ep{};
  ep.bias = nullptr;
  ep.w_off = ColParam{nullptr, rhs_offset};
  ep.out_pre = ColParam{nullptr, out_pre};
  ep.out_post = ColParam{nullptr, out_post};
  ep.out_scale = ColParam{nullptr, out_scale};
  ep.a_off = lhs_offset;
  ep.out_off = out_offset;
  ep.act = MI355X_ACT_NONE;
  return fc_common(out, lhs, rhs_nk_workspace, ep, M, K, N, rhs_offset != 0,
                   stream);
}

int mi355x_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_kn,
                     int8_t *rhs_nk_workspace, int repack, size_t M, size_t K,
                     size_t N, int32_t out_offset, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, void *stream) {
  return mi355x_matmul_i8_impl(out, lhs, rhs_kn, rhs_nk_workspace, repack, M, K, N, out_offset, lhs_offset, rhs_offset, out_pre, out_post, out_scale, stream);
}

int mi355x_matmul_i8_opts(int8_t *out, const int8_t *lhs, const int8_t *rhs_kn,
                     int8_t *rhs_nk_workspace, int repack, size_t M, size_t K,
                     size_t N, int32_t out_offset, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, void *stream,
    const mi355x_launch_opts *opts) {
  OptsScope scope(opts);
  if (scope.rc != MI355X_OK) return scope.rc;
  return mi355x_matmul_i8_impl(out, lhs, rhs_kn, rhs_nk_workspace, repack, M, K, N, out_offset, lhs_offset, rhs_offset, out_pre, out_post, out_scale, stream);
}

} // extern "C"
