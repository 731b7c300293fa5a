// RowwiseQuantizedFullyConnected, FullyConnected and MatMul for int8 tensors
// on the int8 matrix cores (reference
// lib/LLVMIRCodeGen/libjit/libjit_matmul.cpp:254-316, 353-371, 395-450).
// All three are the same contraction with different parameter shapes:
// per-row weight offsets and requantisation vectors for the rowwise form,
// scalars for the other two.
#include "gemm_i8.h"

namespace mi355x {

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
  const bool al_a = aligned_rows(in, K), al_b = aligned_rows(w_nk, K);
  const bool need_sb = ep.a_off != 0;
  return gemm_dispatch(A, B, ep, (int)M, (int)N, (int)K, 1, 0, need_sa, need_sb,
                       al_a, al_b, as_stream(stream));
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

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

int mi355x_rwq_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                     const void *bias, int bias_is_i8,
                     const int32_t *weights_offsets, const int32_t *bias_pre,
                     const int32_t *bias_post, const int32_t *bias_scale,
                     const int32_t *out_pre, const int32_t *out_post,
                     const int32_t *out_scale, size_t M, size_t K, size_t N,
                     int32_t out_offset, int32_t in_offset,
                     int32_t bias_offset, int weights_offsets_all_zero,
                     void *stream) {
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
  return fc_common(out, in, weights, ep, M, K, N, !weights_offsets_all_zero,
                   stream);
}

int mi355x_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights_kn,
                 int8_t *weights_nk_workspace, int repack, const void *bias,
                 int bias_is_i8, size_t M, size_t K, size_t N,
                 int32_t out_offset, int32_t in_offset, int32_t weights_offset,
                 int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                 int32_t bias_scale, int32_t out_pre, int32_t out_post,
                 int32_t out_scale, void *stream) {
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
  return fc_common(out, in, weights_nk_workspace, ep, M, K, N,
                   weights_offset != 0, stream);
}

int mi355x_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_kn,
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

} // extern "C"
