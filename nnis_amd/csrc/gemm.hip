// Matrix products of the projections: Y[M, N] = X[M, K] * W[N, K]^T, the weight
// in the checkpoint's [out, in] orientation (K contiguous in both operands).
//
// gemm_ordered_kernel is the 32-bit path: operands of either storage type are
// widened exactly, every output element is one fused-multiply-add chain over
// ascending k that starts at +0, as in the reference's kernels
// (/root/reference/crates/nnis-kernels/src/gemm.rs:16-64, gemv.rs:45-62), so a
// row's result depends neither on the other rows nor on where the tile lies.
#include "common.h"

namespace {

constexpr int kTile = 64;   // output tile edge of the ordered kernel
constexpr int kStepK = 16;  // k extent staged per iteration

__global__ __launch_bounds__(256) void gemm_ordered_kernel(const void* __restrict__ x, int x_dtype,
                                                           const void* __restrict__ w, int w_dtype,
                                                           void* __restrict__ y, int y_dtype, int m, int n, int k) {
  __shared__ float xs[kStepK][kTile + 1];
  __shared__ float ws[kStepK][kTile + 1];
  const int tid = threadIdx.x;
  const int row0 = blockIdx.y * kTile;
  const int col0 = blockIdx.x * kTile;
  const int ty = tid / 16, tx = tid % 16;
  // staging: thread loads 4 consecutive k of one row of each operand
  const int load_row = tid / 4;
  const int load_k = (tid % 4) * 4;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

  for (int k0 = 0; k0 < k; k0 += kStepK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int kk = k0 + load_k + e;
      const int xr = row0 + load_row;
      const int wr = col0 + load_row;
      xs[load_k + e][load_row] = (xr < m && kk < k) ? load_as_f32(x, x_dtype, (size_t)xr * k + kk) : 0.0f;
      ws[load_k + e][load_row] = (wr < n && kk < k) ? load_as_f32(w, w_dtype, (size_t)wr * k + kk) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kStepK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < n) store_from_f32(y, y_dtype, (size_t)r * n + c, acc[i][j]);
    }
  }
}

}  // namespace

extern "C" int nnis_gemm_ordered(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype, int m,
                                 int n, int k, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype) && nnis_dtype_ok(w_dtype) && nnis_dtype_ok(y_dtype),
               "gemm: unknown dtype (x %d, w %d, y %d)", x_dtype, w_dtype, y_dtype);
  NNIS_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm: bad sizes m=%d n=%d k=%d", m, n, k);
  if (m == 0) return 0;
  const dim3 grid((n + kTile - 1) / kTile, (m + kTile - 1) / kTile);
  NNIS_REQUIRE(grid.y <= 65535, "gemm: %d rows exceed the grid limit", m);
  hipLaunchKernelGGL(gemm_ordered_kernel, grid, dim3(256), 0, (hipStream_t)stream, x, x_dtype, w, w_dtype, y, y_dtype,
                     m, n, k);
  NNIS_LAUNCH_CHECK("gemm_ordered");
  return 0;
}
