// Y[M, N] = X[M, K] * W[N, K]^T (+ bias[N]) with plain 32-bit fused multiply-adds: no matrix
// cores, no reduced-precision mode.  This is the product of the true 32-bit path (the
// reference's F.linear, src/turboserve/engine/model/layers.py:142, at dtype float32) and the
// checked stand-in for any faster product.  Every output element is one k-ordered chain of
// fmaf, so a row's result does not depend on which other rows are in the batch.
//
// Tiles of 64 x 64 outputs per 256-thread block, 16-deep slices of K staged through LDS; every
// load and store is bounds-checked, so M, N and K are arbitrary.
#include "common.hpp"

#define GP_BM 64
#define GP_BN 64
#define GP_BK 16

template <typename TIn, typename TOut>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(TOut* __restrict__ y, const TIn* __restrict__ x, const TIn* __restrict__ w,
                  const TIn* __restrict__ bias, int m, int n, int k, long x_stride, long y_stride) {
  __shared__ float xs[GP_BK][GP_BM + 1];
  __shared__ float ws[GP_BK][GP_BN + 1];
  const int tid = threadIdx.x;
  const int tx = tid % 16;
  const int ty = tid / 16;
  const int m0 = blockIdx.y * GP_BM;
  const int n0 = blockIdx.x * GP_BN;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < k; k0 += GP_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      const int r = idx / GP_BK;
      const int c = idx % GP_BK;
      const int gm = m0 + r;
      const int gn = n0 + r;
      const int gk = k0 + c;
      xs[c][r] = (gm < m && gk < k) ? to_float(x[(size_t)gm * x_stride + gk]) : 0.f;
      ws[c][r] = (gn < n && gk < k) ? to_float(w[(size_t)gn * k + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GP_BK; ++kk) {
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
    const int gm = m0 + ty * 4 + i;
    if (gm >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= n) continue;
      float v = acc[i][j];
      if (bias) v += to_float(bias[gn]);
      y[(size_t)gm * y_stride + gn] = from_float<TOut>(v);
    }
  }
}

// dtype: type of x, w and bias.  out_f32 != 0: y is float whatever dtype is.
extern "C" int ts_gemm_plain(void* y, const void* x, const void* w, const void* bias, int m, int n,
                             int k, long x_stride, long y_stride, int dtype, int out_f32,
                             hipStream_t stream) {
  if (m == 0 || n == 0) return TS_OK;
  if (!y || !x || !w || k < 1 || x_stride < k || y_stride < n) return TS_ERR_ARG;
  dim3 grid((n + GP_BN - 1) / GP_BN, (m + GP_BM - 1) / GP_BM), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  if (dtype == TS_F32)
    hipLaunchKernelGGL((gemm_plain_kernel<float, float>), grid, block, 0, stream, (float*)y, (const float*)x, (const float*)w, (const float*)bias, m, n, k, x_stride, y_stride);
  else if (dtype == TS_BF16 && out_f32)
    hipLaunchKernelGGL((gemm_plain_kernel<bf16_t, float>), grid, block, 0, stream, (float*)y, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, m, n, k, x_stride, y_stride);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL((gemm_plain_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (bf16_t*)y, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, m, n, k, x_stride, y_stride);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
