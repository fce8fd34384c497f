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

// The same product, the same chain of fmaf per output (so the same bits), laid out for a few
// rows: a decode step's products in the 32-bit path are bound by reading W, and 64 x 64 tiles
// give eight rows against [3584, 18944] 56 workgroups that each walk 4.8 MB.  Here a workgroup
// owns 16 x 16 outputs, one per thread, and walks K in slices of 64 that travel global ->
// registers -> LDS (two buffers, one barrier a slice); a thread fetches four consecutive k of one
// row (one 16-byte load where K allows), so a row's slice is 256 contiguous bytes, and its loads
// are GF_AHEAD slices ahead of the arithmetic (a ring of registers).  Every load is unconditional
// (addresses clamped into the tensor, what lies outside replaced by zero afterwards), so that
// the compiler can count the loads in flight.
#define GF_BM 16
#define GF_BN 16
#define GF_BK 64
#define GF_ROW (GF_BK + 4)  // floats; keeps rows 16-byte aligned and apart in the banks
#ifndef GF_AHEAD
#define GF_AHEAD 2  // slices of loads in flight (even)
#endif

typedef float gf_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int gf_u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void few_rows_load4(float (&dst)[4], const float* p) {
  const gf_f32x4 v = *reinterpret_cast<const gf_f32x4*>(p);
  dst[0] = v[0], dst[1] = v[1], dst[2] = v[2], dst[3] = v[3];
}
__device__ __forceinline__ void few_rows_load4(float (&dst)[4], const bf16_t* p) {
  const gf_u32x2 v = *reinterpret_cast<const gf_u32x2*>(p);
  dst[0] = __uint_as_float(v[0] << 16), dst[1] = __uint_as_float(v[0] & 0xffff0000u);
  dst[2] = __uint_as_float(v[1] << 16), dst[3] = __uint_as_float(v[1] & 0xffff0000u);
}

// Four consecutive k of one row, from k0 on; zeros for a row or a k outside the tensor.  VEC: K, the
// row stride and the base address are multiples of four elements, so the four lie in the tensor
// together or not at all and travel as one load.
template <bool VEC, typename TIn>
__device__ __forceinline__ void few_rows_fetch(float (&dst)[4], const TIn* base, long stride, int row, int rows, int k0,
                                               int k) {
  const TIn* from = base + (size_t)min(row, rows - 1) * stride;
  if (VEC) {
    few_rows_load4(dst, from + min(k0, k - 4));
    const bool inside = row < rows && k0 < k;
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = inside ? dst[i] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = to_float(from[min(k0 + i, k - 1)]);
      dst[i] = (row < rows && k0 + i < k) ? v : 0.f;
    }
  }
}

template <bool VEC, typename TIn, typename TOut>
__global__ void __launch_bounds__(256)
gemm_plain_few_rows_kernel(TOut* __restrict__ y, const TIn* __restrict__ x, const TIn* __restrict__ w,
                           const TIn* __restrict__ bias, int m, int n, int k, long x_stride, long y_stride) {
  __shared__ __attribute__((aligned(16))) float xs[2][GF_BM][GF_ROW];
  __shared__ __attribute__((aligned(16))) float ws[2][GF_BN][GF_ROW];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GF_BM;
  const int n0 = blockIdx.x * GF_BN;
  const int fetch_row = tid / 16;       // the row of both tiles this thread fetches ...
  const int fetch_k = (tid % 16) * 4;   // ... and its four consecutive k within a slice
  const int out_m = tid % 16;           // the output this thread owns
  const int out_n = tid / 16;
  float xr[GF_AHEAD][4], wr[GF_AHEAD][4];  // slot j: a slice whose number is j modulo GF_AHEAD
  auto fetch = [&](int slot, int slice) __attribute__((always_inline)) {
    few_rows_fetch<VEC>(xr[slot], x, x_stride, m0 + fetch_row, m, slice * GF_BK + fetch_k, k);
    few_rows_fetch<VEC>(wr[slot], w, (long)k, n0 + fetch_row, n, slice * GF_BK + fetch_k, k);
  };
  auto stage = [&](int slot, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xs[buf][fetch_row][fetch_k + i] = xr[slot][i];
      ws[buf][fetch_row][fetch_k + i] = wr[slot][i];
    }
  };
#pragma unroll
  for (int j = 0; j < GF_AHEAD; ++j) fetch(j, j);  // slices past the end read the last k again and count as zeros
  stage(0, 0);
  __syncthreads();
  float acc = 0.f;
  const int slices = (k + GF_BK - 1) / GF_BK;
  for (int s0 = 0; s0 < slices; s0 += GF_AHEAD) {
#pragma unroll
    for (int j = 0; j < GF_AHEAD; ++j) {
      const int s = s0 + j;
      if (s < slices) {  // the same for every thread of the grid
        const int buf = j & 1;  // GF_AHEAD is even: slice s lies in buffer s & 1 = j & 1
        fetch(j, s + GF_AHEAD);  // slot j held slice s, which is in LDS already
        const float* a = xs[buf][out_m];
        const float* b = ws[buf][out_n];
#pragma unroll
        for (int kk = 0; kk < GF_BK; ++kk) acc = fmaf(a[kk], b[kk], acc);  // in the order of k
        // The other buffer was last read in the slice before this one, which every thread has left.
        stage((j + 1) % GF_AHEAD, buf ^ 1);
        __syncthreads();
      }
    }
  }
  const int gm = m0 + out_m, gn = n0 + out_n;
  if (gm < m && gn < n) {
    if (bias) acc += to_float(bias[gn]);
    y[(size_t)gm * y_stride + gn] = from_float<TOut>(acc);
  }
}

// Rows up to which the layout for a few rows runs.
#define GF_MAX_ROWS 32

// dtype: type of x, w and bias.  out_f32 != 0: y is float whatever dtype is.
extern "C" int ts_gemm_plain(void* y, const void* x, const void* w, const void* bias, int m, int n,
                             int k, long x_stride, long y_stride, int dtype, int out_f32,
                             hipStream_t stream) {
  if (m == 0 || n == 0) return TS_OK;
  if (!y || !x || !w || k < 1 || x_stride < k || y_stride < n) return TS_ERR_ARG;
  dim3 grid((n + GP_BN - 1) / GP_BN, (m + GP_BM - 1) / GP_BM), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  if (m <= GF_MAX_ROWS) {
    dim3 few((n + GF_BN - 1) / GF_BN, (m + GF_BM - 1) / GF_BM);
    const size_t elem = dtype == TS_F32 ? 4 : 2;
    const bool vec = k % 4 == 0 && x_stride % 4 == 0 && (uintptr_t)x % (4 * elem) == 0 && (uintptr_t)w % (4 * elem) == 0;
#define TS_FEW_ROWS(V, TI, TO) \
  hipLaunchKernelGGL((gemm_plain_few_rows_kernel<V, TI, TO>), few, block, 0, stream, (TO*)y, (const TI*)x, (const TI*)w, \
                     (const TI*)bias, m, n, k, x_stride, y_stride)
    if (dtype == TS_F32) {
      if (vec) TS_FEW_ROWS(true, float, float); else TS_FEW_ROWS(false, float, float);
    } else if (dtype == TS_BF16 && out_f32) {
      if (vec) TS_FEW_ROWS(true, bf16_t, float); else TS_FEW_ROWS(false, bf16_t, float);
    } else if (dtype == TS_BF16) {
      if (vec) TS_FEW_ROWS(true, bf16_t, bf16_t); else TS_FEW_ROWS(false, bf16_t, bf16_t);
    } else {
      return TS_ERR_DTYPE;
    }
#undef TS_FEW_ROWS
    return ts_launch_status();
  }
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
