// Shared device helpers for the gfx950 kernels: storage types, wavefront reductions, error codes.
//
// Every kernel entry point is `extern "C"`, takes raw device pointers and a hipStream_t and
// returns 0 or one of the TS_ERR_* codes; shapes are validated on the host before any launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TS_OK 0
#define TS_ERR_DTYPE 1     // dtype code is not one of TS_F32 / TS_BF16
#define TS_ERR_SHAPE 2     // a size the kernel does not take
#define TS_ERR_LAUNCH 3    // hipGetLastError() after the launch was not hipSuccess
#define TS_ERR_ARG 4       // null pointer or inconsistent arguments

#define TS_F32 0
#define TS_BF16 1

#define TS_WAVE 64

// bfloat16 as raw bits; conversions written out so that rounding is the same everywhere
// (round to nearest even, NaN kept quiet).
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

template <typename T>
__device__ __forceinline__ T from_float(float v);

template <>
__device__ __forceinline__ float from_float<float>(float v) {
  return v;
}

template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
  uint32_t u = __float_as_uint(v);
  bf16_t out;
  if ((u & 0x7fffffffu) > 0x7f800000u) {  // NaN
    out.bits = (uint16_t)((u >> 16) | 0x0040u);
    return out;
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  out.bits = (uint16_t)(u >> 16);
  return out;
}

// Round a 32-bit value to the storage type and back: the value the storage type would hold.
template <typename T>
__device__ __forceinline__ float round_to(float v) {
  return to_float(from_float<T>(v));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TS_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TS_WAVE));
  return v;
}

// Sum over a block of `blockDim.x` threads (a multiple of 64, at most 1024); `scratch` holds at
// least 16 floats of LDS.  Every thread returns the total.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const int waves = (blockDim.x + TS_WAVE - 1) / TS_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const int waves = (blockDim.x + TS_WAVE - 1) / TS_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

static inline int ts_launch_status() { return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH; }
