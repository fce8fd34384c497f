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

// Sums and maxima over a wavefront by data-parallel moves between lanes (an instruction each;
// the shuffles the compiler makes of __shfl_xor go through the LDS crossbar and cost six trips of
// some hundred cycles).  Lanes meet in a fixed order: the four of a quad, the two quads of a
// half row, the two halves of a row of 16, then the rows; every lane returns the result.  All 64
// lanes must be active at the call (a lane that is switched off contributes nothing, where a
// shuffle would still read its register): call them from code the whole wavefront runs.
template <int CONTROL, int ROW_MASK>
__device__ __forceinline__ float lanes_moved(float keep, float v) {
  // Lanes of rows outside ROW_MASK, and lanes whose source does not exist, get `keep`.
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, keep), __builtin_bit_cast(int, v),
                                                               CONTROL, ROW_MASK, 0xF, false));
}

__device__ __forceinline__ float wave_sum(float v) {
  v += lanes_moved<0xB1, 0xF>(0.f, v);   // quad_perm [1,0,3,2]
  v += lanes_moved<0x4E, 0xF>(0.f, v);   // quad_perm [2,3,0,1]
  v += lanes_moved<0x141, 0xF>(0.f, v);  // row_half_mirror
  v += lanes_moved<0x140, 0xF>(0.f, v);  // row_mirror: every lane holds its row's sum
  v += lanes_moved<0x142, 0xA>(0.f, v);  // row_bcast15 into rows 1 and 3
  v += lanes_moved<0x143, 0xC>(0.f, v);  // row_bcast31 into rows 2 and 3: row 3 holds all
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), TS_WAVE - 1));
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lanes_moved<0xB1, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x4E, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x141, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x140, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x142, 0xA>(v, v));
  v = fmaxf(v, lanes_moved<0x143, 0xC>(v, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), TS_WAVE - 1));
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

// A 16-byte load of data that a kernel reads once (weights, cached keys and values): marked
// non-temporal, so that it does not displace what the caches hold for others.  On an MI355X a
// kernel that only reads streams 6.6 to 7.0 TB/s this way against 5.9 to 6.2 with plain loads.
typedef unsigned int ts_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ ts_u32x4 load_once16(const void* at) {
  return __builtin_nontemporal_load(reinterpret_cast<const ts_u32x4*>(at));
}

static inline int ts_launch_status() { return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH; }
