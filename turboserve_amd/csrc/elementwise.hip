// Row-wise kernels of the decoder: embedding gather, RMSNorm (with the residual sum fused in),
// SwiGLU, and rotary encoding fused with the scatter of keys and values into cache pages.
//
// Formulas restate src/turboserve/engine/model/layers.py:202-208 (RMSNorm), :214-222 and
// :290-302 (rotary, half-split pairs), :437-440 (SwiGLU) and
// src/turboserve/engine/core/kv_cache.py:601-631 (cache write at slot = block * BS + offset).
// Reductions, the residual sum and the rotation are computed in 32-bit whatever T is.
#include <type_traits>

#include "common.hpp"

// ---------------------------------------------------------------------------------------------
// embedding: residual[t, :] = float(table[ids[t], :])
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(float* __restrict__ residual, const T* __restrict__ table,
                             const int* __restrict__ ids, int hidden, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  const bool valid = id >= 0 && id < vocab;
  const T* row = table + (size_t)(valid ? id : 0) * hidden;
  float* out = residual + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    // An id outside the table is a host error; it yields NaN instead of a read out of bounds.
    out[i] = valid ? to_float(row[i]) : __uint_as_float(0x7fc00000u);
  }
}

extern "C" int ts_embed(void* residual, const void* table, const int* ids, int tokens, int hidden,
                        int vocab, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!residual || !table || !ids || hidden < 1 || vocab < 1) return TS_ERR_ARG;
  dim3 grid(tokens), block(256);
  if (dtype == TS_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (float*)residual, (const float*)table, ids, hidden, vocab);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (float*)residual, (const bf16_t*)table, ids, hidden, vocab);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// RMSNorm.  y = w * round_T(x * rsqrt(mean(x^2) + eps)): the normalised value is rounded to the
// storage type before the gain, as the reference does (layers.py:208).
//
// add_rmsnorm: s = residual + pending (32-bit); residual = s; y = norm(s).  With `rows` the
// kernel reads rows[i] and writes y[i] only (residual untouched): the final norm at the wanted
// positions.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void rmsnorm_kernel(T* __restrict__ y, const T* __restrict__ x, const T* __restrict__ w,
                               float eps, int hidden) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_float(x[base + i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float n = round_to<T>(to_float(x[base + i]) * rstd);
    y[base + i] = from_float<T>(to_float(w[i]) * n);
  }
}

// `init` plus the `splits` values that lie `stride` elements apart, added in split order; the loads
// of up to eight splits are in flight together (see add_splits4).
template <typename P>
__device__ __forceinline__ float add_splits(const P* p, int splits, size_t stride, float init) {
  float s = init;
  if (splits == 1) return s + to_float(p[0]);
  int sp0 = 0;
  do {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = to_float(p[(size_t)min(sp0 + j, splits - 1) * stride]);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (sp0 + j < splits) s += v[j];
    sp0 += 8;
  } while (sp0 < splits);
  return s;
}

// P is the type of `pending`: T, or float for `splits` partial sums of a product that are
// `split_stride` elements apart and are added up here.
template <typename T, typename P>
__global__ void add_rmsnorm_kernel(T* __restrict__ y, float* __restrict__ residual,
                                   const P* __restrict__ pending, int splits, size_t split_stride,
                                   const T* __restrict__ w, const int* __restrict__ rows, float eps,
                                   int hidden) {
  __shared__ float scratch[16];
  const int src = rows ? rows[blockIdx.x] : blockIdx.x;
  const size_t in_base = (size_t)src * hidden;
  const size_t out_base = (size_t)blockIdx.x * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float s = residual[in_base + i];
    if (pending) {
      s = add_splits(pending + in_base + i, splits, split_stride, s);
      if (!rows) residual[in_base + i] = s;  // re-read below by this same thread
    }
    ss += s * s;
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float s = residual[in_base + i];
    if (rows && pending) s = add_splits(pending + in_base + i, splits, split_stride, s);
    const float n = round_to<T>(s * rstd);
    y[out_base + i] = from_float<T>(to_float(w[i]) * n);
  }
}

extern "C" int ts_rmsnorm(void* y, const void* x, const void* w, float eps, int tokens, int hidden,
                          int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!y || !x || !w || hidden < 1) return TS_ERR_ARG;
  dim3 grid(tokens), block(hidden <= 1024 ? 256 : 1024);
  if (dtype == TS_F32)
    hipLaunchKernelGGL(rmsnorm_kernel<float>, grid, block, 0, stream, (float*)y, (const float*)x, (const float*)w, eps, hidden);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, (const bf16_t*)x, (const bf16_t*)w, eps, hidden);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// The same, four elements per thread per item and the row kept in registers between the two
// passes: for hidden sizes that are a multiple of 4 and at most 16 * blockDim.x.  A decode step
// has few rows, so each row gets a large block and the loads of all splits are in flight at once.
template <typename T>
struct Vec4Of;
template <>
struct Vec4Of<float> {
  typedef float4 type;
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct Vec4Of<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    uint2 x;
    x.x = (uint32_t)from_float<bf16_t>(v[0]).bits | ((uint32_t)from_float<bf16_t>(v[1]).bits << 16);
    x.y = (uint32_t)from_float<bf16_t>(v[2]).bits | ((uint32_t)from_float<bf16_t>(v[3]).bits << 16);
    *reinterpret_cast<uint2*>(p) = x;
  }
};

// Partial sums of a product lie `stride` elements apart.  The loads of a batch of splits are
// issued together and only then added, in split order: a loop that loads and adds one split at a
// time makes every split wait a full trip to memory, and these kernels are nothing but such
// trips.  Up to 16 splits are one batch in straight-line code (so that the caller's own loads,
// issued before, are waited for only where they are used); more go in batches of 8.  A value
// that is not split (splits == 1) takes the one load.
template <int N, typename P>
__device__ __forceinline__ void add_split_batch4(const P* p, int first, int splits, size_t stride, float (&s)[4]) {
  float v[N][4];
#pragma unroll
  for (int j = 0; j < N; ++j) Vec4Of<P>::load(p + (size_t)min(first + j, splits - 1) * stride, v[j]);
#pragma unroll
  for (int j = 0; j < N; ++j) {
    if (first + j < splits) {
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] += v[j][e];
    }
  }
}

template <typename P>
__device__ __forceinline__ void add_splits4(const P* p, int splits, size_t stride, float (&s)[4]) {
  if (splits == 1) {
    add_split_batch4<1>(p, 0, 1, stride, s);
  } else if (splits <= 4) {
    add_split_batch4<4>(p, 0, splits, stride, s);
  } else if (splits <= 8) {
    add_split_batch4<8>(p, 0, splits, stride, s);
  } else if (splits <= 16) {
    add_split_batch4<16>(p, 0, splits, stride, s);
  } else {
    for (int first = 0; first < splits; first += 8) add_split_batch4<8>(p, first, splits, stride, s);
  }
}

#define NORM_ITEMS 4

template <typename T, typename P>
__global__ void add_rmsnorm_vec4_kernel(T* __restrict__ y, float* __restrict__ residual,
                                        const P* __restrict__ pending, int splits, size_t split_stride,
                                        const T* __restrict__ w, const int* __restrict__ rows, float eps,
                                        int hidden) {
  __shared__ float scratch[16];
  const int src = rows ? rows[blockIdx.x] : blockIdx.x;
  const size_t in_base = (size_t)src * hidden;
  const size_t out_base = (size_t)blockIdx.x * hidden;
  const int quads = hidden / 4;
  float s[NORM_ITEMS][4], g[NORM_ITEMS][4];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NORM_ITEMS; ++it) {
    const int qd = threadIdx.x + it * blockDim.x;
    if (qd < quads) {
      Vec4Of<float>::load(residual + in_base + 4 * qd, s[it]);
      Vec4Of<T>::load(w + 4 * qd, g[it]);  // with the other loads, not behind the reduction's barriers
      if (pending) {
        add_splits4(pending + in_base + 4 * qd, splits, split_stride, s[it]);
        if (!rows) Vec4Of<float>::store(residual + in_base + 4 * qd, s[it]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += s[it][e] * s[it][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int it = 0; it < NORM_ITEMS; ++it) {
    const int qd = threadIdx.x + it * blockDim.x;
    if (qd < quads) {
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = g[it][e] * round_to<T>(s[it][e] * rstd);
      Vec4Of<T>::store(y + out_base + 4 * qd, o);
    }
  }
}

template <typename T, typename P>
static void launch_add_rmsnorm(void* y, float* residual, const void* pending, int splits, long split_stride,
                               const void* w, const int* rows, float eps, int out_rows, int hidden,
                               hipStream_t stream) {
  // Few rows (decode): one large block per row; many rows (prefill): just enough threads.
  int threads = out_rows <= 256 ? 1024 : 256;
  const int need = (hidden / 4 + NORM_ITEMS - 1) / NORM_ITEMS;
  if (threads < need) threads = ((need + 63) / 64) * 64;
  if (hidden % 4 == 0 && threads <= 1024) {
    hipLaunchKernelGGL((add_rmsnorm_vec4_kernel<T, P>), dim3(out_rows), dim3(threads), 0, stream, (T*)y, residual,
                       (const P*)pending, splits, (size_t)split_stride, (const T*)w, rows, eps, hidden);
  } else {
    hipLaunchKernelGGL((add_rmsnorm_kernel<T, P>), dim3(out_rows), dim3(hidden <= 1024 ? 256 : 1024), 0, stream,
                       (T*)y, residual, (const P*)pending, splits, (size_t)split_stride, (const T*)w, rows, eps,
                       hidden);
  }
}

// `out_rows` = rows of y written: the number of entries of `rows` if given, else the tokens.
// pending_f32 != 0: `pending` holds `splits` 32-bit partial sums, `split_stride` elements apart.
extern "C" int ts_add_rmsnorm(void* y, float* residual, const void* pending, int pending_f32, int splits,
                              long split_stride, const void* w, const int* rows, float eps, int out_rows,
                              int hidden, int dtype, hipStream_t stream) {
  if (out_rows == 0) return TS_OK;
  if (!y || !residual || !w || hidden < 1 || splits < 1) return TS_ERR_ARG;
  if (dtype == TS_F32)
    launch_add_rmsnorm<float, float>(y, residual, pending, splits, split_stride, w, rows, eps, out_rows, hidden, stream);
  else if (dtype == TS_BF16 && pending_f32)
    launch_add_rmsnorm<bf16_t, float>(y, residual, pending, splits, split_stride, w, rows, eps, out_rows, hidden, stream);
  else if (dtype == TS_BF16)
    launch_add_rmsnorm<bf16_t, bf16_t>(y, residual, pending, splits, split_stride, w, rows, eps, out_rows, hidden, stream);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// SwiGLU over the fused gate|up projection [T, 2 I]: out[t, i] = silu(gate[t, i]) * up[t, i], with
// gate in the first I columns and up in the last (paired == 0), or alternating: gate i in column
// 2 i, up i in column 2 i + 1 (paired != 0).
// ---------------------------------------------------------------------------------------------
// P: type of the projection output: T, or float for `splits` partial sums to be added up.
template <typename T, typename P>
__global__ void swiglu_kernel(T* __restrict__ out, const P* __restrict__ gate_up, int splits,
                              size_t split_stride, int inter, size_t total, int paired) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / inter;
  const int i = (int)(idx - t * inter);
  const size_t gate_at = t * 2 * inter + (paired ? 2 * i : i);
  const size_t up_at = paired ? gate_at + 1 : gate_at + inter;
  const float g = add_splits(gate_up + gate_at, splits, split_stride, 0.f);
  const float u = add_splits(gate_up + up_at, splits, split_stride, 0.f);
  const float act = g / (1.f + expf(-g));
  out[idx] = from_float<T>(act * u);
}

// Four outputs per thread with 8- or 16-byte loads: for I a multiple of 4.
template <typename T, typename P>
__global__ void swiglu_vec4_kernel(T* __restrict__ out, const P* __restrict__ gate_up, int splits,
                                   size_t split_stride, int inter, size_t quads, int paired) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= quads) return;
  const int per_row = inter / 4;
  const size_t t = idx / per_row;
  const int i = (int)(idx - t * per_row) * 4;
  float g[4], u[4];
  float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
  if (paired) {  // eight consecutive columns: g0 u0 g1 u1 | g2 u2 g3 u3
    add_splits4(gate_up + t * 2 * inter + 2 * i, splits, split_stride, a);
    add_splits4(gate_up + t * 2 * inter + 2 * i + 4, splits, split_stride, b);
    g[0] = a[0]; u[0] = a[1]; g[1] = a[2]; u[1] = a[3];
    g[2] = b[0]; u[2] = b[1]; g[3] = b[2]; u[3] = b[3];
  } else {
    add_splits4(gate_up + t * 2 * inter + i, splits, split_stride, a);
    add_splits4(gate_up + t * 2 * inter + inter + i, splits, split_stride, b);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      g[e] = a[e];
      u[e] = b[e];
    }
  }
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = g[e] / (1.f + expf(-g[e])) * u[e];
  Vec4Of<T>::store(out + t * inter + i, o);
}

// Eight outputs per thread with 16-byte loads and stores: bfloat16 in and out, one split, I a
// multiple of 8 (the many-row case: a product of the library's, then this).  The same arithmetic
// per element as above.
__global__ void swiglu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gate_up, int inter,
                                     size_t octets, int paired) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= octets) return;
  const int per_row = inter / 8;
  const size_t t = idx / per_row;
  const int i = (int)(idx - t * per_row) * 8;
  const bf16_t* row = gate_up + t * 2 * inter;
  // paired: sixteen consecutive columns g0 u0 .. g7 u7; else eight of the gate and eight of the up half
  const uint4 a = *reinterpret_cast<const uint4*>(paired ? row + 2 * i : row + i);
  const uint4 b = *reinterpret_cast<const uint4*>(paired ? row + 2 * i + 8 : row + inter + i);
  const uint32_t wa[4] = {a.x, a.y, a.z, a.w}, wb[4] = {b.x, b.y, b.z, b.w};
  float g[8], u[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float a_lo = __uint_as_float(wa[e] << 16), a_hi = __uint_as_float(wa[e] & 0xffff0000u);
    const float b_lo = __uint_as_float(wb[e] << 16), b_hi = __uint_as_float(wb[e] & 0xffff0000u);
    if (paired) {
      g[e] = a_lo; u[e] = a_hi; g[4 + e] = b_lo; u[4 + e] = b_hi;
    } else {
      g[2 * e] = a_lo; g[2 * e + 1] = a_hi; u[2 * e] = b_lo; u[2 * e + 1] = b_hi;
    }
  }
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = g[e] / (1.f + expf(-g[e])) * u[e];
  uint32_t w[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    w[e] = (uint32_t)from_float<bf16_t>(o[2 * e]).bits | ((uint32_t)from_float<bf16_t>(o[2 * e + 1]).bits << 16);
  *reinterpret_cast<uint4*>(out + t * inter + i) = make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename T, typename P>
static void launch_swiglu(void* out, const void* gate_up, int splits, long split_stride, int tokens, int inter,
                          int paired, hipStream_t stream) {
  if (std::is_same<T, bf16_t>::value && std::is_same<P, bf16_t>::value && splits == 1 && inter % 8 == 0) {
    const size_t octets = (size_t)tokens * (inter / 8);
    hipLaunchKernelGGL(swiglu_bf16x8_kernel, dim3((unsigned)((octets + 255) / 256)), dim3(256), 0, stream,
                       (bf16_t*)out, (const bf16_t*)gate_up, inter, octets, paired);
  } else if (inter % 4 == 0) {
    const size_t quads = (size_t)tokens * (inter / 4);
    hipLaunchKernelGGL((swiglu_vec4_kernel<T, P>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream,
                       (T*)out, (const P*)gate_up, splits, (size_t)split_stride, inter, quads, paired);
  } else {
    const size_t total = (size_t)tokens * inter;
    hipLaunchKernelGGL((swiglu_kernel<T, P>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (T*)out,
                       (const P*)gate_up, splits, (size_t)split_stride, inter, total, paired);
  }
}

extern "C" int ts_swiglu(void* out, const void* gate_up, int in_f32, int splits, long split_stride,
                         int tokens, int inter, int paired, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !gate_up || inter < 1 || splits < 1) return TS_ERR_ARG;
  if (dtype == TS_F32)
    launch_swiglu<float, float>(out, gate_up, splits, split_stride, tokens, inter, paired, stream);
  else if (dtype == TS_BF16 && in_f32)
    launch_swiglu<bf16_t, float>(out, gate_up, splits, split_stride, tokens, inter, paired, stream);
  else if (dtype == TS_BF16)
    launch_swiglu<bf16_t, bf16_t>(out, gate_up, splits, split_stride, tokens, inter, paired, stream);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Rotary encoding + cache write.  The projection output is [T, (Hq + 2 Hkv) * D]: q heads, then
// k heads, then v heads; it is either of type T, or `splits` 32-bit partial sums that are added
// up here.  One block per (token, head).  q and k are rotated by the angles of the token's
// position (cos/sin tables are 32-bit, [capacity, D/2]; pair (i, i + D/2)); the rotated q goes
// to q_out (rows q_stride apart; with a projection of type T this may be the projection itself:
// rotation in place); k (rotated) and v go to the pages at slot = block * BS + offset.  Key
// pages are [NB, Hkv, BS, D]; value pages are transposed, [NB, Hkv, D, BS], so that the
// attention kernels read eight consecutive keys' values of one head dimension with a single
// 16-byte load.  rotate == 0 skips the rotation (a position encoding that only stores).
// slots == nullptr or a negative slot: nothing is stored for that token.
// ---------------------------------------------------------------------------------------------
// One rotation, written out so that every kernel rounds it the same way.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float& o1, float& o2) {
  o1 = __builtin_fmaf(x1, c, -(x2 * s));
  o2 = __builtin_fmaf(x2, c, x1 * s);
}

template <typename T, typename P>
__global__ void rope_store_kernel(T* q_out, long q_stride, const P* proj, int splits,
                                  size_t split_stride, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                  const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                  const int* __restrict__ positions, const int* __restrict__ slots,
                                  int heads, int kv_heads, int dim, int block_size, int rotate) {
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int half = dim / 2;
  const int width = (heads + 2 * kv_heads) * dim;
  const P* row = proj + (size_t)t * width + (size_t)h * dim;
  const int pos = positions[t];
  const int slot = slots ? slots[t] : -1;
  T* page = nullptr;   // this token's row of a key page
  T* vpage = nullptr;  // this token's column of a value page (elements block_size apart)
  if (h >= heads && slot >= 0) {
    const int kvh = (h - heads) % kv_heads;
    const size_t blk = (size_t)(slot / block_size);
    const int off = slot % block_size;
    const size_t head_base = (blk * kv_heads + kvh) * (size_t)block_size * dim;
    if (h < heads + kv_heads)
      page = k_pages + head_base + (size_t)off * dim;
    else
      vpage = v_pages + head_base + off;
  }
  T* qrow = (h < heads) ? q_out + (size_t)t * q_stride + (size_t)h * dim : nullptr;
  if (h < heads + kv_heads) {
    const float* c = cos_table + (size_t)pos * half;
    const float* s = sin_table + (size_t)pos * half;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      float x1 = add_splits(row + i, splits, split_stride, 0.f);
      float x2 = add_splits(row + i + half, splits, split_stride, 0.f);
      float r1 = x1, r2 = x2;
      if (rotate) rotate_pair(x1, x2, c[i], s[i], r1, r2);
      const T o1 = from_float<T>(r1);
      const T o2 = from_float<T>(r2);
      if (qrow) {
        qrow[i] = o1;
        qrow[i + half] = o2;
      }
      if (page) {
        page[i] = o1;
        page[i + half] = o2;
      }
    }
  } else if (vpage) {
    for (int i = threadIdx.x; i < dim; i += blockDim.x) {
      const float x = add_splits(row + i, splits, split_stride, 0.f);
      vpage[(size_t)i * block_size] = from_float<T>(x);
    }
  }
}

// The same for many tokens at once (prompt portions): bfloat16 in and out, no partial sums, head
// size a multiple of 16.  One block per (group of 8 consecutive tokens, head).  q and k heads: a
// thread rotates 8 pairs with 16-byte loads and stores.  v heads: a thread collects one head
// dimension of the 8 tokens; when the group's slots are 8 consecutive ones starting at a multiple
// of 8 (the usual case inside a prompt: they lie in one page, block_size being a multiple of 8)
// that is one 16-byte store into the transposed value page, else one 2-byte store per token.
constexpr int ROPE_GROUP = 8;

__global__ void __launch_bounds__(64)
rope_store_group_kernel(bf16_t* q_out, long q_stride, const bf16_t* proj, bf16_t* __restrict__ k_pages,
                        bf16_t* __restrict__ v_pages, const float* __restrict__ cos_table,
                        const float* __restrict__ sin_table, const int* __restrict__ positions,
                        const int* __restrict__ slots, int tokens, int heads, int kv_heads, int dim,
                        int block_size, int rotate) {
  typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  const int t0 = blockIdx.x * ROPE_GROUP;
  const int h = blockIdx.y;
  const int half = dim / 2;
  const int width = (heads + 2 * kv_heads) * dim;
  const int count = min(ROPE_GROUP, tokens - t0);
  if (h < heads + kv_heads) {
    const bool is_key = h >= heads;
    const int kvh = h - heads;
    const int vectors = half / 8;  // 16-byte pieces of a half row
    for (int item = threadIdx.x; item < ROPE_GROUP * vectors; item += blockDim.x) {
      const int j = item / vectors, i = (item % vectors) * 8;
      if (j >= count) continue;
      const int t = t0 + j;
      const bf16_t* row = proj + (size_t)t * width + (size_t)h * dim;
      const u16x8 a = *reinterpret_cast<const u16x8*>(row + i);
      const u16x8 b = *reinterpret_cast<const u16x8*>(row + i + half);
      u16x8 o1 = a, o2 = b;
      if (rotate) {
        const float* c = cos_table + (size_t)positions[t] * half + i;
        const float* s = sin_table + (size_t)positions[t] * half + i;
        const f32x4v c0 = *reinterpret_cast<const f32x4v*>(c), c1 = *reinterpret_cast<const f32x4v*>(c + 4);
        const f32x4v s0 = *reinterpret_cast<const f32x4v*>(s), s1 = *reinterpret_cast<const f32x4v*>(s + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float cv = e < 4 ? c0[e & 3] : c1[e & 3], sv = e < 4 ? s0[e & 3] : s1[e & 3];
          float r1, r2;
          rotate_pair(to_float(bf16_t{a[e]}), to_float(bf16_t{b[e]}), cv, sv, r1, r2);
          o1[e] = from_float<bf16_t>(r1).bits;
          o2[e] = from_float<bf16_t>(r2).bits;
        }
      }
      if (!is_key) {
        bf16_t* qrow = q_out + (size_t)t * q_stride + (size_t)h * dim;
        *reinterpret_cast<u16x8*>(qrow + i) = o1;
        *reinterpret_cast<u16x8*>(qrow + i + half) = o2;
      } else {
        const int slot = slots ? slots[t] : -1;
        if (slot < 0) continue;
        bf16_t* page = k_pages + (((size_t)(slot / block_size) * kv_heads + kvh) * block_size + slot % block_size) * dim;
        *reinterpret_cast<u16x8*>(page + i) = o1;
        *reinterpret_cast<u16x8*>(page + i + half) = o2;
      }
    }
    return;
  }
  if (!slots) return;
  const int kvh = h - heads - kv_heads;
  int slot[ROPE_GROUP];
#pragma unroll
  for (int j = 0; j < ROPE_GROUP; ++j) slot[j] = j < count ? slots[t0 + j] : -1;
  bool run = count == ROPE_GROUP && slot[0] >= 0 && (slot[0] & 7) == 0 && (block_size & 7) == 0;
#pragma unroll
  for (int j = 1; j < ROPE_GROUP; ++j) run = run && slot[j] == slot[0] + j;
  const bf16_t* column = proj + (size_t)t0 * width + (size_t)h * dim;
  for (int d = threadIdx.x; d < dim; d += blockDim.x) {
    u16x8 v;
#pragma unroll
    for (int j = 0; j < ROPE_GROUP; ++j) v[j] = j < count ? column[(size_t)j * width + d].bits : (uint16_t)0;
    if (run) {
      bf16_t* dst = v_pages + (((size_t)(slot[0] / block_size) * kv_heads + kvh) * dim + d) * block_size + slot[0] % block_size;
      *reinterpret_cast<u16x8*>(dst) = v;
    } else {
#pragma unroll
      for (int j = 0; j < ROPE_GROUP; ++j) {
        if (slot[j] < 0) continue;
        v_pages[(((size_t)(slot[j] / block_size) * kv_heads + kvh) * dim + d) * block_size + slot[j] % block_size] = bf16_t{v[j]};
      }
    }
  }
}

extern "C" int ts_rope_store(void* q_out, long q_stride, const void* proj, int in_f32, int splits,
                             long split_stride, void* k_pages, void* v_pages, const float* cos_table,
                             const float* sin_table, const int* positions, const int* slots, int tokens,
                             int heads, int kv_heads, int dim, int block_size, int rotate, int dtype,
                             hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!q_out || !proj || !positions || heads < 1 || kv_heads < 1 || dim < 2 || (dim & 1) || block_size < 1 ||
      splits < 1)
    return TS_ERR_ARG;
  if (rotate && (!cos_table || !sin_table)) return TS_ERR_ARG;
  if (slots && (!k_pages || !v_pages)) return TS_ERR_ARG;
  dim3 grid(tokens, heads + 2 * kv_heads), block(64);
  const bool aligned = ((uintptr_t)q_out | (uintptr_t)proj | (uintptr_t)k_pages | (uintptr_t)v_pages |
                        (uintptr_t)cos_table | (uintptr_t)sin_table) % 16 == 0 && q_stride % 8 == 0;
  if (dtype == TS_BF16 && !in_f32 && splits == 1 && dim % 16 == 0 && tokens >= 4 * ROPE_GROUP && aligned) {
    dim3 groups((tokens + ROPE_GROUP - 1) / ROPE_GROUP, heads + 2 * kv_heads);
    hipLaunchKernelGGL(rope_store_group_kernel, groups, block, 0, stream, (bf16_t*)q_out, q_stride, (const bf16_t*)proj, (bf16_t*)k_pages, (bf16_t*)v_pages, cos_table, sin_table, positions, slots, tokens, heads, kv_heads, dim, block_size, rotate);
    return ts_launch_status();
  }
  if (dtype == TS_F32)
    hipLaunchKernelGGL((rope_store_kernel<float, float>), grid, block, 0, stream, (float*)q_out, q_stride, (const float*)proj, splits, (size_t)split_stride, (float*)k_pages, (float*)v_pages, cos_table, sin_table, positions, slots, heads, kv_heads, dim, block_size, rotate);
  else if (dtype == TS_BF16 && in_f32)
    hipLaunchKernelGGL((rope_store_kernel<bf16_t, float>), grid, block, 0, stream, (bf16_t*)q_out, q_stride, (const float*)proj, splits, (size_t)split_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, cos_table, sin_table, positions, slots, heads, kv_heads, dim, block_size, rotate);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL((rope_store_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (bf16_t*)q_out, q_stride, (const bf16_t*)proj, splits, (size_t)split_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, cos_table, sin_table, positions, slots, heads, kv_heads, dim, block_size, rotate);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// gather rows: out[i, :] = x[rows[i], :]
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ x,
                                   const int* __restrict__ rows, int width) {
  const size_t src = (size_t)rows[blockIdx.x] * width;
  const size_t dst = (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[dst + i] = x[src + i];
}

extern "C" int ts_gather_rows(void* out, const void* x, const int* rows, int n, int width,
                              int dtype, hipStream_t stream) {
  if (n == 0) return TS_OK;
  if (!out || !x || !rows || width < 1) return TS_ERR_ARG;
  dim3 grid(n), block(256);
  if (dtype == TS_F32)
    hipLaunchKernelGGL(gather_rows_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)x, rows, width);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(gather_rows_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const bf16_t*)x, rows, width);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// patch_tokens: token_ids[i] = source[patch[i]] where patch[i] >= 0 (else left as it is).  A step
// that is launched before the host has read the tokens the step before sampled takes them from
// the sampler's device buffer this way.  patch[i] must be below `sources`; a value at or beyond
// it is ignored (nothing is read out of bounds).
// ---------------------------------------------------------------------------------------------
__global__ void patch_tokens_kernel(int* __restrict__ token_ids, const int* __restrict__ patch,
                                    const int* __restrict__ source, int n, int sources) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int from = patch[i];
  if (from >= 0 && from < sources) token_ids[i] = source[from];
}

extern "C" int ts_patch_tokens(int* token_ids, const int* patch, const int* source, int n, int sources,
                               hipStream_t stream) {
  if (n == 0) return TS_OK;
  if (!token_ids || !patch || !source || n < 0 || sources < 1) return TS_ERR_ARG;
  hipLaunchKernelGGL(patch_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, token_ids, patch, source, n,
                     sources);
  return ts_launch_status();
}
