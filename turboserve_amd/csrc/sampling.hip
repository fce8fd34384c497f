// Token sampling on the device: one block per row of 32-bit logits.
//
// Stages and their order follow src/turboserve/engine/core/sampler.py:216-238: repetition
// penalty (:83-122), log-probability snapshot, temperature (:125-135), top-k (:138-148),
// top-p (:151-168), then argmax for greedy rows (temperature 0; truncation ignored) or a draw.
// The draw is this engine's own rule, because a kernel cannot follow torch.multinomial's
// stream (sampler.py:285-296): u = Philox-4x32-10(key = seed, counter = draw index) in [0, 1),
// and the token is the first one, in vocabulary order, whose cumulative probability exceeds u.
// top-k and top-p are applied as value thresholds found by bisection over the ordered bit
// patterns of the logits, so equal logits are kept or dropped together.
#include "common.hpp"
#include "ts_no_alloc.h"

#include <mutex>

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t ordered_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const int waves = blockDim.x / TS_WAVE;
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TS_WAVE);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  int total = 0;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float philox_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t index) {
  uint32_t c0 = index, c1 = 0u, c2 = 0u, c3 = 0u;
  uint32_t k0 = seed_lo, k1 = seed_hi;
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0;
    const uint32_t n2 = hi0 ^ c3 ^ k1;
    c0 = n0;
    c1 = lo1;
    c2 = n2;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return (float)(c0 >> 8) * (1.0f / 16777216.0f);
}

// Lowest index among the largest values of a row.
__device__ __forceinline__ int block_argmax(const float* __restrict__ row, int vocab, float* fscratch,
                                            int* iscratch) {
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    if (best_i == 0x7fffffff || v > best) {  // i only grows, so the first of equal values stays
      best = v;
      best_i = i;
    }
  }
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, TS_WAVE);
    const int oi = __shfl_xor(best_i, off, TS_WAVE);
    if (oi != 0x7fffffff && (best_i == 0x7fffffff || ov > best || (ov == best && oi < best_i))) {
      best = ov;
      best_i = oi;
    }
  }
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const int waves = blockDim.x / TS_WAVE;
  __syncthreads();
  if (lane == 0) {
    fscratch[wave] = best;
    iscratch[wave] = best_i;
  }
  __syncthreads();
  best = fscratch[0];
  best_i = iscratch[0];
  for (int w = 1; w < waves; ++w) {
    const float ov = fscratch[w];
    const int oi = iscratch[w];
    if (oi != 0x7fffffff && (best_i == 0x7fffffff || ov > best || (ov == best && oi < best_i))) {
      best = ov;
      best_i = oi;
    }
  }
  __syncthreads();
  return best_i == 0x7fffffff ? 0 : best_i;
}

// Greedy rows in two stages, so that a handful of rows still spreads over the device: stage one
// finds the best (value, lowest index) of each slice of the vocabulary, stage two of each row.
#define ARGMAX_SLICES 64
#define ARGMAX_THREADS 256

__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_slices_kernel(float* __restrict__ slice_value, int* __restrict__ slice_index,
                     const float* __restrict__ logits, int vocab) {
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  const int row = blockIdx.y;
  const int per = (vocab + ARGMAX_SLICES - 1) / ARGMAX_SLICES;
  const int begin = blockIdx.x * per;
  const int count = min(per, vocab - begin);
  float best_value = -INFINITY;
  int best = 0x7fffffff;
  if (count > 0) {
    const int local = block_argmax(logits + (size_t)row * vocab + begin, count, fscratch, iscratch);
    best = begin + local;
    best_value = logits[(size_t)row * vocab + best];
  }
  if (threadIdx.x == 0) {
    slice_value[row * ARGMAX_SLICES + blockIdx.x] = best_value;
    slice_index[row * ARGMAX_SLICES + blockIdx.x] = best;
  }
}

__global__ void __launch_bounds__(ARGMAX_SLICES)
argmax_rows_kernel(int* __restrict__ tokens, const float* __restrict__ slice_value,
                   const int* __restrict__ slice_index) {
  const int row = blockIdx.x;
  float v = slice_value[row * ARGMAX_SLICES + threadIdx.x];
  int i = slice_index[row * ARGMAX_SLICES + threadIdx.x];
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, TS_WAVE);
    const int oi = __shfl_xor(i, off, TS_WAVE);
    if (oi != 0x7fffffff && (i == 0x7fffffff || ov > v || (ov == v && oi < i))) {
      v = ov;
      i = oi;
    }
  }
  if (threadIdx.x == 0) tokens[row] = (i == 0x7fffffff) ? 0 : i;
}

// scratch: rows * 64 floats followed by rows * 64 ints.
extern "C" int ts_argmax(int* tokens, const float* logits, void* scratch, int rows, int vocab, hipStream_t stream) {
  if (rows == 0) return TS_OK;
  if (!tokens || !logits || !scratch || vocab < 1 || rows > 65535) return TS_ERR_ARG;
  float* values = (float*)scratch;
  int* indices = (int*)(values + (size_t)rows * ARGMAX_SLICES);
  hipLaunchKernelGGL(argmax_slices_kernel, dim3(ARGMAX_SLICES, rows), dim3(ARGMAX_THREADS), 0, stream, values,
                     indices, logits, vocab);
  if (hipGetLastError() != hipSuccess) return TS_ERR_LAUNCH;
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(ARGMAX_SLICES), 0, stream, tokens, values, indices);
  return ts_launch_status();
}

// The same two stages with the partial results in an array of the library's own, for callers
// that cannot allocate (see ts_no_alloc.h).  Host code never passes the array's name to a
// kernel: its device address is looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[(size_t)TS_ARGMAX_STATIC_MAX_ROWS * ARGMAX_SLICES * 8];

#define TS_MAX_DEVICES 64
static void* scratch_address[TS_MAX_DEVICES];  // per device; null until looked up
static std::mutex scratch_mutex;

// The address of `scratch` on the current device, or null if it cannot be found.
static void* scratch_on_current_device() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= TS_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> guard(scratch_mutex);
  if (scratch_address[device] == nullptr) {
    void* address = nullptr;
    if (hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    scratch_address[device] = address;
  }
  return scratch_address[device];
}

extern "C" int ts_argmax_static(int* tokens, const float* logits, int rows, int vocab, hipStream_t stream) {
  if (rows == 0) return TS_OK;
  if (!tokens || !logits || vocab < 1 || rows < 0) return TS_ERR_ARG;
  if (rows > TS_ARGMAX_STATIC_MAX_ROWS) return TS_ERR_SHAPE;
  void* address = scratch_on_current_device();
  if (address == nullptr) return TS_ERR_LAUNCH;
  // Every element the second kernel reads (rows x 64 values, rows x 64 indices) is written by the
  // first in this call: what an earlier call left in the array does not matter.
  return ts_argmax(tokens, logits, address, rows, vocab, stream);
}

// Per-row parameters, all device arrays of `rows` entries:
//   temperature (0 = greedy), top_k (0 = off), top_p (1 = off), penalty (1 = off),
//   seed_lo / seed_hi / draw_index (Philox key and counter).
// history tokens of row r: history[history_start[r] .. history_start[r + 1]).
// work [rows, vocab]: scratch for the penalised logits.  logprobs may be null.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(int* __restrict__ tokens, float* __restrict__ logprobs,
              const float* __restrict__ logits, float* __restrict__ work, int vocab,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ penalty,
              const uint32_t* __restrict__ seed_lo, const uint32_t* __restrict__ seed_hi,
              const uint32_t* __restrict__ draw_index, const int* __restrict__ history,
              const int* __restrict__ history_start) {
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  __shared__ float partial[SAMPLE_THREADS];
  __shared__ int chosen;

  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const float* src = logits + (size_t)r * vocab;
  float* row = work + (size_t)r * vocab;
  const float temp = temperature[r];
  const float pen = penalty[r];

  // 1. penalised copy.  Reading the untouched logits makes a repeated history token harmless.
  for (int i = tid; i < vocab; i += blockDim.x) row[i] = src[i];
  __syncthreads();
  if (pen != 1.0f) {
    const int h0 = history_start[r], h1 = history_start[r + 1];
    for (int j = h0 + tid; j < h1; j += blockDim.x) {
      const int tok = history[j];
      if (tok >= 0 && tok < vocab) {
        const float v = src[tok];
        row[tok] = v < 0.f ? v * pen : v / pen;
      }
    }
    __syncthreads();
  }

  // 2. log-softmax terms of the penalised logits (before temperature).
  float base_max = 0.f, base_lse = 0.f;
  if (logprobs) {
    float m = -INFINITY;
    for (int i = tid; i < vocab; i += blockDim.x) m = fmaxf(m, row[i]);
    base_max = block_max(m, fscratch);
    float s = 0.f;
    for (int i = tid; i < vocab; i += blockDim.x) s += expf(row[i] - base_max);
    base_lse = logf(block_sum(s, fscratch));
  }

  int token;
  if (temp <= 0.f) {
    token = block_argmax(row, vocab, fscratch, iscratch);
  } else {
    const float inv_temp = 1.0f / temp;
    // 3. top-k: the k-th largest key, by bisection on the bit pattern.
    uint32_t threshold = 0u;
    const int k = top_k[r];
    if (k > 0 && k < vocab) {
      uint32_t t = 0u;
      for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = t | (1u << bit);
        int count = 0;
        for (int i = tid; i < vocab; i += blockDim.x) count += ordered_key(row[i]) >= cand;
        if (block_sum_int(count, iscratch) >= k) t = cand;
      }
      threshold = t;
    }
    // Softmax terms of the scaled logits over what top-k kept.
    float m = -INFINITY;
    for (int i = tid; i < vocab; i += blockDim.x)
      if (ordered_key(row[i]) >= threshold) m = fmaxf(m, row[i]);
    m = block_max(m, fscratch);
    // 4. top-p: keep a token while the mass strictly above it is <= p.
    const float p = top_p[r];
    if (p < 1.0f) {
      float z = 0.f;
      for (int i = tid; i < vocab; i += blockDim.x)
        if (ordered_key(row[i]) >= threshold) z += expf((row[i] - m) * inv_temp);
      z = block_sum(z, fscratch);
      const float limit = p * z;
      uint32_t t = 0u;  // the largest key whose mass above still exceeds the limit
      for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = t | (1u << bit);
        float above = 0.f;
        for (int i = tid; i < vocab; i += blockDim.x) {
          const uint32_t key = ordered_key(row[i]);
          if (key > cand && key >= threshold) above += expf((row[i] - m) * inv_temp);
        }
        if (block_sum(above, fscratch) > limit) t = cand;
      }
      if (t + 1u > threshold) threshold = t + 1u;
    }
    // 5. draw: contiguous chunks per thread, scan of the chunk sums, walk inside one chunk.
    const int chunk = (vocab + blockDim.x - 1) / blockDim.x;
    const int c0 = tid * chunk;
    const int c1 = (c0 + chunk < vocab) ? c0 + chunk : vocab;
    float local = 0.f;
    for (int i = c0; i < c1; ++i)
      if (ordered_key(row[i]) >= threshold) local += expf((row[i] - m) * inv_temp);
    partial[tid] = local;
    if (tid == 0) chosen = -1;
    __syncthreads();
    if (tid == 0) {
      float running = 0.f;
      for (int i = 0; i < (int)blockDim.x; ++i) {
        const float v = partial[i];
        partial[i] = running;  // exclusive prefix
        running += v;
      }
      fscratch[0] = running;
    }
    __syncthreads();
    const float total = fscratch[0];
    const float u = philox_uniform(seed_lo[r], seed_hi[r], draw_index[r]);
    float target = u * total;
    const float below_total = __uint_as_float(__float_as_uint(total) - 1u);
    if (target > below_total) target = below_total;
    const float prefix = partial[tid];
    if (local > 0.f && prefix <= target && target < prefix + local) {
      // Same order of additions as `local`, so prefix + inner ends at prefix + local > target.
      float inner = 0.f;
      int pick = -1;
      for (int i = c0; i < c1; ++i) {
        if (ordered_key(row[i]) >= threshold) {
          inner += expf((row[i] - m) * inv_temp);
          pick = i;
          if (prefix + inner > target) break;
        }
      }
      chosen = pick;
    }
    __syncthreads();
    token = chosen;
    if (token < 0) token = block_argmax(row, vocab, fscratch, iscratch);  // degenerate row (NaN)
  }
  if (tid == 0) {
    tokens[r] = token;
    if (logprobs) logprobs[r] = (row[token] - base_max) - base_lse;
  }
}

extern "C" int ts_sample(int* tokens, float* logprobs, const float* logits, float* work, int rows,
                         int vocab, const float* temperature, const int* top_k, const float* top_p,
                         const float* penalty, const uint32_t* seed_lo, const uint32_t* seed_hi,
                         const uint32_t* draw_index, const int* history, const int* history_start,
                         hipStream_t stream) {
  if (rows == 0) return TS_OK;
  if (!tokens || !logits || !work || vocab < 1 || !temperature || !top_k || !top_p || !penalty ||
      !seed_lo || !seed_hi || !draw_index || !history_start)
    return TS_ERR_ARG;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, tokens, logprobs,
                     logits, work, vocab, temperature, top_k, top_p, penalty, seed_lo, seed_hi,
                     draw_index, history, history_start);
  return ts_launch_status();
}
