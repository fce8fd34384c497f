// Token sampling on the device: one block per row of 32-bit logits.
//
// Stages and their order follow src/turboserve/engine/core/sampler.py:216-238: repetition
// penalty (:83-122), log-probability snapshot, temperature (:125-135), top-k (:138-148),
// top-p (:151-168), then argmax for greedy rows (temperature 0; truncation ignored) or a draw.
// The draw is this engine's own rule, because a kernel cannot follow torch.multinomial's
// stream (sampler.py:285-296): u = Philox-4x32-10(key = seed, counter = draw index) in [0, 1),
// and the token is the first one, in vocabulary order, whose cumulative probability exceeds u.
// top-k and top-p are applied as value thresholds on the ordered bit patterns of the logits (the
// k-th largest pattern; the largest pattern whose mass strictly above exceeds p), so equal logits
// are kept or dropped together.
#include "common.hpp"
#include "ts_no_alloc.h"

#include <mutex>

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t ordered_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// The logit whose ordered key is `key`.
__device__ __forceinline__ float key_value(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
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

// f(index, value) for every element of the row, each thread of the block taking every
// blockDim-th group of four (or every blockDim-th element where the row is not 16-byte aligned).
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ row, int vocab, F f) {
  const int tid = threadIdx.x;
  const int step = blockDim.x;
  if ((reinterpret_cast<uintptr_t>(row) & 15u) == 0) {
    const float4* quads = reinterpret_cast<const float4*>(row);
    const int count = vocab >> 2;
    int i = tid;
    for (; i + 3 * step < count; i += 4 * step) {
      const float4 a = quads[i], b = quads[i + step], c = quads[i + 2 * step], d = quads[i + 3 * step];
      f(4 * i, a.x); f(4 * i + 1, a.y); f(4 * i + 2, a.z); f(4 * i + 3, a.w);
      f(4 * (i + step), b.x); f(4 * (i + step) + 1, b.y); f(4 * (i + step) + 2, b.z); f(4 * (i + step) + 3, b.w);
      f(4 * (i + 2 * step), c.x); f(4 * (i + 2 * step) + 1, c.y); f(4 * (i + 2 * step) + 2, c.z);
      f(4 * (i + 2 * step) + 3, c.w);
      f(4 * (i + 3 * step), d.x); f(4 * (i + 3 * step) + 1, d.y); f(4 * (i + 3 * step) + 2, d.z);
      f(4 * (i + 3 * step) + 3, d.w);
    }
    for (; i < count; i += step) {
      const float4 a = quads[i];
      f(4 * i, a.x); f(4 * i + 1, a.y); f(4 * i + 2, a.z); f(4 * i + 3, a.w);
    }
    for (int j = 4 * count + tid; j < vocab; j += step) f(j, row[j]);
  } else {
    int i = tid;
    for (; i + 3 * step < vocab; i += 4 * step) {
      const float a = row[i], b = row[i + step], c = row[i + 2 * step], d = row[i + 3 * step];
      f(i, a); f(i + step, b); f(i + 2 * step, c); f(i + 3 * step, d);
    }
    for (; i < vocab; i += step) f(i, row[i]);
  }
}

// Lowest index among the largest values of a row.
__device__ __forceinline__ int block_argmax(const float* __restrict__ row, int vocab, float* fscratch,
                                            int* iscratch) {
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for_each_logit(row, vocab, [&](int i, float v) {  // indices come in no particular order
    if (best_i == 0x7fffffff || v > best || (v == best && i < best_i)) {
      best = v;
      best_i = i;
    }
  });
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

// ---------------------------------------------------------------------------------------------
// The sampling kernel proper.  One workgroup works through a row of a large vocabulary, so every
// walk over the row matters: rows are visited with 16-byte loads, several in flight per thread;
// the two truncations pick their thresholds eight bits at a time from histograms in LDS, over
// a list of the row's likely tokens where a truncation leaves few (four light walks over the
// row), else over the row itself (four walks per truncation); the draw scans partial sums in
// parallel.  Everything is a function of the row alone and is added up in a fixed order
// (histograms hold integers), so a row's token does not depend on its neighbours or on the run.
// ---------------------------------------------------------------------------------------------
#define SAMPLE_WAVES (SAMPLE_THREADS / TS_WAVE)
#define MASS_COPIES 4  // histograms of mass per workgroup (wavefront w adds to copy w % 4)
#define SAMPLE_CANDIDATES 2048  // most tokens the truncations may leave for the short way through the kernel
// Probability mass as an integer: exp((x - max) / T) <= 1 in units of 2^-32.  Sums of a whole
// vocabulary stay far below 2^64, integer sums do not depend on their order, and a token whose
// mass is below 2^-33 of the likeliest one's counts as none.
__device__ __forceinline__ unsigned long long mass_units(float x, float m, float inv_temp) {
  return (unsigned long long)(expf((x - m) * inv_temp) * 4294967296.0f);
}

// A token's mass in the draw, e^x for x <= 0: the hardware's exponential (a few units in the last
// place off, which moves a token's probability by a millionth of itself).  Every walk of a draw
// uses this one function, so the sums a walk retraces come out the same.  (The thresholds' integer
// masses above take the exact one: whether a token is kept must not hang on that millionth.)
__device__ __forceinline__ float draw_mass(float x) { return __expf(x); }

__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* scratch) {
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TS_WAVE);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  unsigned long long total = 0;
  for (int w = 0; w < SAMPLE_WAVES; ++w) total += scratch[w];
  return total;
}

// The sum of `value` over the threads of higher index among the block's first `threads` threads
// (a multiple of 64); called by every thread of the block.  scratch: a place per wavefront.
__device__ __forceinline__ unsigned long long sum_above(unsigned long long value, int threads,
                                                        unsigned long long* scratch) {
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const unsigned long long own = (int)threadIdx.x < threads ? value : 0ull;
  unsigned long long v = own;  // becomes own + the lanes above
#pragma unroll
  for (int off = 1; off < TS_WAVE; off <<= 1) {
    const unsigned long long other = __shfl_down(v, off, TS_WAVE);
    if (lane + off < TS_WAVE) v += other;
  }
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  unsigned long long higher = 0ull;
  for (int w = wave + 1; w < threads / TS_WAVE; ++w) higher += scratch[w];
  return v - own + higher;
}

// What a walk down from digit 255 finds, all digits looked at at once (a single thread's walk
// over 256 places in LDS costs 14 us, and a row needs eight).  bins[d]: keys with digit d.  The
// digit at which the keys counted from the top reach `wanted` goes to picked[0] (0 if they never
// do), and how many of that digit's keys are still wanted to picked[1].
__device__ __forceinline__ void pick_digit_by_count(const unsigned int* bins, unsigned int wanted, unsigned int* picked,
                                                    unsigned long long* scratch) {
  const int tid = threadIdx.x;
  const unsigned int mine = tid < 256 ? bins[tid] : 0u;
  const unsigned int above = (unsigned int)sum_above(mine, 256, scratch);
  if (tid == 0) {
    picked[0] = 0u;
    picked[1] = wanted - above;
  }
  __syncthreads();
  if (tid > 0 && tid < 256 && above < wanted && above + mine >= wanted) {  // one thread at most
    picked[0] = (unsigned int)tid;
    picked[1] = wanted - above;
  }
  __syncthreads();
}

// Likewise for top-p.  total[d], exact[d]: the mass of the keys with digit d, and of those among
// them whose lower digits are zero; `above`: the mass of the keys above the prefix.  The largest
// digit d for which the mass strictly above the key (prefix, d, zeros) exceeds `limit` goes to
// picked[0] (0 if there is none), the mass above that digit's keys to *carried.
__device__ __forceinline__ void pick_digit_by_mass(const unsigned long long* total, const unsigned long long* exact,
                                                   unsigned long long above, unsigned long long limit,
                                                   unsigned int* picked, unsigned long long* carried,
                                                   unsigned long long* scratch) {
  const int tid = threadIdx.x;
  const unsigned long long mine = tid < 256 ? total[tid] : 0ull;
  const unsigned long long mine_exact = tid < 256 ? exact[tid] : 0ull;
  const unsigned long long higher = above + sum_above(mine, 256, scratch);
  if (tid == 0) {
    picked[0] = 0u;
    *carried = higher;
  }
  __syncthreads();
  if (tid > 0 && tid < 256 && higher + (mine - mine_exact) > limit) atomicMax(&picked[0], (unsigned int)tid);
  __syncthreads();
  if (tid > 0 && tid == (int)picked[0]) *carried = higher;
  __syncthreads();
}

// Per-row parameters, all device arrays of `rows` entries:
//   temperature (0 = greedy), top_k (0 = off), top_p (1 = off), penalty (1 = off),
//   seed_lo / seed_hi / draw_index (Philox key and counter).
// history tokens of row r: history[history_start[r] .. history_start[r + 1]).
// unread_tokens / unread_row (both may be null): a row whose request has one more token that
// the host has not read yet (it was sampled by a launch still in flight) names that token's
// place in `unread_tokens`, or -1; it counts as part of the row's history.
// work [rows, vocab]: scratch for the penalised logits.  logprobs may be null.
// max_listed: the most tokens the short way may list (at most SAMPLE_CANDIDATES; 0: every row
// goes the long way).
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(int* __restrict__ tokens, float* __restrict__ logprobs,
              const float* __restrict__ logits, float* __restrict__ work, int vocab,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ penalty,
              const uint32_t* __restrict__ seed_lo, const uint32_t* __restrict__ seed_hi,
              const uint32_t* __restrict__ draw_index, const int* __restrict__ history,
              const int* __restrict__ history_start, const int* __restrict__ unread_tokens,
              const int* __restrict__ unread_row, int max_listed) {
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  __shared__ unsigned long long lscratch[SAMPLE_WAVES];
  __shared__ unsigned int counts[SAMPLE_WAVES][256];             // top-k: keys per digit, one histogram a wavefront
  __shared__ unsigned long long mass[MASS_COPIES][256];          // top-p: mass per digit
  __shared__ unsigned long long mass_exact[MASS_COPIES][256];    // of which: keys whose lower digits are all zero
  __shared__ unsigned int picked[2];                             // what thread 0 decided in a round
  __shared__ unsigned long long carried;
  __shared__ float wave_total[SAMPLE_WAVES];
  __shared__ int chosen;
  __shared__ unsigned int totals[256];                           // the short way: keys per digit, all wavefronts
  __shared__ unsigned int wave_first[SAMPLE_WAVES];              // the short way: tokens listed by each wavefront
  __shared__ uint32_t cand_key[SAMPLE_CANDIDATES];               // the list, in vocabulary order: ordered key
  __shared__ int cand_index[SAMPLE_CANDIDATES];                  //   and token

  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & (TS_WAVE - 1);
  const int wave = tid / TS_WAVE;
  const float* src = logits + (size_t)r * vocab;
  const float temp = temperature[r];
  const float pen = penalty[r];

  // 1. penalised copy (only where there is a penalty; else the logits themselves are read).
  // Reading the untouched logits makes a repeated history token harmless.
  const float* row = src;
  if (pen != 1.0f) {
    float* copy = work + (size_t)r * vocab;
    for (int i = tid; i < vocab; i += blockDim.x) copy[i] = src[i];
    __syncthreads();
    const int h0 = history_start[r], h1 = history_start[r + 1];
    for (int j = h0 + tid; j < h1; j += blockDim.x) {
      const int tok = history[j];
      if (tok >= 0 && tok < vocab) {
        const float v = src[tok];
        copy[tok] = v < 0.f ? v * pen : v / pen;
      }
    }
    if (tid == 0 && unread_tokens && unread_row && unread_row[r] >= 0) {
      const int tok = unread_tokens[unread_row[r]];
      if (tok >= 0 && tok < vocab) {
        const float v = src[tok];
        copy[tok] = v < 0.f ? v * pen : v / pen;
      }
    }
    __syncthreads();
    row = copy;
  }

  // 2. log-softmax terms of the penalised logits (before temperature).
  float base_max = 0.f, base_lse = 0.f;
  if (logprobs) {
    float m = -INFINITY;
    for_each_logit(row, vocab, [&](int, float v) { m = fmaxf(m, v); });
    base_max = block_max(m, fscratch);
    float s = 0.f;
    for_each_logit(row, vocab, [&](int, float v) { s += expf(v - base_max); });
    base_lse = logf(block_sum(s, fscratch));
  }

  int token;
  if (temp <= 0.f) {
    token = block_argmax(row, vocab, fscratch, iscratch);
  } else {
    const float inv_temp = 1.0f / temp;
    const int k = top_k[r];
    const float p = top_p[r];
    const bool use_k = k > 0 && k < vocab;
    const bool use_p = p < 1.0f;
    // The vocabulary is cut into one stretch per wavefront, a stretch into blocks of 256 tokens,
    // four consecutive ones per lane.
    const int block_tokens = 4 * TS_WAVE;
    const int blocks_total = (vocab + block_tokens - 1) / block_tokens;
    const int blocks_per_wave = (blocks_total + SAMPLE_WAVES - 1) / SAMPLE_WAVES;
    const int first_block = wave * blocks_per_wave;
    const int last_block = min(first_block + blocks_per_wave, blocks_total);  // exclusive
    const bool row_aligned = (reinterpret_cast<uintptr_t>(row) & 15u) == 0;
    auto lane_logits = [&](int block, float (&v)[4]) {  // beyond the vocabulary: -inf
      const int at = block * block_tokens + 4 * lane;
      if (row_aligned && at + 3 < vocab) {
        const float4 q = *reinterpret_cast<const float4*>(row + at);
        v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = at + j < vocab ? row[at + j] : -INFINITY;
      }
    };
    // f(block, the lanes' four logits) for every block of this wavefront's stretch, in order, the
    // loads of four blocks under way together (one at a time, a walk waits a trip to memory a block).
    auto walk_stretch = [&](auto f) __attribute__((always_inline)) {
      int block = first_block;
      for (; block + 3 < last_block; block += 4) {
        float a[4], b[4], c[4], d[4];
        lane_logits(block, a);
        lane_logits(block + 1, b);
        lane_logits(block + 2, c);
        lane_logits(block + 3, d);
        f(block, a);
        f(block + 1, b);
        f(block + 2, c);
        f(block + 3, d);
      }
      for (; block < last_block; ++block) {
        float a[4];
        lane_logits(block, a);
        f(block, a);
      }
    };

    // The short way, taken where a truncation leaves few tokens (the usual case: top-k of some
    // tens, or the nucleus of a peaked distribution).  One compute unit works through a row at
    // about a microsecond per instruction and element, so what counts is how often the whole row
    // is walked and with how many instructions.  Whatever a truncation keeps lies among the
    // largest logits.  The row is walked four times with a few instructions per element: for
    // its largest logit; for a histogram, 16 bits of the key deep, of the tokens whose keys lie in
    // the largest logit's leading-digit class or the one below it (for positive logits: at least
    // a quarter of the largest), from which a bound L follows at or above which at least k and at
    // most max_listed tokens lie; to count each wavefront's tokens at or above L; and to
    // list them, in vocabulary order.  Thresholds, sums and the draw then walk that list in LDS.
    // The arithmetic is that of the long way below (the same integer masses and comparisons), so
    // both choose the same thresholds; where no such L exists or a nucleus reaches below it, the
    // long way is taken.
    bool listed = false;  // the same in every thread
    float row_max = 0.f;  // what the short way has found out that the long way can use
    bool have_row_max = false;
    unsigned long long z_lane = 0ull;  // top-p alone: this thread's share of the mass of all tokens
    if (use_k || use_p) {
      float mx = -INFINITY;
      for_each_logit(row, vocab, [&](int, float v) { mx = fmaxf(mx, v); });
      const float m = block_max(mx, fscratch);  // the masses' reference: the largest logit kept is the row's largest
      row_max = m;
      have_row_max = true;
      const uint32_t top_digit = ordered_key(m) >> 24;
      const uint32_t coarse_key = (top_digit > 0u ? top_digit - 1u : 0u) << 24;
      // A token whose mass rounds to no unit at all (see mass_units) is skipped without the exponential.
      const float massless_below = m - 22.5f * temp;
      unsigned int* fine = &counts[0][0];  // 512 classes: (key - coarse_key) >> 16, the last one open above
      for (int i = tid; i < 512; i += blockDim.x) fine[i] = 0u;
      __syncthreads();
      walk_stretch([&](int block, const float (&v)[4]) __attribute__((always_inline)) {
        const int at = block * block_tokens + 4 * lane;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t key = ordered_key(v[j]);
          if (at + j < vocab) {
            if (!use_k && v[j] >= massless_below) z_lane += mass_units(v[j], m, inv_temp);  // top-p alone: the mass of all
            if (key >= coarse_key) atomicAdd(&fine[min((key - coarse_key) >> 16, 511u)], 1u);
          }
        }
      });
      __syncthreads();
      {
        // picked[0]: the lowest class listed, 512 if there is none to take: with top-k the class
        // at which the keys counted from the top reach k (if no more than the list holds lie at
        // or above it), else the lowest class from which up the list holds them all.
        const unsigned int mine = tid < 512 ? fine[tid] : 0u;
        const unsigned int above = (unsigned int)sum_above(mine, 512, lscratch);
        if (tid == 0) picked[0] = 512u;
        __syncthreads();
        if (tid < 512) {
          if (use_k) {
            if (above < (unsigned int)k && above + mine >= (unsigned int)k && above + mine <= (unsigned int)max_listed)
              picked[0] = (unsigned int)tid;  // one thread at most
          } else if (above + mine <= (unsigned int)max_listed) {
            atomicMin(&picked[0], (unsigned int)tid);
          }
        }
      }
      __syncthreads();
      const uint32_t low_class = picked[0];
      __syncthreads();
      bool fits = low_class < 512u;
      const uint32_t low_key = coarse_key + (low_class << 16);
      unsigned int listed_count = 0u;
      if (fits) {
        // How many each wavefront will list, then the listing itself.
        unsigned int mine = 0u;
        walk_stretch([&](int block, const float (&v)[4]) __attribute__((always_inline)) {
          const int at = block * block_tokens + 4 * lane;
#pragma unroll
          for (int j = 0; j < 4; ++j) mine += (at + j < vocab && ordered_key(v[j]) >= low_key) ? 1u : 0u;
        });
#pragma unroll
        for (int off = TS_WAVE / 2; off > 0; off >>= 1) mine += __shfl_xor(mine, off, TS_WAVE);
        if (lane == 0) wave_first[wave] = mine;
        __syncthreads();
        unsigned int next = 0u;  // where this wavefront's tokens begin
        for (int w = 0; w < SAMPLE_WAVES; ++w) {
          if (w == wave) next = listed_count;
          listed_count += wave_first[w];
        }
        const unsigned long long below = (1ull << lane) - 1ull;
        walk_stretch([&](int block, const float (&v)[4]) __attribute__((always_inline)) {
          const int at = block * block_tokens + 4 * lane;
          uint32_t key[4];
          unsigned long long has[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            key[j] = ordered_key(v[j]);
            has[j] = __ballot(at + j < vocab && key[j] >= low_key);
          }
          if ((has[0] | has[1] | has[2] | has[3]) == 0ull) return;
          unsigned int before = 0u, all = 0u;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            before += (unsigned int)__popcll(has[j] & below);
            all += (unsigned int)__popcll(has[j]);
          }
          unsigned int place = next + before;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if ((has[j] >> lane) & 1ull) {
              cand_key[place] = key[j];
              cand_index[place] = at + j;
              ++place;
            }
          }
          next += all;
        });
        __syncthreads();
      }
      auto stands = [&](int slot) { return (unsigned int)slot < listed_count; };
      auto listed_key = [&](int slot) -> uint32_t { return stands(slot) ? cand_key[slot] : 0u; };
      if (fits) {
        // top-k among the listed, eight bits at a time as on the long way.
        uint32_t threshold = 0u;
        if (use_k) {
          uint32_t prefix = 0u;
          unsigned int wanted = (unsigned int)k;
          for (int shift = 24; shift >= 0; shift -= 8) {
            for (int i = tid; i < SAMPLE_WAVES * 256; i += blockDim.x) (&counts[0][0])[i] = 0u;
            __syncthreads();
            const uint32_t high_mask = shift == 24 ? 0u : ~0u << (shift + 8);
            for (int slot = tid; stands(slot); slot += blockDim.x) {
              const uint32_t key = cand_key[slot];
              if ((key & high_mask) == prefix) atomicAdd(&counts[wave][(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid < 256) {
              unsigned int total = 0u;
              for (int w = 0; w < SAMPLE_WAVES; ++w) total += counts[w][tid];
              totals[tid] = total;
            }
            __syncthreads();
            pick_digit_by_count(totals, wanted, picked, lscratch);
            prefix |= picked[0] << shift;
            wanted = picked[1];
            __syncthreads();
          }
          threshold = prefix;
        }
        // top-p among the listed, as on the long way; a nucleus that reaches below the list is
        // the long way's business.
        bool inside = true;  // the same in every thread
        if (use_p) {
          unsigned long long z_listed = 0ull;
          for (int slot = tid; stands(slot); slot += blockDim.x) {
            const uint32_t key = cand_key[slot];
            if (key >= threshold) z_listed += mass_units(key_value(key), m, inv_temp);
          }
          z_listed = block_sum_u64(z_listed, lscratch);
          const unsigned long long z = use_k ? z_listed : block_sum_u64(z_lane, lscratch);
          const unsigned long long limit = (unsigned long long)((double)p * (double)z);
          inside = use_k || z_listed > limit;
          if (inside) {
            uint32_t prefix = 0u;
            unsigned long long above = 0ull;
            for (int shift = 24; shift >= 0; shift -= 8) {
              for (int i = tid; i < MASS_COPIES * 256; i += blockDim.x) {
                (&mass[0][0])[i] = 0ull;
                (&mass_exact[0][0])[i] = 0ull;
              }
              __syncthreads();
              const uint32_t high_mask = shift == 24 ? 0u : ~0u << (shift + 8);
              const uint32_t low_mask = shift == 0 ? 0u : ~0u >> (32 - shift);
              for (int slot = tid; stands(slot); slot += blockDim.x) {
                const uint32_t key = cand_key[slot];
                if (key >= threshold && (key & high_mask) == prefix) {
                  const unsigned long long units = mass_units(key_value(key), m, inv_temp);
                  const uint32_t digit = (key >> shift) & 255u;
                  atomicAdd(&mass[wave % MASS_COPIES][digit], units);
                  if ((key & low_mask) == 0u) atomicAdd(&mass_exact[wave % MASS_COPIES][digit], units);
                }
              }
              __syncthreads();
              if (tid < 256) {
                unsigned long long total = 0ull, exact = 0ull;
                for (int c = 0; c < MASS_COPIES; ++c) {
                  total += mass[c][tid];
                  exact += mass_exact[c][tid];
                }
                mass[0][tid] = total;
                mass_exact[0][tid] = exact;
              }
              __syncthreads();
              pick_digit_by_mass(mass[0], mass_exact[0], above, limit, picked, &carried, lscratch);
              prefix |= picked[0] << shift;
              above = carried;
              __syncthreads();
            }
            if (prefix + 1u > threshold) threshold = prefix + 1u;
          }
        }
        if (inside) {
          // The draw, by the first wavefront: the list 64 places at a time, in vocabulary order,
          // the cumulative mass added up in a fixed order; as on the long way the intervals join,
          // and where rounding lets the walk end below the target the last token with mass is taken.
          if (tid == 0) chosen = -1;
          __syncthreads();
          if (wave == 0) {
            auto lane_mass = [&](int slot) {
              const uint32_t key = listed_key(slot);
              return (stands(slot) && key >= threshold) ? draw_mass((key_value(key) - m) * inv_temp) : 0.f;
            };
            auto inclusive = [&](float v) {
#pragma unroll
              for (int off = 1; off < TS_WAVE; off <<= 1) {
                const float other = __shfl_up(v, off, TS_WAVE);
                if (lane >= off) v += other;
              }
              return v;
            };
            float total = 0.f;
            for (int s0 = 0; stands(s0); s0 += TS_WAVE)
              total += __shfl(inclusive(lane_mass(s0 + lane)), TS_WAVE - 1, TS_WAVE);
            const float u = philox_uniform(seed_lo[r], seed_hi[r], draw_index[r]);
            float target = u * total;
            const float below_total = __uint_as_float(__float_as_uint(total) - 1u);
            if (target > below_total) target = below_total;
            float sum = 0.f;
            int last_with_mass = -1;
            bool found = false;
            for (int s0 = 0; stands(s0) && !found; s0 += TS_WAVE) {
              const float mine = lane_mass(s0 + lane);
              const float through = inclusive(mine);
              const unsigned long long with_mass = __ballot(mine > 0.f);
              const unsigned long long over = __ballot(mine > 0.f && sum + through > target);
              if (over != 0ull) {
                if (lane == __ffsll((long long)over) - 1) chosen = cand_index[s0 + lane];
                found = true;
              } else if (with_mass != 0ull) {
                last_with_mass = s0 + 63 - __clzll((long long)with_mass);
              }
              sum += __shfl(through, TS_WAVE - 1, TS_WAVE);
            }
            if (!found && last_with_mass >= 0 && lane == 0) chosen = cand_index[last_with_mass];
          }
          listed = true;
        }
      }
    }
    if (!listed) {
    // 3. top-k: the k-th largest key, found eight bits at a time: the digit whose keys, with
    // those of higher digits, reach k, then the same among the keys that share it.
    uint32_t threshold = 0u;
    if (k > 0 && k < vocab) {
      uint32_t prefix = 0u;
      unsigned int wanted = (unsigned int)k;  // among the keys that share `prefix`
      for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = tid; i < SAMPLE_WAVES * 256; i += blockDim.x) (&counts[0][0])[i] = 0u;
        __syncthreads();
        const uint32_t high_mask = shift == 24 ? 0u : ~0u << (shift + 8);
        for_each_logit(row, vocab, [&](int, float v) {
          const uint32_t key = ordered_key(v);
          if ((key & high_mask) == prefix) atomicAdd(&counts[wave][(key >> shift) & 255u], 1u);
        });
        __syncthreads();
        if (tid < 256) {  // one histogram, in counts[0]
          unsigned int total = 0u;
          for (int w = 0; w < SAMPLE_WAVES; ++w) total += counts[w][tid];
          counts[0][tid] = total;
        }
        __syncthreads();
        pick_digit_by_count(counts[0], wanted, picked, lscratch);
        prefix |= picked[0] << shift;
        wanted = picked[1];
        __syncthreads();
      }
      threshold = prefix;
    }
    // Softmax terms of the scaled logits over what top-k kept: their largest is the row's largest.
    float m = row_max;
    if (!have_row_max) {
      float mx = -INFINITY;
      for_each_logit(row, vocab, [&](int, float v) { mx = fmaxf(mx, v); });
      m = block_max(mx, fscratch);
    }
    const float massless_below = m - 22.5f * temp;  // below it a token's mass rounds to no unit (see mass_units)
    // 4. top-p: keep a token while the mass strictly above it is <= p.  T is the largest key whose
    // mass strictly above still exceeds the limit, again eight bits at a time: for a candidate whose
    // lower digits are zero, the mass above it is that of the higher digits plus that of its own
    // digit less the keys that equal the candidate itself.
    if (p < 1.0f) {
      unsigned long long z = z_lane;  // top-p alone: added up on the short way already
      if (use_k || !have_row_max) {
        z = 0ull;
        for_each_logit(row, vocab, [&](int, float v) {
          if (v >= massless_below && ordered_key(v) >= threshold) z += mass_units(v, m, inv_temp);
        });
      }
      z = block_sum_u64(z, lscratch);
      const unsigned long long limit = (unsigned long long)((double)p * (double)z);
      uint32_t prefix = 0u;
      unsigned long long above = 0ull;  // mass of the keys whose higher digits exceed the prefix's
      for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = tid; i < MASS_COPIES * 256; i += blockDim.x) {
          (&mass[0][0])[i] = 0ull;
          (&mass_exact[0][0])[i] = 0ull;
        }
        __syncthreads();
        const uint32_t high_mask = shift == 24 ? 0u : ~0u << (shift + 8);
        const uint32_t low_mask = shift == 0 ? 0u : ~0u >> (32 - shift);
        for_each_logit(row, vocab, [&](int, float v) {
          const uint32_t key = ordered_key(v);
          if (v >= massless_below && key >= threshold && (key & high_mask) == prefix) {
            const unsigned long long units = mass_units(v, m, inv_temp);
            const uint32_t digit = (key >> shift) & 255u;
            atomicAdd(&mass[wave % MASS_COPIES][digit], units);
            if ((key & low_mask) == 0u) atomicAdd(&mass_exact[wave % MASS_COPIES][digit], units);
          }
        });
        __syncthreads();
        if (tid < 256) {
          unsigned long long total = 0ull, exact = 0ull;
          for (int c = 0; c < MASS_COPIES; ++c) {
            total += mass[c][tid];
            exact += mass_exact[c][tid];
          }
          mass[0][tid] = total;
          mass_exact[0][tid] = exact;
        }
        __syncthreads();
        pick_digit_by_mass(mass[0], mass_exact[0], above, limit, picked, &carried, lscratch);
        prefix |= picked[0] << shift;
        above = carried;
        __syncthreads();
      }
      // prefix is T only if the mass above it does exceed the limit; otherwise nothing is cut here
      // (every digit fell through to 0: T = 0, as the search bit by bit would leave it).
      if (prefix + 1u > threshold) threshold = prefix + 1u;
    }
    // 5. draw, over the wavefronts' stretches.  Cumulative mass is added up in a fixed order (a
    // lane's four, the lanes of a block by a scan, blocks and stretches one after the other); every
    // interval ends where the next begins by construction, so exactly one stretch, block, lane
    // and token take the target, and where rounding lets a walk end below it, the last token
    // with mass does.
    auto lane_masses = [&](int block, float (&e)[4]) {
      const int at = block * block_tokens + 4 * lane;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = at + j;
        const float v = i < vocab ? row[i] : -INFINITY;
        e[j] = (i < vocab && ordered_key(v) >= threshold) ? draw_mass((v - m) * inv_temp) : 0.f;
      }
    };
    auto wave_inclusive = [&](float v) {  // sum over lanes 0 .. lane, always by the same additions
#pragma unroll
      for (int off = 1; off < TS_WAVE; off <<= 1) {
        const float other = __shfl_up(v, off, TS_WAVE);
        if (lane >= off) v += other;
      }
      return v;
    };
    float stretch = 0.f;
    walk_stretch([&](int block, const float (&v)[4]) __attribute__((always_inline)) {
      const int at = block * block_tokens + 4 * lane;
      float e[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        e[j] = (at + j < vocab && ordered_key(v[j]) >= threshold) ? draw_mass((v[j] - m) * inv_temp) : 0.f;
      stretch += __shfl(wave_inclusive((e[0] + e[1]) + (e[2] + e[3])), TS_WAVE - 1, TS_WAVE);
    });
    if (lane == 0) wave_total[wave] = stretch;
    if (tid == 0) chosen = -1;
    __syncthreads();
    float before = 0.f, after = 0.f, total = 0.f;  // cumulative mass where this stretch begins and ends, and all of it
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
      if (w == wave) before = total;
      total += wave_total[w];
      if (w == wave) after = total;
    }
    const float u = philox_uniform(seed_lo[r], seed_hi[r], draw_index[r]);
    float target = u * total;
    const float below_total = __uint_as_float(__float_as_uint(total) - 1u);
    if (target > below_total) target = below_total;
    if (before <= target && target < after) {  // true in one wavefront, for all of its lanes
      float sum = before;
      int fallback_block = -1;
      bool found = false;
      for (int block = first_block; block < last_block && !found; ++block) {
        float e[4];
        lane_masses(block, e);
        const float mine = (e[0] + e[1]) + (e[2] + e[3]);
        const float through = wave_inclusive(mine);
        float upto_previous = __shfl_up(through, 1, TS_WAVE);
        if (lane == 0) upto_previous = 0.f;
        const unsigned long long with_mass = __ballot(mine > 0.f);
        const unsigned long long over = __ballot(mine > 0.f && sum + through > target);
        if (over != 0ull) {
          if (lane == __ffsll((long long)over) - 1) {
            float inner = sum + upto_previous;
            int pick = -1;
            for (int j = 0; j < 4; ++j) {
              if (e[j] > 0.f) {
                inner += e[j];
                pick = block * block_tokens + 4 * lane + j;
                if (inner > target) break;
              }
            }
            chosen = pick;
          }
          found = true;
        } else if (with_mass != 0ull) {
          fallback_block = block;
        }
        sum += __shfl(through, TS_WAVE - 1, TS_WAVE);
      }
      if (!found && fallback_block >= 0) {
        float e[4];
        lane_masses(fallback_block, e);
        const unsigned long long with_mass = __ballot((e[0] + e[1]) + (e[2] + e[3]) > 0.f);
        if (lane == 63 - __clzll((long long)with_mass)) {
          int pick = -1;
          for (int j = 0; j < 4; ++j)
            if (e[j] > 0.f) pick = fallback_block * block_tokens + 4 * lane + j;
          chosen = pick;
        }
      }
    }
    }  // the long way
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
                         const int* unread_tokens, const int* unread_row, int max_listed, hipStream_t stream) {
  if (rows == 0) return TS_OK;
  if (!tokens || !logits || !work || vocab < 1 || !temperature || !top_k || !top_p || !penalty ||
      !seed_lo || !seed_hi || !draw_index || !history_start || max_listed < 0)
    return TS_ERR_ARG;
  if (max_listed > SAMPLE_CANDIDATES) max_listed = SAMPLE_CANDIDATES;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, tokens, logprobs,
                     logits, work, vocab, temperature, top_k, top_p, penalty, seed_lo, seed_hi,
                     draw_index, history, history_start, unread_tokens, unread_row, max_listed);
  return ts_launch_status();
}
