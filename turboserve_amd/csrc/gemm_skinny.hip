// Weight-streaming product for a few rows, activations resident in LDS:
//   partial[s][m][n] = sum over the k-range of split s of  X[m][k] * W[n][k]   (+ bias[n] in split 0)
// for M <= 16 rows of bfloat16 activations, bfloat16 weights [N, K] as the checkpoint stores
// them (F.linear's layout, src/turboserve/engine/model/layers.py:142), 32-bit accumulation on
// the matrix cores and 32-bit partial sums out.  The consumer (norm, rotary/cache write,
// SwiGLU, or nobody when splits == 1) adds the splits up, so no rounding happens between the
// product and its consumer.  (gemm_tiled.hip holds the product for up to 64 rows; this one
// serves small matrices, whose product lasts a few microseconds and gains from many small
// workgroups that start quickly, and the widest matrices at up to eight rows.)
//
// The product is bound by reading W once from HBM.  Layout of the work:
//   * a workgroup of 4 or 8 wavefronts owns 64 or 128 consecutive weight rows (16 per
//     wavefront) and one k-range; the grid is (row blocks, splits);
//   * the k-range is walked in chunks of 256: eight loads per lane, each of which has the four
//     lane groups of a weight row cover 64 contiguous bytes (so a load instruction touches 16
//     rows x 64 bytes, and the eight of a chunk 512 contiguous bytes per row), issued one chunk
//     ahead of the matrix cores;
//   * v_mfma_f32_16x16x32_bf16 with A = 16 weight rows, B = 16 activation rows, step j of a
//     chunk covering k = chunk + 32 j .. + 31.
#include "common.hpp"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int CHUNK = 256;          // k per iteration
constexpr int STEPS = CHUNK / 32;   // matrix-core steps per chunk
constexpr int ROWS_PER_WAVE = 16;

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

struct WeightChunk {
  u32x4 piece[STEPS];  // k = chunk + 32 j + 8 g .. + 7 of the lane's row, j = 0..7
};

// `row` points at the lane's weight row; k_limit = K: pieces at or beyond it read as zero
// (K is a multiple of 8, so a piece is wholly inside or wholly outside).
template <bool ONCE>
__device__ __forceinline__ void load_weights(WeightChunk& w, const uint16_t* row, int k0, int group, int k_limit) {
  auto load = [](const uint16_t* p) -> u32x4 { return ONCE ? load_once16(p) : *reinterpret_cast<const u32x4*>(p); };
  const int base = k0 + 8 * group;
  if (k0 + CHUNK <= k_limit) {
#pragma unroll
    for (int j = 0; j < STEPS; ++j) w.piece[j] = load(row + base + 32 * j);
  } else {
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      const int k = base + 32 * j;
      w.piece[j] = (k < k_limit) ? load(row + k) : u32x4{0u, 0u, 0u, 0u};
    }
  }
}

// The same product for M <= 16 with the activations resident in LDS: a workgroup stages its
// split's activations X[0..mpad-1][k-range] once (in stretches of `stage_chunks` chunks when
// the range is longer than LDS should hold) and its wavefronts then stream their weight rows
// without meeting at a barrier again, two chunks of loads in flight each.  mpad is 8 or 16;
// lanes whose activation row is beyond mpad read a real row again and drop the result.
template <int WAVES, bool ONCE>
__global__ void __launch_bounds__(WAVES * TS_WAVE)
gemm_skinny_resident_kernel(float* __restrict__ partial, const uint16_t* __restrict__ x, long x_stride,
                            const uint16_t* __restrict__ w, const uint16_t* __restrict__ bias, int m, int mpad,
                            int n, int k, int chunks_per_split, int stage_chunks) {
  extern __shared__ __attribute__((aligned(16))) uint16_t xs_resident[];
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const int lane16 = lane & 15;
  const int group = lane >> 4;
  const int split = blockIdx.y;
  const int n0 = (blockIdx.x * WAVES + wave) * ROWS_PER_WAVE;
  const int total_chunks = (k + CHUNK - 1) / CHUNK;
  const int first = split * chunks_per_split;
  const int last = min(first + chunks_per_split, total_chunks);  // exclusive

  const int row_index = min(n0 + lane16, n - 1);
  const uint16_t* wrow = w + (size_t)row_index * k;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};

  if (first < last) {
    const int stage = min(stage_chunks, last - first);  // chunks per stretch; even unless it is the whole range
    const int x_row = stage * CHUNK + 8;                 // LDS row stride in elements
    const int pieces_per_row = stage * (CHUNK / 8);
    const uint16_t* xl = xs_resident + (lane16 % mpad) * x_row + 8 * group;
    WeightChunk wa, wb;
    load_weights<ONCE>(wa, wrow, first * CHUNK, group, k);
    if (first + 1 < last) load_weights<ONCE>(wb, wrow, (first + 1) * CHUNK, group, k);
    for (int begin = first; begin < last; begin += stage) {
      const int end = min(begin + stage, last);
      if (begin != first) __syncthreads();  // everyone has read the previous stretch
      const int k_begin = begin * CHUNK;
      const int live_pieces = (end - begin) * (CHUNK / 8);
      for (int idx = threadIdx.x; idx < mpad * pieces_per_row; idx += WAVES * TS_WAVE) {
        const int row = idx / pieces_per_row;
        const int piece = idx - row * pieces_per_row;
        if (piece >= live_pieces) continue;
        const int kk = k_begin + 8 * piece;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (row < m && kk < k) v = *reinterpret_cast<const u32x4*>(x + (size_t)row * x_stride + kk);
        *reinterpret_cast<u32x4*>(xs_resident + row * x_row + 8 * piece) = v;
      }
      __syncthreads();
      // A stretch other than the last has an even number of chunks, so it starts on `wa`.
      for (int c = begin; c < end; c += 2) {
        const uint16_t* xc = xl + (c - begin) * CHUNK;
#pragma unroll
        for (int j = 0; j < STEPS; ++j) {
          const u32x4 b = *reinterpret_cast<const u32x4*>(xc + 32 * j);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa.piece[j]), as_bf16x8(b), acc, 0, 0, 0);
        }
        if (c + 2 < last) load_weights<ONCE>(wa, wrow, (c + 2) * CHUNK, group, k);
        if (c + 1 >= end) break;
#pragma unroll
        for (int j = 0; j < STEPS; ++j) {
          const u32x4 b = *reinterpret_cast<const u32x4*>(xc + CHUNK + 32 * j);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wb.piece[j]), as_bf16x8(b), acc, 0, 0, 0);
        }
        if (c + 3 < last) load_weights<ONCE>(wb, wrow, (c + 3) * CHUNK, group, k);
      }
    }
  }

  // acc[i] = sum for weight row n0 + 4 g + i and activation row lane16.
  const int nrow = n0 + 4 * group;
  if (nrow < n && lane16 < m) {
    f32x4 b = {0.f, 0.f, 0.f, 0.f};
    if (bias && split == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nrow + i < n) b[i] = to_float(bf16_t{bias[nrow + i]});
    }
    float* dst = partial + ((size_t)split * m + lane16) * n + nrow;
    const f32x4 v = acc + b;
    if (nrow + 3 < n && (n & 3) == 0) {
      *reinterpret_cast<f32x4*>(dst) = v;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nrow + i < n) dst[i] = v[i];
    }
  }
}

}  // namespace

// partial [splits, m, n] float (contiguous); x [m, k] bfloat16 with row stride x_stride; w [n, k]
// bfloat16 contiguous; bias [n] bfloat16 or null.  Needs m <= 16, k % 8 == 0.  chunks_per_split
// 256-wide chunks of k go to each of `splits` = ceil(ceil(k / 256) / chunks_per_split).  waves:
// wavefronts (16 weight rows each) per workgroup, 4 or 8.  stage_chunks: chunks staged at a time,
// an even number unless it covers a whole split; the LDS it needs,
// mpad * (min(stage_chunks, chunks_per_split) * 256 + 8) * 2 bytes with mpad = 8 or 16, must be <= 64 KiB.
// once: the weights are read with non-temporal loads.
extern "C" int ts_gemm_skinny_resident(float* partial, const void* x, long x_stride, const void* w, const void* bias,
                                       int m, int n, int k, int chunks_per_split, int splits, int waves,
                                       int stage_chunks, int once, hipStream_t stream) {
  if (m == 0 || n == 0) return TS_OK;
  if (!partial || !x || !w || m < 0 || n < 0 || k < 8) return TS_ERR_ARG;
  if (m > 16 || (k & 7) != 0 || x_stride < k || (x_stride & 7) != 0) return TS_ERR_SHAPE;
  const int total_chunks = (k + CHUNK - 1) / CHUNK;
  if (chunks_per_split < 1 || splits != (total_chunks + chunks_per_split - 1) / chunks_per_split) return TS_ERR_SHAPE;
  if (stage_chunks < 1 || (stage_chunks < chunks_per_split && (stage_chunks & 1) != 0)) return TS_ERR_SHAPE;
  const int mpad = m <= 8 ? 8 : 16;
  const int stage = stage_chunks < chunks_per_split ? stage_chunks : chunks_per_split;
  const size_t lds = (size_t)mpad * (stage * CHUNK + 8) * sizeof(uint16_t);
  if (lds > 64 * 1024 || splits > 65535) return TS_ERR_SHAPE;
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
  const uint16_t* bp = (const uint16_t*)bias;
  dim3 grid((n + 16 * waves - 1) / (16 * waves), splits), block(waves * TS_WAVE);
  if (waves != 4 && waves != 8) return TS_ERR_SHAPE;
#define TS_LAUNCH_RESIDENT(W, O)                                                                                      \
  hipLaunchKernelGGL((gemm_skinny_resident_kernel<W, O>), grid, block, lds, stream, partial, xp, x_stride, wp, bp, m, \
                     mpad, n, k, chunks_per_split, stage_chunks)
  if (waves == 4 && once) TS_LAUNCH_RESIDENT(4, true);
  else if (waves == 4) TS_LAUNCH_RESIDENT(4, false);
  else if (once) TS_LAUNCH_RESIDENT(8, true);
  else TS_LAUNCH_RESIDENT(8, false);
#undef TS_LAUNCH_RESIDENT
  return ts_launch_status();
}
