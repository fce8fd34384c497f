// Weight-streaming product for decode-sized batches, tiled through LDS:
//   partial[s][m][n] = sum over the k-range of split s of  X[m][k] * W[n][k]   (+ bias[n] in split 0)
// for M <= 128 rows of bfloat16 activations, bfloat16 weights [N, K] as the checkpoint stores
// them (F.linear's layout, src/turboserve/engine/model/layers.py:142), 32-bit accumulation on
// the matrix cores and 32-bit partial sums out; the consumer adds the splits up.
//
// The product is bound by reading W once from HBM, and what decides its rate is how the reading
// is spread over the device, not how much of it is in flight:
//   * a workgroup of four wavefronts (2 x 2) owns a tile of NT = 32 TN weight rows (TN = 2, 4
//     or 5; 8 for up to 32 activation rows) by all activation rows (16 of them, 32 when M > 16, 64 when M > 32, 128 when M > 64: rows beyond M
//     are repeats that cost loads and LDS writes, so the tile is no larger than it must be) and
//     one range of K; the host
//     sizes tiles and ranges so that
//     the grid is about one workgroup per compute unit (two for the smallest tile): every
//     compute unit then streams one contiguous block of each of its rows, start to end;
//   * the range is walked 128 deep: both operands travel global memory -> registers (16-byte
//     pieces; consecutive threads take consecutive pieces of a row, 256 contiguous bytes per row)
//     -> LDS (two buffers, rows padded by 16 bytes against bank conflicts) -> matrix cores.  The
//     loads of an iteration are issued one iteration ahead; more in flight measured slower;
//   * every load is issued on every path (rows beyond N or M repeat the last row, iterations
//     beyond the range repeat its last one), so the compiler can count the loads in flight and
//     waits only for those it needs; pieces beyond K are cleared on their way into LDS;
//   * a wavefront computes TN x MB tiles of v_mfma_f32_16x16x32_bf16 (A = 16 weight rows, B = 16
//     activation rows; MB = 1, 2 or 4): each weight fragment it reads from LDS serves MB
//     products, each activation fragment TN.
#include "common.hpp"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int DEPTH = 128;            // k per iteration
constexpr int LDS_ROW = DEPTH + 8;    // LDS row stride in elements
constexpr int M_MAX = 128;            // most activation rows (a workgroup covers 32 MB: rows beyond M are repeats)
constexpr int THREADS = 256;
constexpr int ROW_PIECES = DEPTH / 8; // 16-byte pieces of a row of an iteration

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// XROWS: activation rows of a workgroup's tile, 32 MB (each half of the wavefronts takes 16 MB of
// them), or 16 with MB = 1: then both halves read the same 16 rows, the second half's products
// are duplicates that nobody stores, and half as much is fetched and staged.
template <int TN, int XROWS>
struct TileRegs {
  static constexpr int W_PIECES = 32 * TN * ROW_PIECES / THREADS;  // 2 TN
  static constexpr int X_PIECES = XROWS * ROW_PIECES / THREADS;    // XROWS / 16
  u32x4 w[W_PIECES];
  u32x4 x[X_PIECES];
};

template <int TN, int MB, int XROWS>
__global__ void __launch_bounds__(THREADS)
gemm_tiled_kernel(float* __restrict__ partial, uint16_t* __restrict__ gated, const uint16_t* __restrict__ x,
                  long x_stride, const uint16_t* __restrict__ w, const uint16_t* __restrict__ bias, int m, int n,
                  int k, int iters_per_split) {
  constexpr int NT = 32 * TN;
  static_assert(XROWS == 32 * MB || (XROWS == 16 && MB == 1), "a tile of 32 MB activation rows, or of 16");
  constexpr bool SHARED_ROWS = XROWS == 16;  // both halves of the wavefronts work on the same 16 rows
  constexpr int STAGE = (NT + XROWS) * LDS_ROW;  // elements of one LDS buffer: weight rows, then activation rows
  typedef TileRegs<TN, XROWS> Regs;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [2][STAGE]
  const int tid = threadIdx.x;
  const int lane = tid & (TS_WAVE - 1);
  const int wave = tid / TS_WAVE;
  const int lane16 = lane & 15;
  const int group = lane >> 4;
  const int wave_n = wave >> 1;  // which half of the tile's weight rows
  const int wave_m = wave & 1;   // which half of the activation rows
  const int n_base = blockIdx.x * NT;
  const int split = blockIdx.y;
  const int total = (k + DEPTH - 1) / DEPTH;
  const int first = split * iters_per_split;
  const int last = min(first + iters_per_split, total);  // exclusive
  if (first >= last) return;                              // the whole workgroup leaves together

  // This thread's pieces: piece p = tid + 256 i of a tile is row p / 16, bytes 16 (p % 16) of the
  // iteration's 256.  Source pointers are at k = 0; destinations are offsets inside a buffer.
  const uint16_t* wsrc[Regs::W_PIECES];
  const uint16_t* xsrc[Regs::X_PIECES];
  const int piece_k = 8 * (tid % ROW_PIECES);
  const int piece_row = tid / ROW_PIECES;  // rows advance by 16 per i
#pragma unroll
  for (int i = 0; i < Regs::W_PIECES; ++i)
    wsrc[i] = w + (size_t)min(n_base + piece_row + 16 * i, n - 1) * k;
#pragma unroll
  for (int i = 0; i < Regs::X_PIECES; ++i)
    xsrc[i] = x + (size_t)min(piece_row + 16 * i, m - 1) * x_stride;
  const int dst = piece_row * LDS_ROW + piece_k;  // + 16 i rows

  auto fetch = [&](Regs& r, int it) {
    // Iterations beyond the range repeat its last one; a piece beyond K reads the last piece of
    // the row instead (cleared in `stage`).
    const int k0 = min(min(it, last - 1) * DEPTH + piece_k, k - 8);
#pragma unroll
    for (int i = 0; i < Regs::X_PIECES; ++i) r.x[i] = *reinterpret_cast<const u32x4*>(xsrc[i] + k0);
#pragma unroll
    for (int i = 0; i < Regs::W_PIECES; ++i) r.w[i] = load_once16(wsrc[i] + k0);
  };
  auto stage = [&](const Regs& r, int buf, int it) {
    uint16_t* base = lds + buf * STAGE + dst;
    if ((it + 1) * DEPTH <= k) {  // the same in every thread; the usual case, kept free of selects
#pragma unroll
      for (int i = 0; i < Regs::X_PIECES; ++i) *reinterpret_cast<u32x4*>(base + (NT + 16 * i) * LDS_ROW) = r.x[i];
#pragma unroll
      for (int i = 0; i < Regs::W_PIECES; ++i) *reinterpret_cast<u32x4*>(base + 16 * i * LDS_ROW) = r.w[i];
    } else {  // the last iteration of a K that is no multiple of 128 (or one past the end, never read)
      const bool beyond = it * DEPTH + piece_k >= k;
      const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int i = 0; i < Regs::X_PIECES; ++i)
        *reinterpret_cast<u32x4*>(base + (NT + 16 * i) * LDS_ROW) = beyond ? zero : r.x[i];
#pragma unroll
      for (int i = 0; i < Regs::W_PIECES; ++i)
        *reinterpret_cast<u32x4*>(base + 16 * i * LDS_ROW) = beyond ? zero : r.w[i];
    }
  };

  f32x4 acc[TN][MB];
#pragma unroll
  for (int a = 0; a < TN; ++a) {
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  auto multiply = [&](int buf) {
    const uint16_t* base = lds + buf * STAGE + lane16 * LDS_ROW + 8 * group;
#pragma unroll
    for (int step = 0; step < DEPTH / 32; ++step) {
      u32x4 xf[MB];
#pragma unroll
      for (int b = 0; b < MB; ++b)
        xf[b] = *reinterpret_cast<const u32x4*>(base + (NT + (SHARED_ROWS ? 0 : 16 * MB * wave_m) + 16 * b) * LDS_ROW + 32 * step);
#pragma unroll
      for (int a = 0; a < TN; ++a) {
        const u32x4 wf = *reinterpret_cast<const u32x4*>(base + (wave_n * TN + a) * 16 * LDS_ROW + 32 * step);
#pragma unroll
        for (int b = 0; b < MB; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wf), as_bf16x8(xf[b]), acc[a][b], 0, 0, 0);
      }
    }
  };

  // Invariant at the top of a round for iteration `it`: LDS buffer (it - first) % 2 holds it
  // (complete, behind a barrier) and `regs` holds iteration it + 1 (its loads were issued a
  // round ago).
  Regs regs;
  fetch(regs, first);
  stage(regs, 0, first);
  fetch(regs, first + 1);
  __syncthreads();
  for (int it = first; it < last; ++it) {
    const int buf = (it - first) & 1;
    stage(regs, buf ^ 1, it + 1);  // that buffer was last read a round ago, before the barrier
    fetch(regs, it + 2);
    multiply(buf);
    __syncthreads();
  }

  // acc[a][b][i] = sum for weight row n_base + 16 (wave_n TN + a) + 4 g + i and activation row
  // 16 MB wave_m + 16 b + lane16 (with shared rows: row lane16, stored by the first half only).
  if (SHARED_ROWS && wave_m != 0) return;
#pragma unroll
  for (int a = 0; a < TN; ++a) {
    const int nrow = n_base + (wave_n * TN + a) * 16 + 4 * group;
    if (nrow >= n) continue;
    f32x4 bv = {0.f, 0.f, 0.f, 0.f};
    if (bias && split == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nrow + i < n) bv[i] = to_float(bf16_t{bias[nrow + i]});
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int row = (SHARED_ROWS ? 0 : 16 * MB * wave_m) + 16 * b + lane16;
      if (row >= m) continue;
      if (gated) {
        // The matrix is a gate|up projection with rows alternating gate, up (one range of K, no
        // bias): the lane holds two such pairs and writes silu(gate) * up for both, rounded once,
        // by the formula of the stand-alone SwiGLU kernel.
        const f32x4 s = acc[a][b];
        const float lo = s[0] / (1.f + expf(-s[0])) * s[1];
        const float hi = s[2] / (1.f + expf(-s[2])) * s[3];
        uint16_t* out = gated + (size_t)row * (n / 2) + nrow / 2;
        if (nrow + 3 < n) {
          *reinterpret_cast<uint32_t*>(out) =
              (uint32_t)from_float<bf16_t>(lo).bits | ((uint32_t)from_float<bf16_t>(hi).bits << 16);
        } else if (nrow + 1 < n) {
          out[0] = from_float<bf16_t>(lo).bits;
        }
        continue;
      }
      float* out = partial + ((size_t)split * m + row) * n + nrow;
      const f32x4 v = acc[a][b] + bv;
      if (nrow + 3 < n && (n & 3) == 0) {
        *reinterpret_cast<f32x4*>(out) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nrow + i < n) out[i] = v[i];
      }
    }
  }
}

template <int TN, int MB, int XROWS = 32 * MB>
int launch_tiled_rows(float* partial, uint16_t* gated, const uint16_t* x, long x_stride, const uint16_t* w,
                      const uint16_t* bias, int m, int n, int k, int iters_per_split, int splits,
                      hipStream_t stream) {
  constexpr int NT = 32 * TN;
  constexpr size_t lds_bytes = (size_t)2 * (NT + XROWS) * LDS_ROW * sizeof(uint16_t);
  static_assert(lds_bytes <= 160 * 1024, "two buffers must fit the LDS of a compute unit");
  if (lds_bytes > 48 * 1024) {
    static bool raised = false;  // per process; the attribute belongs to the kernel
    if (!raised) {
      if (hipFuncSetAttribute((const void*)gemm_tiled_kernel<TN, MB, XROWS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds_bytes) != hipSuccess)
        return TS_ERR_LAUNCH;
      raised = true;
    }
  }
  dim3 grid((n + NT - 1) / NT, splits);
  hipLaunchKernelGGL((gemm_tiled_kernel<TN, MB, XROWS>), grid, dim3(THREADS), lds_bytes, stream, partial, gated, x, x_stride,
                     w, bias, m, n, k, iters_per_split);
  return ts_launch_status();
}

template <int TN>
int launch_tiled(float* partial, uint16_t* gated, const uint16_t* x, long x_stride, const uint16_t* w,
                 const uint16_t* bias, int m, int n, int k, int iters_per_split, int splits, hipStream_t stream) {
  if (m <= 16)
    return launch_tiled_rows<TN, 1, 16>(partial, gated, x, x_stride, w, bias, m, n, k, iters_per_split, splits, stream);
  if (m <= 32)
    return launch_tiled_rows<TN, 1>(partial, gated, x, x_stride, w, bias, m, n, k, iters_per_split, splits, stream);
  if (m <= 64)
    return launch_tiled_rows<TN, 2>(partial, gated, x, x_stride, w, bias, m, n, k, iters_per_split, splits, stream);
  return launch_tiled_rows<TN, 4>(partial, gated, x, x_stride, w, bias, m, n, k, iters_per_split, splits, stream);
}

// Tiles of 256 weight rows (TN = 8): with more than 32 activation rows two buffers no longer fit
// the LDS of a compute unit.
constexpr int M_MAX_TALL = 32;

template <int TN>
int launch_tiled_tall(float* partial, uint16_t* gated, const uint16_t* x, long x_stride, const uint16_t* w,
                      const uint16_t* bias, int m, int n, int k, int iters_per_split, int splits, hipStream_t stream) {
  if (m <= 16)
    return launch_tiled_rows<TN, 1, 16>(partial, gated, x, x_stride, w, bias, m, n, k, iters_per_split, splits, stream);
  if (m <= M_MAX_TALL)
    return launch_tiled_rows<TN, 1>(partial, gated, x, x_stride, w, bias, m, n, k, iters_per_split, splits, stream);
  return TS_ERR_SHAPE;
}

}  // namespace

// partial [splits, m, n] float (contiguous); x [m, k] bfloat16 with row stride x_stride;
// w [n, k] bfloat16 contiguous; bias [n] bfloat16 or null.  Needs m <= 128, k % 8 == 0.
// iters_per_split iterations of 128 of k go to each of `splits` = ceil(ceil(k / 128) / iters_per_split).
// tile: 16-row tiles of weights per wavefront, 2, 4 or 5 (a workgroup covers 64, 128 or 160 rows),
// or, for m <= 32, 8 (256 rows).
// gated (bfloat16 [m, n / 2], contiguous) instead of partial: w is a gate|up projection whose rows
// alternate gate, up, and the kernel writes silu(gate) * up; needs splits == 1, no bias, n even.
extern "C" int ts_gemm_tiled(float* partial, void* gated, const void* x, long x_stride, const void* w,
                             const void* bias, int m, int n, int k, int iters_per_split, int splits, int tile,
                             hipStream_t stream) {
  if (m == 0 || n == 0) return TS_OK;
  if (!x || !w || m < 0 || n < 0 || k < 8 || (partial == nullptr) == (gated == nullptr)) return TS_ERR_ARG;
  if (m > M_MAX || (k & 7) != 0 || x_stride < k || (x_stride & 7) != 0) return TS_ERR_SHAPE;
  const int total = (k + DEPTH - 1) / DEPTH;
  if (iters_per_split < 1 || splits != (total + iters_per_split - 1) / iters_per_split || splits > 65535)
    return TS_ERR_SHAPE;
  if (gated && (splits != 1 || bias || (n & 1) != 0)) return TS_ERR_ARG;
  uint16_t* gp = (uint16_t*)gated;
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
  const uint16_t* bp = (const uint16_t*)bias;
  if (tile == 2) return launch_tiled<2>(partial, gp, xp, x_stride, wp, bp, m, n, k, iters_per_split, splits, stream);
  if (tile == 4) return launch_tiled<4>(partial, gp, xp, x_stride, wp, bp, m, n, k, iters_per_split, splits, stream);
  if (tile == 5) return launch_tiled<5>(partial, gp, xp, x_stride, wp, bp, m, n, k, iters_per_split, splits, stream);
  if (tile == 8) return launch_tiled_tall<8>(partial, gp, xp, x_stride, wp, bp, m, n, k, iters_per_split, splits, stream);
  return TS_ERR_SHAPE;
}
