// The product of steps with more rows than a decode step has (129 rows and up), tiled through LDS:
//   Y[m][n] = sum over k of X[m][k] * W[n][k]  (+ bias[n])
// bfloat16 activations X [M, K] and weights W [N, K] as the checkpoint stores them (F.linear's
// layout, src/turboserve/engine/model/layers.py:142), 32-bit accumulation on the matrix cores.
// It is gemm_tiled.hip's scheme with taller activation tiles and a grid over them:
//   * a workgroup of 2 x WM wavefronts (WM = 2 or 4) owns NT = 32 TN weight rows (TN = 2, 4 or
//     5) by XROWS = 16 WM MB activation rows (128 or 256) and one range of K, walked 64 deep: both
//     operands travel global memory -> registers (16-byte pieces, eight consecutive threads a
//     row's 128 bytes) -> LDS (two buffers, the pieces of a row swizzled against bank conflicts) ->
//     matrix cores.  The loads
//     of an iteration are issued two iterations ahead into one of two sets of registers, and an
//     iteration's registers go to LDS between the two halves of the iteration before's products,
//     so that a wavefront's LDS writes, LDS reads and matrix instructions overlap; every load is
//     issued on every path (rows beyond N or M repeat the last row, pieces beyond K the row's
//     last piece, cleared on their way into LDS);
//   * a wavefront computes TN x MB tiles of v_mfma_f32_16x16x32_bf16: each weight fragment it
//     reads from LDS serves MB products, each activation fragment TN (at 5 x 8: 13 KB of LDS
//     reads for 40 matrix instructions);
//   * the grid is one-dimensional and numbered so that the workgroups that share a weight tile
//     (the tiles of activation rows over it) run on the same die, one after the other in its
//     dispatch order: consecutive workgroup ids go to the eight dies in turn, so id -> die id % 8,
//     and of a die's ids consecutive ones take the same weight tile's activation tiles.  The
//     weights then come from memory once and from that die's L2 afterwards.
// Results: bfloat16 Y (one range of K; bias added), or 32-bit partial sums [S, M, N] over S
// ranges of K (bias in the first; the consumer adds them up), or, for a gate|up matrix whose rows
// alternate gate, up, silu(gate) * up as bfloat16 [M, N / 2] (one range of K, no bias).
#include "common.hpp"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int DIES = 8;

__device__ __forceinline__ bf16x8 wide_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// WM: wavefronts along the activation rows (the workgroup has 2 WM wavefronts).  DP: k per
// iteration, 64, or 128 for tiles small enough that two buffers still fit LDS (the iterations of
// a few activation rows hold little work, and half as many barriers tell).
template <int TN, int MB, int WM, int DP>
struct WideRegs {
  static constexpr int THREADS = 2 * WM * TS_WAVE;
  static constexpr int LDS_ROW = DP;          // LDS row stride in elements: no padding, the pieces of a row are swizzled
  static constexpr int ROW_PIECES = DP / 8;   // 16-byte pieces of a row of an iteration
  static constexpr int PIECE_ROWS = THREADS / ROW_PIECES;  // rows one pass of the threads covers
  static constexpr int NT = 32 * TN;
  static constexpr int XROWS = 16 * WM * MB;
  static constexpr int W_PIECES = (NT + PIECE_ROWS - 1) / PIECE_ROWS;
  static constexpr int X_PIECES = XROWS / PIECE_ROWS;
  static_assert(XROWS % PIECE_ROWS == 0, "the activation rows are a whole number of passes");
  u32x4 w[W_PIECES];
  u32x4 x[X_PIECES];
};

// out: bfloat16 [m, n] (mode 0), partial: float [splits, m, n] (mode 1), out: bfloat16 [m, n / 2] (mode 2).
template <int TN, int MB, int WM, int DP, int MODE, bool ONCE>
__global__ void __launch_bounds__(2 * WM * TS_WAVE)
gemm_wide_kernel(float* __restrict__ partial, uint16_t* __restrict__ out, const uint16_t* __restrict__ x, long x_stride,
                 const uint16_t* __restrict__ w, const uint16_t* __restrict__ bias, int m, int n, int k,
                 int iters_per_split, int splits, int n_tiles, int m_tiles) {
  typedef WideRegs<TN, MB, WM, DP> Regs;
  constexpr int NT = Regs::NT;
  constexpr int XROWS = Regs::XROWS;
  constexpr int W_PIECE_ROWS = Regs::PIECE_ROWS;
  constexpr int W_DEPTH = DP;
  constexpr int W_LDS_ROW = Regs::LDS_ROW;
  constexpr int W_ROW_PIECES = Regs::ROW_PIECES;
  constexpr int STAGE = (NT + XROWS) * W_LDS_ROW;  // elements of one LDS buffer: weight rows, then activation rows
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [2][STAGE]
  // Workgroup id -> (weight tile and range of K, tile of activation rows): see the head of the file.
  const int die = blockIdx.x % DIES;
  const int turn = blockIdx.x / DIES;
  const int m_tile = turn % m_tiles;
  const int unit = (turn / m_tiles) * DIES + die;  // weight tile x range of K
  if (unit >= n_tiles * splits) return;            // the whole workgroup leaves together
  const int n_base = (unit % n_tiles) * NT;
  const int split = unit / n_tiles;
  const int m_base = m_tile * XROWS;

  const int tid = threadIdx.x;
  const int lane = tid & (TS_WAVE - 1);
  const int wave = tid / TS_WAVE;
  const int lane16 = lane & 15;
  const int group = lane >> 4;
  const int wave_n = wave / WM;
  const int wave_m = wave % WM;
  const int total = (k + W_DEPTH - 1) / W_DEPTH;
  const int first = split * iters_per_split;
  const int last = min(first + iters_per_split, total);  // exclusive
  if (first >= last) return;

  const uint16_t* wsrc[Regs::W_PIECES];
  const uint16_t* xsrc[Regs::X_PIECES];
  const int piece_k = 8 * (tid % W_ROW_PIECES);
  const int piece_row = tid / W_ROW_PIECES;  // rows advance by W_PIECE_ROWS per i
  // (the last pass of the weight rows may reach past the tile: those pieces repeat the tile's
  // last row and are not staged)
#pragma unroll
  for (int i = 0; i < Regs::W_PIECES; ++i)
    wsrc[i] = w + (size_t)min(n_base + min(piece_row + W_PIECE_ROWS * i, NT - 1), n - 1) * k;
#pragma unroll
  for (int i = 0; i < Regs::X_PIECES; ++i)
    xsrc[i] = x + (size_t)min(m_base + piece_row + W_PIECE_ROWS * i, m - 1) * x_stride;
  // Where a piece lies in its LDS row: piece p of row r at p ^ key(r), key = (r / 2) % 8 for rows of
  // eight pieces (128 bytes: two rows span the 64 banks) and r % 16 for rows of sixteen.  Sixteen
  // lanes that write a row's (or two rows') consecutive pieces, and sixteen lanes that read the
  // same piece of sixteen consecutive rows, then each touch every bank once; with padded rows
  // instead the writes of neighbouring rows overlapped (a third of the LDS cycles of the 256 x 256
  // tile were bank conflicts).  Tiles start at multiples of 16 rows, so a thread's key is constant.
  auto swizzle_key = [](int row) { return W_ROW_PIECES == 8 ? (row >> 1) & 7 : row & 15; };
  const int dst = piece_row * W_LDS_ROW + 8 * ((tid % W_ROW_PIECES) ^ swizzle_key(piece_row));
  static_assert(W_PIECE_ROWS % 16 == 0 && NT % 16 == 0, "a thread's rows differ by multiples of 16");

  auto fetch = [&](Regs& r, int it) {
    const int k0 = min(min(it, last - 1) * W_DEPTH + piece_k, k - 8);
#pragma unroll
    for (int i = 0; i < Regs::X_PIECES; ++i) r.x[i] = *reinterpret_cast<const u32x4*>(xsrc[i] + k0);
#pragma unroll
    for (int i = 0; i < Regs::W_PIECES; ++i)
      r.w[i] = ONCE ? load_once16(wsrc[i] + k0) : *reinterpret_cast<const u32x4*>(wsrc[i] + k0);
  };
  auto stage = [&](const Regs& r, int buf, int it) {
    uint16_t* base = lds + buf * STAGE + dst;
    if ((it + 1) * W_DEPTH <= k) {
#pragma unroll
      for (int i = 0; i < Regs::X_PIECES; ++i)
        *reinterpret_cast<u32x4*>(base + (NT + W_PIECE_ROWS * i) * W_LDS_ROW) = r.x[i];
#pragma unroll
      for (int i = 0; i < Regs::W_PIECES; ++i)
        if (NT % W_PIECE_ROWS == 0 || piece_row + W_PIECE_ROWS * i < NT)
          *reinterpret_cast<u32x4*>(base + W_PIECE_ROWS * i * W_LDS_ROW) = r.w[i];
    } else {  // the last iteration of a K that is no multiple of 64 (or one past the end, never read)
      const bool beyond = it * W_DEPTH + piece_k >= k;
      const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int i = 0; i < Regs::X_PIECES; ++i)
        *reinterpret_cast<u32x4*>(base + (NT + W_PIECE_ROWS * i) * W_LDS_ROW) = beyond ? zero : r.x[i];
#pragma unroll
      for (int i = 0; i < Regs::W_PIECES; ++i)
        if (NT % W_PIECE_ROWS == 0 || piece_row + W_PIECE_ROWS * i < NT)
          *reinterpret_cast<u32x4*>(base + W_PIECE_ROWS * i * W_LDS_ROW) = beyond ? zero : r.w[i];
    }
  };

  f32x4 acc[TN][MB];
#pragma unroll
  for (int a = 0; a < TN; ++a) {
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // The products of the iteration staged in buffer `buf`; between its two halves the registers
  // `next` (iteration `it_next`) go to the other buffer.
  auto multiply = [&](int buf, const Regs& next, int it_next) {
    const uint16_t* base = lds + buf * STAGE + lane16 * W_LDS_ROW;
    const int key = swizzle_key(lane16);
#pragma unroll
    for (int step = 0; step < W_DEPTH / 32; ++step) {
      const int piece = 8 * ((4 * step + group) ^ key);  // this lane's piece of the step, in every row it reads
      u32x4 xf[MB];
#pragma unroll
      for (int b = 0; b < MB; ++b)
        xf[b] = *reinterpret_cast<const u32x4*>(base + (NT + 16 * MB * wave_m + 16 * b) * W_LDS_ROW + piece);
#pragma unroll
      for (int a = 0; a < TN; ++a) {
        const u32x4 wf = *reinterpret_cast<const u32x4*>(base + (wave_n * TN + a) * 16 * W_LDS_ROW + piece);
#pragma unroll
        for (int b = 0; b < MB; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wide_bf16x8(wf), wide_bf16x8(xf[b]), acc[a][b], 0, 0, 0);
      }
      if (step == W_DEPTH / 64 - 1) stage(next, buf ^ 1, it_next);  // between the halves
    }
#ifndef TS_WIDE_NO_SCHED
    // Order asked of the scheduler for the round (one basic block: the loads of the iteration
    // after next, the two halves of the products, the staging between them): a few LDS reads
    // ahead, then per four matrix instructions two LDS reads, an LDS write and a global load.
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int i = 0; i < TN * MB * (W_DEPTH / 32) / 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);  // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // DS read
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // DS write
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM read
    }
#endif
  };

  // Invariant at the top of a round for iteration `it`: LDS buffer 0 (1 in the second half of
  // the loop's body) holds it, complete, behind a barrier; one set of registers holds iteration
  // it + 1, and the other is free for the loads of it + 2.
  Regs r0, r1;
  fetch(r0, first);
  fetch(r1, first + 1);
  stage(r0, 0, first);
  __syncthreads();
  for (int it = first; it < last; it += 2) {
    fetch(r0, it + 2);
    multiply(0, r1, it + 1);
    __syncthreads();
    if (it + 1 >= last) break;
    fetch(r1, it + 3);
    multiply(1, r0, it + 2);
    __syncthreads();
  }

  // acc[a][b][i] = sum for weight row n_base + 16 (wave_n TN + a) + 4 g + i and activation row
  // m_base + 16 MB wave_m + 16 b + lane16.
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
      const int row = m_base + 16 * MB * wave_m + 16 * b + lane16;
      if (row >= m) continue;
      if (MODE == 2) {
        // rows of the matrix alternate gate, up: the lane holds two such pairs (the stand-alone
        // SwiGLU kernel's formula, rounded once)
        const f32x4 s = acc[a][b];
        const float lo = s[0] / (1.f + expf(-s[0])) * s[1];
        const float hi = s[2] / (1.f + expf(-s[2])) * s[3];
        uint16_t* at = out + (size_t)row * (n / 2) + nrow / 2;
        if (nrow + 3 < n) {
          *reinterpret_cast<uint32_t*>(at) =
              (uint32_t)from_float<bf16_t>(lo).bits | ((uint32_t)from_float<bf16_t>(hi).bits << 16);
        } else if (nrow + 1 < n) {
          at[0] = from_float<bf16_t>(lo).bits;
        }
      } else if (MODE == 1) {
        float* at = partial + ((size_t)split * m + row) * n + nrow;
        const f32x4 v = acc[a][b] + bv;
        if (nrow + 3 < n && (n & 3) == 0) {
          *reinterpret_cast<f32x4*>(at) = v;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (nrow + i < n) at[i] = v[i];
        }
      } else {
        uint16_t* at = out + (size_t)row * n + nrow;
        const f32x4 v = acc[a][b] + bv;
        if (nrow + 3 < n && (n & 3) == 0) {
          uint2 packed;
          packed.x = (uint32_t)from_float<bf16_t>(v[0]).bits | ((uint32_t)from_float<bf16_t>(v[1]).bits << 16);
          packed.y = (uint32_t)from_float<bf16_t>(v[2]).bits | ((uint32_t)from_float<bf16_t>(v[3]).bits << 16);
          *reinterpret_cast<uint2*>(at) = packed;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (nrow + i < n) at[i] = from_float<bf16_t>(v[i]).bits;
        }
      }
    }
  }
}

template <int TN, int MB, int WM, int DP, int MODE, bool ONCE>
int launch_wide_kernel(float* partial, uint16_t* out, const uint16_t* x, long x_stride, const uint16_t* w,
                       const uint16_t* bias, int m, int n, int k, int iters_per_split, int splits, hipStream_t stream) {
  typedef WideRegs<TN, MB, WM, DP> Regs;
  constexpr size_t lds_bytes = (size_t)2 * (Regs::NT + Regs::XROWS) * Regs::LDS_ROW * sizeof(uint16_t);
  static_assert(lds_bytes <= 160 * 1024, "two buffers must fit the LDS of a compute unit");
  if (lds_bytes > 48 * 1024) {
    static bool raised = false;  // per process; the attribute belongs to the kernel
    if (!raised) {
      if (hipFuncSetAttribute((const void*)gemm_wide_kernel<TN, MB, WM, DP, MODE, ONCE>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
        return TS_ERR_LAUNCH;
      raised = true;
    }
  }
  const int n_tiles = (n + Regs::NT - 1) / Regs::NT;
  const int m_tiles = (m + Regs::XROWS - 1) / Regs::XROWS;
  const long units = (long)n_tiles * splits;
  const long ids = ((units + DIES - 1) / DIES) * DIES * m_tiles;
  if (ids > 0x7fffffffL) return TS_ERR_SHAPE;
  hipLaunchKernelGGL((gemm_wide_kernel<TN, MB, WM, DP, MODE, ONCE>), dim3((unsigned)ids), dim3(Regs::THREADS), lds_bytes,
                     stream, partial, out, x, x_stride, w, bias, m, n, k, iters_per_split, splits, n_tiles, m_tiles);
  return ts_launch_status();
}

template <int TN, int MB, int WM, int DP>
int launch_wide(int mode, float* partial, uint16_t* out, const uint16_t* x, long x_stride, const uint16_t* w,
                const uint16_t* bias, int m, int n, int k, int iters_per_split, int splits, hipStream_t stream) {
  // One tile of activation rows: every weight is read once, with non-temporal loads; more: the
  // tiles over a weight tile share it through their die's L2.
  const bool once = m <= WideRegs<TN, MB, WM, DP>::XROWS;
#define TS_WIDE_MODE(MODE)                                                                                            \
  return once ? launch_wide_kernel<TN, MB, WM, DP, MODE, true>(partial, out, x, x_stride, w, bias, m, n, k,              \
                                                           iters_per_split, splits, stream)                           \
              : launch_wide_kernel<TN, MB, WM, DP, MODE, false>(partial, out, x, x_stride, w, bias, m, n, k,             \
                                                            iters_per_split, splits, stream)
  if (mode == 0) TS_WIDE_MODE(0);
  if (mode == 1) TS_WIDE_MODE(1);
  TS_WIDE_MODE(2);
#undef TS_WIDE_MODE
}

}  // namespace

// x [m, k] bfloat16 with row stride x_stride; w [n, k] bfloat16 contiguous; bias [n] bfloat16 or
// null; k % 8 == 0.  mode 0: out = bfloat16 [m, n] (splits must be 1); mode 1: partial = float
// [splits, m, n]; mode 2: out = bfloat16 [m, n / 2] = silu(gate) * up for a w whose rows alternate
// gate, up (splits 1, no bias, n even).  depth: k per iteration, 64 or (tiles of 64 activation rows
// only) 128; iters_per_split iterations of `depth` of k go to each of `splits` =
// ceil(ceil(k / depth) / iters_per_split) ranges.  tile: 2, 4, 5 or (with 8 wavefronts and 256 activation rows) 8 (64, 128, 160 or 256
// weight rows a workgroup); x_rows: 128 or 256 (with 8 wavefronts also 64) activation rows a workgroup; waves: 4 or 8
// wavefronts a workgroup (two, or four, along the activation rows).
extern "C" int ts_gemm_wide(float* partial, void* out, const void* x, long x_stride, const void* w, const void* bias,
                            int m, int n, int k, int iters_per_split, int splits, int tile, int x_rows, int waves,
                            int depth, int mode, hipStream_t stream) {
  if (m == 0 || n == 0) return TS_OK;
  if (!x || !w || m < 0 || n < 0 || k < 8 || mode < 0 || mode > 2) return TS_ERR_ARG;
  if ((mode == 1) != (partial != nullptr) || (mode != 1) != (out != nullptr)) return TS_ERR_ARG;
  if ((k & 7) != 0 || x_stride < k || (x_stride & 7) != 0) return TS_ERR_SHAPE;
  if (depth != 64 && depth != 128) return TS_ERR_SHAPE;
  const int total = (k + depth - 1) / depth;
  if (iters_per_split < 1 || splits != (total + iters_per_split - 1) / iters_per_split) return TS_ERR_SHAPE;
  if (mode != 1 && splits != 1) return TS_ERR_ARG;
  if (mode == 2 && (bias || (n & 1) != 0)) return TS_ERR_ARG;
  uint16_t* op = (uint16_t*)out;
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
  const uint16_t* bp = (const uint16_t*)bias;
#define TS_WIDE(TN, MB, WM, DP) \
  return launch_wide<TN, MB, WM, DP>(mode, partial, op, xp, x_stride, wp, bp, m, n, k, iters_per_split, splits, stream)
  if (depth == 128) {  // tiles of 64 activation rows, eight wavefronts
    if (waves == 8 && x_rows == 64) {
      if (tile == 2) TS_WIDE(2, 1, 4, 128);
      if (tile == 4) TS_WIDE(4, 1, 4, 128);
      if (tile == 5) TS_WIDE(5, 1, 4, 128);
    }
    return TS_ERR_SHAPE;
  }
  if (waves == 4 && x_rows == 128) {
    if (tile == 2) TS_WIDE(2, 4, 2, 64);
    if (tile == 4) TS_WIDE(4, 4, 2, 64);
    if (tile == 5) TS_WIDE(5, 4, 2, 64);
  } else if (waves == 4 && x_rows == 256) {
    if (tile == 2) TS_WIDE(2, 8, 2, 64);
    if (tile == 4) TS_WIDE(4, 8, 2, 64);
    if (tile == 5) TS_WIDE(5, 8, 2, 64);
    // (tiles of 256 x 256 on four wavefronts, 128 x 128 outputs each, do not fit the registers
    // beside two sets of staging registers: the compiler spills)
  } else if (waves == 8 && x_rows == 64) {
    if (tile == 2) TS_WIDE(2, 1, 4, 64);
    if (tile == 4) TS_WIDE(4, 1, 4, 64);
    if (tile == 5) TS_WIDE(5, 1, 4, 64);
    if (tile == 8) TS_WIDE(8, 1, 4, 64);
  } else if (waves == 8 && x_rows == 128) {
    if (tile == 2) TS_WIDE(2, 2, 4, 64);
    if (tile == 4) TS_WIDE(4, 2, 4, 64);
    if (tile == 5) TS_WIDE(5, 2, 4, 64);
    if (tile == 8) TS_WIDE(8, 2, 4, 64);
  } else if (waves == 8 && x_rows == 256) {
    if (tile == 2) TS_WIDE(2, 4, 4, 64);
    if (tile == 4) TS_WIDE(4, 4, 4, 64);
    if (tile == 5) TS_WIDE(5, 4, 4, 64);
    if (tile == 8) TS_WIDE(8, 4, 4, 64);
  }
#undef TS_WIDE
  return TS_ERR_SHAPE;
}
