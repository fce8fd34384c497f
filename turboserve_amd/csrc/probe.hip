// A kernel that only reads: what the memory gives a given way of walking it, with nothing else
// in the way.  It walks memory as the weight-streaming products do (gemm_tiled.hip): a workgroup
// of 256 threads reads, per iteration, PIECES x 256 pieces of 16 bytes (16 consecutive threads a
// 256-byte run, thread groups of 16 one "row" each, rows advancing by 16 per piece), the loads of
// AHEAD iterations in flight, and the strides between workgroups, iterations, blocks of rows and
// rows are arguments: a matrix as the checkpoint stores it (rows K elements apart), the same bytes
// re-laid so that a workgroup's iteration is one contiguous run, or one run per workgroup.  What
// it read is folded into one word per workgroup so that nothing is optimised away.
#include "common.hpp"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// NT: non-temporal loads (the data is read once and should not displace anything in the caches).
template <bool NT>
__device__ __forceinline__ u32x4 load16(const char* at) {
  const u32x4* p = reinterpret_cast<const u32x4*>(at);
  return NT ? __builtin_nontemporal_load(p) : *p;
}

template <int PIECES, int AHEAD, bool NT>
__global__ void __launch_bounds__(256)
hbm_read_kernel(unsigned int* __restrict__ out, const char* __restrict__ src, int iters, long wg_stride, long it_stride,
                int blk_rows, long blk_stride, long row_stride) {
  const int tid = threadIdx.x;
  const char* base = src + (size_t)blockIdx.x * wg_stride + 16 * (tid & 15);
  long offset[PIECES];
#pragma unroll
  for (int i = 0; i < PIECES; ++i) {
    const int row = (tid >> 4) + 16 * i;
    offset[i] = (long)(row / blk_rows) * blk_stride + (long)(row % blk_rows) * row_stride;
  }
  u32x4 ring[AHEAD][PIECES];
  u32x4 sum = {0u, 0u, 0u, 0u};
  // Every load is issued on every path (iterations past the end repeat the last), as in the
  // products, so the compiler counts the loads in flight.
#pragma unroll
  for (int a = 0; a < AHEAD; ++a) {
    const long it = min(a, iters - 1) * it_stride;
#pragma unroll
    for (int i = 0; i < PIECES; ++i) ring[a][i] = load16<NT>(base + it + offset[i]);
  }
  for (int it = 0; it < iters; it += AHEAD) {
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
#pragma unroll
      for (int i = 0; i < PIECES; ++i) sum ^= ring[a][i];
      const long next = min(it + a + AHEAD, iters - 1) * it_stride;
#pragma unroll
      for (int i = 0; i < PIECES; ++i) ring[a][i] = load16<NT>(base + next + offset[i]);
    }
  }
  unsigned int folded = sum[0] ^ sum[1] ^ sum[2] ^ sum[3];
#pragma unroll
  for (int a = 0; a < AHEAD; ++a)
#pragma unroll
    for (int i = 0; i < PIECES; ++i) folded ^= ring[a][i][0] & 0u;  // the loads in flight at the end are waited for
  if (folded == 0x9e3779b9u || tid == 0) out[blockIdx.x] = folded;
}

template <int PIECES, bool NT>
int launch_read(unsigned int* out, const char* src, int workgroups, int iters, int ahead, long wg_stride, long it_stride,
                int blk_rows, long blk_stride, long row_stride, hipStream_t stream) {
  if (ahead == 1)
    hipLaunchKernelGGL((hbm_read_kernel<PIECES, 1, NT>), dim3(workgroups), dim3(256), 0, stream, out, src, iters, wg_stride,
                       it_stride, blk_rows, blk_stride, row_stride);
  else if (ahead == 2)
    hipLaunchKernelGGL((hbm_read_kernel<PIECES, 2, NT>), dim3(workgroups), dim3(256), 0, stream, out, src, iters, wg_stride,
                       it_stride, blk_rows, blk_stride, row_stride);
  else if (ahead == 4)
    hipLaunchKernelGGL((hbm_read_kernel<PIECES, 4, NT>), dim3(workgroups), dim3(256), 0, stream, out, src, iters, wg_stride,
                       it_stride, blk_rows, blk_stride, row_stride);
  else
    return TS_ERR_SHAPE;
  return ts_launch_status();
}

}  // namespace

// out [workgroups] uint32; src: `bytes` of device memory.  A workgroup w reads, for it in
// 0 .. iters - 1 and row in 0 .. 16 pieces - 1, the 256 bytes at
//   w wg_stride + it it_stride + (row / blk_rows) blk_stride + (row % blk_rows) row_stride
// (byte strides; all multiples of 16).  pieces: 2, 4, 8 or 10 (32, 64, 128 or 160 rows a
// workgroup); ahead: iterations of loads in flight, 1, 2 or 4; non_temporal: loads marked as
// read-once.  Refused unless every read lies inside src.
extern "C" int ts_hbm_read(void* out, const void* src, long bytes, int workgroups, int iters, int pieces, int ahead,
                           long wg_stride, long it_stride, int blk_rows, long blk_stride, long row_stride,
                           int non_temporal, hipStream_t stream) {
  if (!out || !src || workgroups < 1 || iters < 1 || blk_rows < 1) return TS_ERR_ARG;
  if (wg_stride < 0 || it_stride < 0 || blk_stride < 0 || row_stride < 0) return TS_ERR_ARG;
  if ((wg_stride | it_stride | blk_stride | row_stride) & 15) return TS_ERR_SHAPE;
  const long rows = 16L * pieces;
  const long furthest = (workgroups - 1) * wg_stride + (iters - 1) * it_stride + ((rows - 1) / blk_rows) * blk_stride +
                        (long)min((long)blk_rows - 1, rows - 1) * row_stride + 256;
  if (furthest > bytes) return TS_ERR_SHAPE;
  unsigned int* o = (unsigned int*)out;
  const char* s = (const char*)src;
  if (pieces == 2)
    return non_temporal ? launch_read<2, true>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream)
                        : launch_read<2, false>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream);
  if (pieces == 4)
    return non_temporal ? launch_read<4, true>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream)
                        : launch_read<4, false>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream);
  if (pieces == 8)
    return non_temporal ? launch_read<8, true>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream)
                        : launch_read<8, false>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream);
  if (pieces == 10)
    return non_temporal ? launch_read<10, true>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream)
                        : launch_read<10, false>(o, s, workgroups, iters, ahead, wg_stride, it_stride, blk_rows, blk_stride, row_stride, stream);
  return TS_ERR_SHAPE;
}
