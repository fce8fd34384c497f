// Paged attention for any mix of query lengths, in the storage type's own precision for loads
// and 32-bit everywhere else (scores, softmax state, accumulators).
//
// One wavefront per (token, query head).  The token at absolute position p of request s sees
// the keys lo..p of that request, lo = max(0, p - window + 1) for a windowed layer and 0
// otherwise (src/turboserve/engine/model/attention.py:139-148: keys <= ctx - q_len + j; the
// window bound is this engine's).  Keys and values are read through the request's block table
// from key pages [NB, Hkv, BS, D] and transposed value pages [NB, Hkv, D, BS]; KV head j serves
// query heads j*G .. j*G+G-1
// (attention.py:196-199).  Online softmax over tiles of 64 keys, as the reference's decode
// kernel does over blocks (src/turboserve/engine/model/triton_attention.py:127-166).
//
// This is the kernel of the true 32-bit path and the one every faster kernel is checked
// against: its result for a token is a function of (p, lo, the request's keys) only, so it is
// bitwise independent of how the request was cut into steps and of the batch around it.
#include "common.hpp"

#define ATTN_MAX_DIM 512
#define ATTN_TILE 64

template <typename T>
__global__ void __launch_bounds__(64)
paged_attention_generic_kernel(T* __restrict__ out, const T* __restrict__ q, long q_stride,
                               const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                               const int* __restrict__ block_table, int table_width,
                               const int* __restrict__ token_seq, const int* __restrict__ positions,
                               int heads, int kv_heads, int dim, int block_size, float scale,
                               int window, const float* __restrict__ slopes) {
  __shared__ float qs[ATTN_MAX_DIM];
  __shared__ float ps[ATTN_TILE];
  __shared__ long long rows[ATTN_TILE];  // per key of the tile: offset of its value column

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (heads / kv_heads);
  const int seq = token_seq[t];
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* table = block_table + (size_t)seq * table_width;
  // A position encoding may bias the scores by the distance: + slope[h] * (key - p), in 32-bit.
  const float slope = slopes ? slopes[h] : 0.f;

  const T* qrow = q + (size_t)t * q_stride + (size_t)h * dim;
  for (int d = lane; d < dim; d += ATTN_TILE) qs[d] = to_float(qrow[d]) * scale;
  __syncthreads();

  constexpr int CHUNKS = ATTN_MAX_DIM / ATTN_TILE;
  float acc[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) acc[c] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;

  for (int base = lo; base <= p; base += ATTN_TILE) {
    const int key = base + lane;
    const bool valid = key <= p;
    float score = -INFINITY;
    long long row = 0;
    if (valid) {
      const int blk = table[key / block_size];
      const long long head_base = ((long long)blk * kv_heads + kvh) * block_size * dim;
      row = head_base + (key % block_size);
      const T* krow = k_pages + head_base + (long long)(key % block_size) * dim;
      float s = 0.f;
      for (int d = 0; d < dim; ++d) s = fmaf(qs[d], to_float(krow[d]), s);
      score = slopes ? fmaf(slope, (float)(key - p), s) : s;
    }
    const float m_new = fmaxf(m_run, wave_max(score));
    const float alpha = expf(m_run - m_new);  // 0 on the first tile (m_run = -inf, m_new finite)
    const float prob = valid ? expf(score - m_new) : 0.f;
    l_run = l_run * alpha + wave_sum(prob);
    m_run = m_new;
    __syncthreads();  // the previous tile's readers are done with ps / rows
    ps[lane] = prob;
    rows[lane] = row;
    __syncthreads();
    const int count = (p - base + 1 < ATTN_TILE) ? p - base + 1 : ATTN_TILE;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int d = lane + c * ATTN_TILE;
      if (d < dim) {
        float a = acc[c] * alpha;
        for (int j = 0; j < count; ++j)
          a = fmaf(ps[j], to_float(v_pages[rows[j] + (long long)d * block_size]), a);
        acc[c] = a;
      }
    }
  }

  T* orow = out + ((size_t)t * heads + h) * dim;
  const float inv = 1.f / l_run;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int d = lane + c * ATTN_TILE;
    if (d < dim) orow[d] = from_float<T>(acc[c] * inv);
  }
}

// out [T, Hq, D] contiguous; q rows are q_stride elements apart (the fused projection output).
// slopes [Hq] (32-bit) or null: the score of key j for the query at position p gets
// slopes[h] * (j - p) added.
extern "C" int ts_paged_attention_generic(void* out, const void* q, long q_stride,
                                          const void* k_pages, const void* v_pages,
                                          const int* block_table, int table_width,
                                          const int* token_seq, const int* positions, int tokens,
                                          int heads, int kv_heads, int dim, int block_size,
                                          float scale, int window, const float* slopes, int dtype,
                                          hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !q || !k_pages || !v_pages || !block_table || !token_seq || !positions) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || heads > 65535) return TS_ERR_SHAPE;
  if (dim < 1 || dim > ATTN_MAX_DIM || block_size < 1 || table_width < 1) return TS_ERR_SHAPE;
  dim3 grid(tokens, heads), block(ATTN_TILE);
  if (dtype == TS_F32)
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)q, q_stride, (const float*)k_pages, (const float*)v_pages, block_table, table_width, token_seq, positions, heads, kv_heads, dim, block_size, scale, window, slopes);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table, table_width, token_seq, positions, heads, kv_heads, dim, block_size, scale, window, slopes);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
