// bfloat16 paged attention on the matrix cores, for one head size (TS_HEAD_DIM, a multiple of 16
// up to 256; the file is compiled once per head size a model needs).
//
// Both kernels compute, for 16 "columns" at a time, S^T = K Q^T (rows: keys, columns: queries)
// with v_mfma_f32_16x16x32_bf16, an online softmax over 32-key windows in the accumulator
// layout, and O^T = V^T P^T with the same instruction.  Two choices make that work without any
// staging through LDS:
//   * value pages are stored transposed ([NB, Hkv, D, BS]), so the A operand of the second
//     product (8 consecutive keys of one head dimension per lane) is one 16-byte load;
//   * the rows of the two 16-key score tiles of a window are assigned to keys so that a lane's
//     8 scores are exactly the 8 keys its B operand of the second product has to hold:
//     row m of tile t  <->  key  window + 8 * (m / 4) + 4 * t + (m % 4).
// Scores, softmax state and output accumulators are 32-bit; probabilities are rounded to
// bfloat16 for the second product.
//
// Decode kernel: the 16 columns are the query heads of one KV head (G of them, the rest
// padding), for one request whose step brings a single token.  The keys lo..ctx-1 are split
// over `splits` wavefronts (flash-decoding); each writes an unnormalised partial (m, l, acc)
// and a second kernel combines them.  Equals the reference's decode kernel
// (src/turboserve/engine/model/triton_attention.py:110-174) and, with a window, keeps only
// the keys p - window + 1 .. p.
//
// Prefill kernel: the 16 columns are 16 consecutive tokens of one request's portion, for one
// query head; up to PF_HEADS heads of the same KV head share each loaded window.  Column j at
// position p_j sees keys lo_j..p_j (src/turboserve/engine/model/attention.py:139-148).
#include "common.hpp"

#ifndef TS_HEAD_DIM
#error "compile with -DTS_HEAD_DIM=<head size>"
#endif
static_assert(TS_HEAD_DIM % 16 == 0 && TS_HEAD_DIM >= 16 && TS_HEAD_DIM <= 256, "head size: 16..256 in steps of 16");

#define TS_CAT2(a, b) a##b
#define TS_CAT(a, b) TS_CAT2(a, b)
#define TS_SYM(name) TS_CAT(name, TS_HEAD_DIM)

namespace {

constexpr int D = TS_HEAD_DIM;
constexpr int NT = D / 16;        // 16-wide tiles of the head dimension (second product)
constexpr int KJ = D / 32;        // 32-deep steps of the first product
constexpr bool KTAIL = (D % 32) != 0;  // one more 16-deep step
constexpr int WINDOW_KEYS = 32;   // keys per iteration
constexpr float LOG2E = 1.4426950408889634f;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

union Frag8 {
  bf16x8 v;
  u32x4 u;
  uint16_t h[8];
};
union Frag4 {
  s16x4 v;
  u32x2 u;
  uint16_t h[4];
};

__device__ __forceinline__ uint16_t bf16_bits(float v) { return from_float<bf16_t>(v).bits; }

// The queries of 16 columns as B operands of the first product: lane l holds, for column
// l % 16, the head dimensions 32 j + 8 (l / 16) .. + 7.
struct QueryFrags {
  Frag8 main[KJ > 0 ? KJ : 1];
  Frag4 tail;
};

__device__ __forceinline__ void load_query(QueryFrags& q, const uint16_t* row, int group) {
#pragma unroll
  for (int j = 0; j < KJ; ++j) {
    if (row) q.main[j].u = *reinterpret_cast<const u32x4*>(row + 32 * j + 8 * group);
    else q.main[j].u = u32x4{0u, 0u, 0u, 0u};
  }
  if (KTAIL) {
    if (row) q.tail.u = *reinterpret_cast<const u32x2*>(row + 32 * KJ + 4 * group);
    else q.tail.u = u32x2{0u, 0u};
  }
}

// One 16-key score tile: S^T[m][col] = sum_d K[key(m)][d] Q[col][d].  `krow` is this lane's key
// row (row m = lane % 16 of the tile) or null when that key is outside the request's range.
__device__ __forceinline__ f32x4 score_tile(const uint16_t* krow, const QueryFrags& q, int group) {
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < KJ; ++j) {
    Frag8 a;
    if (krow) a.u = *reinterpret_cast<const u32x4*>(krow + 32 * j + 8 * group);
    else a.u = u32x4{0u, 0u, 0u, 0u};
    s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, q.main[j].v, s, 0, 0, 0);
  }
  if (KTAIL) {
    Frag4 a;
    if (krow) a.u = *reinterpret_cast<const u32x2*>(krow + 32 * KJ + 4 * group);
    else a.u = u32x2{0u, 0u};
    s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, q.tail.v, s, 0, 0, 0);
  }
  return s;
}

struct PageGeometry {
  const uint16_t* k_pages;
  const uint16_t* v_pages;
  const int* table;  // this request's block table
  int kv_heads;
  int kvh;
  int block_shift;  // log2(block size)
  int block_mask;
};

// Key row pointer: key pages are [NB, Hkv, BS, D].
__device__ __forceinline__ const uint16_t* key_row(const PageGeometry& g, int key) {
  const long long blk = g.table[key >> g.block_shift];
  return g.k_pages + ((blk * g.kv_heads + g.kvh) << g.block_shift) * D + (long long)(key & g.block_mask) * D;
}

// Pointer to the values of 8 consecutive keys (key % 8 == 0) at head dimension 0: value pages
// are [NB, Hkv, D, BS]; dimension d is `d << block_shift` elements further.
__device__ __forceinline__ const uint16_t* value_chunk(const PageGeometry& g, int key) {
  const long long blk = g.table[key >> g.block_shift];
  return g.v_pages + ((blk * g.kv_heads + g.kvh) << g.block_shift) * D + (key & g.block_mask);
}

// Online-softmax state of the lane's column, and the window update shared by both kernels.
struct ColumnState {
  float m;  // running maximum of the scaled scores (log2 domain)
  float l;  // this lane's share of the running sum (summed over lane groups at the end)
  f32x4 acc[NT];
};

__device__ __forceinline__ void init_state(ColumnState& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int n = 0; n < NT; ++n) st.acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// s0 / s1: raw scores of tiles 0 and 1 (lane: column l % 16, keys window + 8 g + 4 t + i).
// `first_valid` .. `last_valid` (inclusive) bound the keys this column may see.
// Returns the probabilities as the B operand of the second product.
__device__ __forceinline__ Frag8 softmax_window(ColumnState& st, f32x4 s0, f32x4 s1, int window_start,
                                                int group, int first_valid, int last_valid,
                                                float scale_log2) {
  float s[8];
  float mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int key = window_start + 8 * group + e;  // e = 4 t + i
    const float raw = (e < 4 ? s0[e] : s1[e - 4]) * scale_log2;
    s[e] = (key >= first_valid && key <= last_valid) ? raw : -INFINITY;
    mx = fmaxf(mx, s[e]);
  }
  mx = fmaxf(mx, __shfl_xor(mx, 16, TS_WAVE));
  mx = fmaxf(mx, __shfl_xor(mx, 32, TS_WAVE));
  const float m_new = fmaxf(st.m, mx);
  Frag8 p;
  if (m_new == -INFINITY) {  // nothing visible to this column so far
    p.u = u32x4{0u, 0u, 0u, 0u};
    return p;
  }
  const float alpha = exp2f(st.m - m_new);  // 0 when st.m is -inf
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float pe = exp2f(s[e] - m_new);  // 0 for masked keys
    sum += pe;
    p.h[e] = bf16_bits(pe);
  }
  st.l = st.l * alpha + sum;
  st.m = m_new;
#pragma unroll
  for (int n = 0; n < NT; ++n) st.acc[n] *= alpha;
  return p;
}

// O^T += V^T P^T for one window.  `vchunk` points at the lane group's 8 keys (dimension 0) or is
// null when the chunk lies wholly outside the request's range; `keep` masks keys of the chunk
// that lie beyond the context (their page bytes are stale).
__device__ __forceinline__ void accumulate_window(ColumnState& st, const uint16_t* vchunk, const Frag8& p,
                                                  int lane16, int block_shift, unsigned keep) {
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    Frag8 a;
    if (vchunk) {
      a.u = *reinterpret_cast<const u32x4*>(vchunk + ((long long)(16 * n + lane16) << block_shift));
      if (keep != 0xffu) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (!((keep >> e) & 1u)) a.h[e] = 0;
      }
    } else {
      a.u = u32x4{0u, 0u, 0u, 0u};
    }
    st.acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, p.v, st.acc[n], 0, 0, 0);
  }
}

// ---------------------------------------------------------------------------------------------
// decode: grid (splits, kv_heads * head_tiles, requests); one wavefront each.
// partial_acc [requests, heads, splits, D] float; partial_ml [requests, heads, splits, 2] float.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(64)
decode_kernel(float* __restrict__ partial_acc, float* __restrict__ partial_ml,
              const uint16_t* __restrict__ q, long q_stride, const uint16_t* __restrict__ k_pages,
              const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table, int table_width,
              const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
              int seq_begin, int heads, int kv_heads, int block_shift, float scale_log2, int window,
              int keys_per_split, int splits) {
  const int lane = threadIdx.x;
  const int lane16 = lane & 15;
  const int group = lane >> 4;
  const int split = blockIdx.x;
  const int gsize = heads / kv_heads;
  const int head_tiles = (gsize + 15) / 16;
  const int kvh = blockIdx.y / head_tiles;
  const int head_in_group = (blockIdx.y % head_tiles) * 16 + lane16;
  const bool head_valid = head_in_group < gsize;
  const int head = kvh * gsize + head_in_group;
  const int seq = seq_begin + blockIdx.z;
  const int ctx = context_lens[seq];
  const int token = query_start_loc[seq];
  const int p = ctx - 1;
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int begin = (lo & ~(WINDOW_KEYS - 1)) + split * keys_per_split;
  const int end = min(begin + keys_per_split, ctx);

  PageGeometry geo{k_pages, v_pages, block_table + (size_t)seq * table_width, kv_heads, kvh, block_shift,
                   (1 << block_shift) - 1};
  QueryFrags qf;
  load_query(qf, head_valid ? q + (size_t)token * q_stride + (size_t)head * D : nullptr, group);
  ColumnState st;
  init_state(st);

  for (int w = begin; w < end; w += WINDOW_KEYS) {
    const int row_key = w + 8 * (lane16 >> 2) + (lane16 & 3);
    const int key0 = row_key, key1 = row_key + 4;
    const f32x4 s0 = score_tile((key0 >= lo && key0 < ctx) ? key_row(geo, key0) : nullptr, qf, group);
    const f32x4 s1 = score_tile((key1 >= lo && key1 < ctx) ? key_row(geo, key1) : nullptr, qf, group);
    const Frag8 pr = softmax_window(st, s0, s1, w, group, lo, p, scale_log2);
    const int chunk = w + 8 * group;
    const bool chunk_live = chunk + 8 > lo && chunk < ctx;
    unsigned keep = 0xffu;
    if (chunk + 8 > ctx) keep = (chunk < ctx) ? ((1u << (ctx - chunk)) - 1u) : 0u;
    accumulate_window(st, chunk_live ? value_chunk(geo, chunk) : nullptr, pr, lane16, block_shift, keep);
  }

  // The lane's column sum lives in four lane groups.
  float l_total = st.l + __shfl_xor(st.l, 16, TS_WAVE);
  l_total += __shfl_xor(l_total, 32, TS_WAVE);
  if (head_valid) {
    const size_t slot = ((size_t)blockIdx.z * heads + head) * splits + split;
    float* acc_out = partial_acc + slot * D;
#pragma unroll
    for (int n = 0; n < NT; ++n)
      *reinterpret_cast<float4*>(acc_out + 16 * n + 4 * group) =
          make_float4(st.acc[n][0], st.acc[n][1], st.acc[n][2], st.acc[n][3]);
    if (group == 0) {
      partial_ml[slot * 2] = st.m;
      partial_ml[slot * 2 + 1] = l_total;
    }
  }
}

// Combine the splits of one (request, head): out = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// grid (requests, heads), D threads.
__global__ void decode_reduce_kernel(uint16_t* __restrict__ out, const float* __restrict__ partial_acc,
                                     const float* __restrict__ partial_ml,
                                     const int* __restrict__ query_start_loc, int seq_begin, int heads,
                                     int splits) {
  const int seq = seq_begin + blockIdx.x;
  const int head = blockIdx.y;
  const int d = threadIdx.x;
  const size_t base = ((size_t)blockIdx.x * heads + head) * splits;
  float m_max = -INFINITY;
  for (int s = 0; s < splits; ++s) m_max = fmaxf(m_max, partial_ml[(base + s) * 2]);
  float num = 0.f, den = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float m = partial_ml[(base + s) * 2];
    if (m == -INFINITY) continue;  // a split past the end of this request's keys
    const float w = exp2f(m - m_max);
    den += partial_ml[(base + s) * 2 + 1] * w;
    num += partial_acc[(base + s) * D + d] * w;
  }
  const int token = query_start_loc[seq];
  out[((size_t)token * heads + head) * D + d] = bf16_bits(num / den);
}

}  // namespace

// Decode attention for the requests seq_begin .. seq_begin + requests - 1 of the step, each of
// which brings one token.  `splits` wavefronts share each request's keys, `keys_per_split`
// (a multiple of 32) each; partial buffers must hold requests * heads * splits entries.
extern "C" int TS_SYM(ts_attention_decode_d)(
    void* out, void* partial_acc, void* partial_ml, const void* q, long q_stride, const void* k_pages,
    const void* v_pages, const int* block_table, int table_width, const int* query_start_loc,
    const int* context_lens, int seq_begin, int requests, int heads, int kv_heads, int block_size,
    float scale, int window, int keys_per_split, int splits, hipStream_t stream) {
  if (requests == 0) return TS_OK;
  if (!out || !partial_acc || !partial_ml || !q || !k_pages || !v_pages || !block_table ||
      !query_start_loc || !context_lens)
    return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0) return TS_ERR_SHAPE;
  if (block_size < 8 || (block_size & (block_size - 1))) return TS_ERR_SHAPE;
  if (keys_per_split < WINDOW_KEYS || keys_per_split % WINDOW_KEYS != 0 || splits < 1) return TS_ERR_SHAPE;
  if (requests > 65535) return TS_ERR_SHAPE;
  int shift = 0;
  while ((1 << shift) < block_size) ++shift;
  const int head_tiles = (heads / kv_heads + 15) / 16;
  if (kv_heads * head_tiles > 65535) return TS_ERR_SHAPE;
  dim3 grid(splits, kv_heads * head_tiles, requests);
  hipLaunchKernelGGL(decode_kernel, grid, dim3(64), 0, stream, (float*)partial_acc, (float*)partial_ml,
                     (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages,
                     block_table, table_width, query_start_loc, context_lens, seq_begin, heads, kv_heads,
                     shift, scale * LOG2E, window, keys_per_split, splits);
  if (hipGetLastError() != hipSuccess) return TS_ERR_LAUNCH;
  hipLaunchKernelGGL(decode_reduce_kernel, dim3(requests, heads), dim3(D), 0, stream, (uint16_t*)out,
                     (const float*)partial_acc, (const float*)partial_ml, query_start_loc, seq_begin, heads,
                     splits);
  return ts_launch_status();
}
