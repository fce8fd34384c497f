// bfloat16 paged attention on the matrix cores, for one head size (TS_HEAD_DIM, a multiple of 16
// up to 256; the file is compiled once per head size a model needs).
//
// Both kernels compute, for 16 "columns" at a time, S^T = K Q^T (rows: keys, columns: queries)
// with v_mfma_f32_16x16x32_bf16, an online softmax over 32-key windows in the accumulator
// layout, and O^T = V^T P^T with the same instruction.  Two choices let a wavefront feed the
// matrix cores straight from what it loaded, with no transposition in between:
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
// Prefill kernels: the 16 columns are 16 consecutive tokens of one request's portion, for one
// query head.  Column j at position p_j sees keys lo_j..p_j
// (src/turboserve/engine/model/attention.py:139-148).  With three or more query heads per KV
// head a workgroup of four wavefronts shares every window through LDS (prefill_shared_kernel);
// with fewer, one wavefront serves two heads from registers alone (prefill_kernel).
#include "common.hpp"

#include <type_traits>

#ifndef TS_HEAD_DIM
#error "compile with -DTS_HEAD_DIM=<head size>"
#endif
static_assert(TS_HEAD_DIM % 16 == 0 && TS_HEAD_DIM >= 16 && TS_HEAD_DIM <= 256, "head size: 16..256 in steps of 16");

// Query heads of one KV head that share each loaded window in the prefill kernel, and
// wavefronts per SIMD the register budgets are set for: the largest head sizes need the whole
// register file of a SIMD for one wavefront (accumulators alone are D / 4 registers a head).
#ifndef TS_PREFILL_HEADS
#define TS_PREFILL_HEADS (TS_HEAD_DIM > 128 ? 1 : 2)
#endif
#define TS_WAVES_PER_SIMD (TS_HEAD_DIM > 128 ? 1 : 2)

#define TS_CAT2(a, b) a##b
#define TS_CAT(a, b) TS_CAT2(a, b)
#define TS_SYM(name) TS_CAT(name, TS_HEAD_DIM)

namespace {

constexpr int D = TS_HEAD_DIM;
constexpr int NT = D / 16;        // 16-wide tiles of the head dimension (second product)
constexpr int KJ = D / 32;        // 32-deep steps of the first product
constexpr bool KTAIL = (D % 32) != 0;  // one more step whose upper 16 of 32 are zero
constexpr int WINDOW_KEYS = 32;   // keys per iteration
constexpr float LOG2E = 1.4426950408889634f;
constexpr int DECODE_MAX_SPLITS = 256;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Matrix-core operands are kept as raw 32-bit words (two bfloat16 each) and reinterpreted with
// __builtin_bit_cast where an instruction wants its own vector type; no unions, no aliasing.
typedef u32x4 Frag8;  // 8 bfloat16
typedef u32x2 Frag4;  // 4 bfloat16

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t bf16_bits(float v) { return from_float<bf16_t>(v).bits; }
// Two floats rounded to nearest-even bfloat16 in one word (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}
// 2^x by the hardware instruction alone: results below the smallest normal number flush to
// zero, which is what a softmax weight that small is worth.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Reductions of a column's value over the four lane groups (lanes l, l ^ 16, l ^ 32, l ^ 48)
// with the row-swap instructions of gfx950: no trip through LDS.
__device__ __forceinline__ void swap_rows(float v, bool halves, float& a, float& b) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, v);
  const u32x2 r = halves ? __builtin_amdgcn_permlane32_swap(bits, bits, false, false)
                         : __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  // Elements go through scalars first: __builtin_bit_cast applied to `r[1]` directly reads
  // element 0 with this compiler.
  const uint32_t first = r[0], second = r[1];
  a = __builtin_bit_cast(float, first);
  b = __builtin_bit_cast(float, second);
}
// The larger of two numbers that are known not to be NaN, as the one instruction (fmaxf would
// first rewrite each operand that comes out of a swap, in case it were a signalling NaN).
__device__ __forceinline__ float max_of_numbers(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float groups_max(float v) {
  float a, b;
  swap_rows(v, false, a, b);
  v = max_of_numbers(a, b);
  swap_rows(v, true, a, b);
  return max_of_numbers(a, b);
}
__device__ __forceinline__ float groups_sum(float v) {
  float a, b;
  swap_rows(v, false, a, b);
  v = a + b;
  swap_rows(v, true, a, b);
  return a + b;
}
__device__ __forceinline__ bf16x8 as_bf16x8(Frag8 f) { return __builtin_bit_cast(bf16x8, f); }
__device__ __forceinline__ Frag8 load8(const uint16_t* p) { return *reinterpret_cast<const u32x4*>(p); }

// The queries of 16 columns as B operands of the first product: lane l holds, for column
// l % 16, the head dimensions 32 j + 8 (l / 16) .. + 7.  Only v_mfma_f32_16x16x32_bf16 is
// used: a 16-deep remainder of the head size is padded with zeros to 32 (feeding one accumulator
// from this instruction and then from the 16-deep one, back to back, gave wrong sums in testing
// on gfx950).
struct QueryFrags {
  Frag8 main[KJ > 0 ? KJ : 1];
  Frag8 tail;  // head sizes that are no multiple of 32: the last 16 dimensions, upper half zero
};

__device__ __forceinline__ void load_query(QueryFrags& q, const uint16_t* row, int group) {
#pragma unroll
  for (int j = 0; j < KJ; ++j) q.main[j] = row ? load8(row + 32 * j + 8 * group) : Frag8{0u, 0u, 0u, 0u};
  if (KTAIL) q.tail = (row && group < 2) ? load8(row + 32 * KJ + 8 * group) : Frag8{0u, 0u, 0u, 0u};
}

struct PageGeometry {
  const uint16_t* k_pages;
  const uint16_t* v_pages;
  const int* table;  // this request's block table
  int table_width;
  int kv_heads;
  int kvh;
  int block_shift;  // log2(block size)
  int block_mask;
};

// The pages that hold the keys w .. w + 31 of a 32-aligned window: 32 / block size of them (one
// when a block holds 32 keys or more).  `w` is the same in every lane, so these are scalar
// loads: they do not queue behind the vector loads of the windows in flight, which a per-lane
// table lookup would have to wait for before it could form an address.  Entries past the
// table's width are never selected (the keys they would hold are past the context).
struct WindowPages {
  int page[4];
};

__device__ __forceinline__ WindowPages window_pages(const PageGeometry& g, int w) {
  WindowPages wp;
  const int first = __builtin_amdgcn_readfirstlane(w) >> g.block_shift;
#pragma unroll
  for (int i = 0; i < 4; ++i) wp.page[i] = g.table[min(first + i, g.table_width - 1)];
  return wp;
}

// Page of `key`, a key of the window starting at w (a block of 32 keys or more: always the first).
// The ids are copied to vector registers first (the empty asm pins them there): selecting
// among scalar registers per lane, the compiler builds a tree of divergent branches instead of
// three v_cndmask.
__device__ __forceinline__ long long page_of(const PageGeometry& g, const WindowPages& wp, int w, int key) {
  int p0 = wp.page[0], p1 = wp.page[1], p2 = wp.page[2], p3 = wp.page[3];
  asm("" : "+v"(p0), "+v"(p1), "+v"(p2), "+v"(p3));
  const int i = (key - w) >> g.block_shift;
  const int low = (i & 1) ? p1 : p0;
  const int high = (i & 1) ? p3 : p2;
  return (i & 2) ? high : low;
}

// A key outside lo..last is replaced by the nearest live key of its window (every window that
// is processed holds one): loads stay unconditional and inside live pages, so they can be
// issued windows ahead; what they bring is masked in the softmax.
__device__ __forceinline__ int live_key(int key, int w, int lo, int last) {
  return min(max(key, max(w, lo)), min(w + WINDOW_KEYS - 1, last));
}

// Key row pointer: key pages are [NB, Hkv, BS, D].
__device__ __forceinline__ const uint16_t* key_row(const PageGeometry& g, const WindowPages& wp, int w, int key) {
  const long long blk = page_of(g, wp, w, key);
  return g.k_pages + ((blk * g.kv_heads + g.kvh) << g.block_shift) * D + (long long)(key & g.block_mask) * D;
}

// Pointer to the values of 8 consecutive keys (key % 8 == 0) at head dimension 0: value pages
// are [NB, Hkv, D, BS]; dimension d is `d << block_shift` elements further.
__device__ __forceinline__ const uint16_t* value_chunk(const PageGeometry& g, const WindowPages& wp, int w, int key) {
  const long long blk = page_of(g, wp, w, key);
  return g.v_pages + ((blk * g.kv_heads + g.kvh) << g.block_shift) * D + (key & g.block_mask);
}

// Everything one 32-key window contributes, as matrix-core operands: the lane's two key rows
// (A operands of the score tiles) and its 8-key value chunk for every head-dimension tile.
struct KeyFrags {
  Frag8 k[2][KJ > 0 ? KJ : 1];
  Frag8 ktail[2];
};
struct ValueFrags {
  Frag8 v[NT];
};
struct WindowFrags : KeyFrags, ValueFrags {};

// Issue the loads of window `w` (keys outside lo..last: see live_key).  ONCE: bit 0, the keys,
// bit 1, the values are read with non-temporal loads (by this wavefront alone: a decode step
// reads every cached key once).  A decode step wants that for the values only (DECODE_ONCE): an
// instruction of theirs reads runs of 512 bytes, one of the keys' 64 bytes of each of 16 rows, so
// two instructions share every 128-byte line, and marking those costs more than it gains
// (7B heads, attention and combine, plain / keys / values / both: 8 requests at 8,192 tokens
// 30.7 / 30.5 / 29.3 / 29.5 us, 64 at 8,192 188 / 177 / 172 / 171, 64 at 640 22.8 / 23.4 / 21.8 /
// 23.4).
constexpr int DECODE_ONCE = 2;
template <int ONCE = 0>
__device__ __forceinline__ void load_window(WindowFrags& f, const PageGeometry& g, int w, int lo, int last,
                                            int lane16, int group) {
  auto load8 = [](const uint16_t* p) -> Frag8 { return (ONCE & 1) ? load_once16(p) : *reinterpret_cast<const u32x4*>(p); };
  auto load8v = [](const uint16_t* p) -> Frag8 { return (ONCE & 2) ? load_once16(p) : *reinterpret_cast<const u32x4*>(p); };
  const WindowPages wp = window_pages(g, w);
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key = w + 8 * (lane16 >> 2) + 4 * t + (lane16 & 3);
    const uint16_t* row = key_row(g, wp, w, live_key(key, w, lo, last));
#pragma unroll
    for (int j = 0; j < KJ; ++j) f.k[t][j] = load8(row + 32 * j + 8 * group);
    if (KTAIL) f.ktail[t] = group < 2 ? load8(row + 32 * KJ + 8 * group) : Frag8{0u, 0u, 0u, 0u};
  }
  const int chunk = w + 8 * group;
  const bool live = chunk + 7 >= lo && chunk <= last;
  const uint16_t* vp = value_chunk(g, wp, w, live ? chunk : (live_key(chunk, w, lo, last) & ~7));
#pragma unroll
  for (int n = 0; n < NT; ++n)
    f.v[n] = load8v(vp + ((long long)(16 * n + lane16) << g.block_shift));
}

// Values of keys beyond `last` are whatever an earlier owner of the page left: clear them, so
// that a stale non-finite value cannot meet a zero probability.  Needed only for a window that
// is not wholly inside lo..last.
__device__ __forceinline__ void clear_stale_values(WindowFrags& f, int w, int lo, int last, int group) {
  const int chunk = w + 8 * group;
  const bool live = chunk + 7 >= lo && chunk <= last;
  // Word i of a fragment holds keys chunk + 2 i (low half) and chunk + 2 i + 1 (high half).
  uint32_t keep[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t low = (live && chunk + 2 * i <= last) ? 0x0000ffffu : 0u;
    const uint32_t high = (live && chunk + 2 * i + 1 <= last) ? 0xffff0000u : 0u;
    keep[i] = low | high;
  }
#pragma unroll
  for (int n = 0; n < NT; ++n) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f.v[n][i] &= keep[i];
  }
}

// S^T tile t of the window for the 16 columns whose queries are in `q`.
__device__ __forceinline__ f32x4 score_tile(const KeyFrags& f, int t, const QueryFrags& q) {
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < KJ; ++j)
    s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(f.k[t][j]), as_bf16x8(q.main[j]), s, 0, 0, 0);
  if (KTAIL) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(f.ktail[t]), as_bf16x8(q.tail), s, 0, 0, 0);
  return s;
}

// Online-softmax state of the lane's column.
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

// The softmax step of one window for one set of 16 columns, from the two score tiles: updates
// the running maximum and sum, returns the probabilities as the B operand of the second
// product and the factor the accumulators must be scaled by first.  With MASKED the lane's
// column sees only the keys first_valid..last_valid (inclusive); without, the caller vouches
// that every key of the window is visible to every column of the wavefront.
template <bool MASKED>
__device__ __forceinline__ Frag8 softmax_window(ColumnState& st, const f32x4 s0, const f32x4 s1, int w, int group,
                                                int first_valid, int last_valid, float scale_log2, float& alpha) {
  float s[8];  // unscaled scores; e = 4 t + i is row 4 g + i of tile t
  float mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float raw = e < 4 ? s0[e & 3] : s1[e & 3];
    if (MASKED) {
      const int key = w + 8 * group + e;
      s[e] = (key >= first_valid && key <= last_valid) ? raw : -INFINITY;
    } else {
      s[e] = raw;
    }
    mx = fmaxf(mx, s[e]);
  }
  mx = groups_max(mx) * scale_log2;  // the scale is positive: the maximum commutes with it
  const float m_new = fmaxf(st.m, mx);
  // Nothing visible to this column so far: keep the state, contribute zeros.
  const float m_use = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
  alpha = fast_exp2(st.m - m_use);  // 0 when st.m is -inf
  float pe[8];
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    pe[e] = fast_exp2(fmaf(s[e], scale_log2, -m_use));  // 0 for masked keys
    sum += pe[e];
  }
  st.l = st.l * alpha + sum;
  st.m = m_new;
  return Frag8{pack2(pe[0], pe[1]), pack2(pe[2], pe[3]), pack2(pe[4], pe[5]), pack2(pe[6], pe[7])};
}

// O^T = alpha O^T + V^T P^T.  Once a column's maximum has settled, alpha is exactly 1: the
// rescaling is skipped when that holds for the whole wavefront.
__device__ __forceinline__ void accumulate(ColumnState& st, const ValueFrags& f, const Frag8 p, float alpha) {
  if (__any(alpha != 1.f)) {
#pragma unroll
    for (int n = 0; n < NT; ++n) st.acc[n] *= alpha;
  }
#pragma unroll
  for (int n = 0; n < NT; ++n)
    st.acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(f.v[n]), as_bf16x8(p), st.acc[n], 0, 0, 0);
}

// One window for one set of 16 columns: scores, online softmax, O^T += V^T P^T.
template <bool MASKED>
__device__ __forceinline__ void attend_window(ColumnState& st, const WindowFrags& f, const QueryFrags& q, int w,
                                              int group, int first_valid, int last_valid, float scale_log2) {
  const f32x4 s0 = score_tile(f, 0, q);
  const f32x4 s1 = score_tile(f, 1, q);
  float alpha;
  const Frag8 p = softmax_window<MASKED>(st, s0, s1, w, group, first_valid, last_valid, scale_log2, alpha);
  accumulate(st, f, p, alpha);
}

// Dispatch on a wavefront-uniform flag: `interior` windows need no masks.
__device__ __forceinline__ void attend(ColumnState& st, const WindowFrags& f, const QueryFrags& q, int w, int group,
                                       int first_valid, int last_valid, float scale_log2, bool interior) {
  if (interior)
    attend_window<false>(st, f, q, w, group, first_valid, last_valid, scale_log2);
  else
    attend_window<true>(st, f, q, w, group, first_valid, last_valid, scale_log2);
}

// Sum of the lane's column over the four lane groups.
__device__ __forceinline__ float column_sum(float l) { return groups_sum(l); }

// ---------------------------------------------------------------------------------------------
// decode: grid (splits, kv_heads * head_tiles, requests); one wavefront each.
// partial_acc [requests, heads, splits, D] float; partial_ml [requests, heads, splits, 2] float.
// ---------------------------------------------------------------------------------------------
template <int ONCE>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(TS_WAVES_PER_SIMD, TS_WAVES_PER_SIMD)))
decode_kernel(float* __restrict__ partial_acc, float* __restrict__ partial_ml,
              const uint16_t* __restrict__ q, long q_stride, const uint16_t* __restrict__ k_pages,
              const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table, int table_width,
              const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
              int seq_begin, int heads, int kv_heads, int block_shift, float scale_log2, int window,
              int keys_per_split, int splits, const int* __restrict__ max_context) {
  // A recorded launch serves growing contexts: the longest context of the step is then read
  // from device memory and the keys are divided evenly over the fixed number of splits.
  if (max_context) {
    int span = *max_context;
    if (window > 0 && span > window + WINDOW_KEYS - 1) span = window + WINDOW_KEYS - 1;
    const int per = (span + WINDOW_KEYS - 1 + splits - 1) / splits;
    keys_per_split = ((per + WINDOW_KEYS - 1) / WINDOW_KEYS) * WINDOW_KEYS;
  }
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

  PageGeometry geo{k_pages, v_pages, block_table + (size_t)seq * table_width, table_width, kv_heads, kvh, block_shift,
                   (1 << block_shift) - 1};
  ColumnState st;
  init_state(st);

  if (begin < end) {
    QueryFrags qf;
    load_query(qf, head_valid ? q + (size_t)token * q_stride + (size_t)head * D : nullptr, group);
    WindowFrags fa, fb;
    load_window<ONCE>(fa, geo, begin, lo, p, lane16, group);
    int w = begin;
    while (true) {
      if (w + WINDOW_KEYS < end) load_window<ONCE>(fb, geo, w + WINDOW_KEYS, lo, p, lane16, group);
      if (w < lo || w + WINDOW_KEYS > ctx) clear_stale_values(fa, w, lo, p, group);
      attend_window<true>(st, fa, qf, w, group, lo, p, scale_log2);
      w += WINDOW_KEYS;
      if (w >= end) break;
      if (w + WINDOW_KEYS < end) load_window<ONCE>(fa, geo, w + WINDOW_KEYS, lo, p, lane16, group);
      if (w < lo || w + WINDOW_KEYS > ctx) clear_stale_values(fb, w, lo, p, group);
      attend_window<true>(st, fb, qf, w, group, lo, p, scale_log2);
      w += WINDOW_KEYS;
      if (w >= end) break;
    }
  }

  const float l_total = column_sum(st.l);
  if (head_valid) {
    const size_t slot = ((size_t)blockIdx.z * heads + head) * splits + split;
    float* acc_out = partial_acc + slot * D;
#pragma unroll
    for (int n = 0; n < NT; ++n)
      *reinterpret_cast<f32x4*>(acc_out + 16 * n + 4 * group) = st.acc[n];
    if (group == 0) {
      partial_ml[slot * 2] = st.m;
      partial_ml[slot * 2 + 1] = l_total;
    }
  }
}

// Combine the splits of one (request, head): out = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// grid (requests, heads), 256 threads.  Each thread first owns one split (its weight), then the
// threads form 1024 / D groups that share the splits between them, a thread adding up four
// head dimensions (one 16-byte load per split), and the groups' sums meet in LDS.
constexpr int REDUCE_THREADS = 256;
static_assert(DECODE_MAX_SPLITS <= REDUCE_THREADS, "one thread per split in the first phase");

__global__ void __launch_bounds__(REDUCE_THREADS)
decode_reduce_kernel(uint16_t* __restrict__ out, const float* __restrict__ partial_acc,
                     const float* __restrict__ partial_ml, const int* __restrict__ query_start_loc,
                     int seq_begin, int heads, int splits) {
  constexpr int LANES_PER_GROUP = D / 4;
  constexpr int GROUPS = REDUCE_THREADS / LANES_PER_GROUP;
  __shared__ float weights[DECODE_MAX_SPLITS];
  __shared__ float sums[GROUPS][D];
  __shared__ float wave_part[2][REDUCE_THREADS / TS_WAVE];
  const int seq = seq_begin + blockIdx.x;
  const int head = blockIdx.y;
  const int tid = threadIdx.x;
  const int wave = tid / TS_WAVE;
  const size_t base = ((size_t)blockIdx.x * heads + head) * splits;
  const int token = query_start_loc[seq];  // the row of the result; fetched with everything else

  // The first four splits of this thread's group are fetched before anything else: their loads
  // travel while the weights of the splits are worked out, instead of after two barriers.
  const int g = tid / LANES_PER_GROUP;
  const int d4 = 4 * (tid % LANES_PER_GROUP);
  const bool sums_here = g < GROUPS;
  f32x4 part[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int sp = g + j * GROUPS;
    part[j] = *reinterpret_cast<const f32x4*>(partial_acc + (base + ((sums_here && sp < splits) ? sp : 0)) * D + d4);
  }

  const bool owns = tid < splits;
  const float m = owns ? partial_ml[(base + tid) * 2] : -INFINITY;
  const float l = owns ? partial_ml[(base + tid) * 2 + 1] : 0.f;
  const float wmax = wave_max(m);
  if ((tid & (TS_WAVE - 1)) == 0) wave_part[0][wave] = wmax;
  __syncthreads();
  float m_max = wave_part[0][0];
#pragma unroll
  for (int i = 1; i < REDUCE_THREADS / TS_WAVE; ++i) m_max = fmaxf(m_max, wave_part[0][i]);
  const float wgt = (m == -INFINITY) ? 0.f : exp2f(m - m_max);  // a split past the request's keys
  if (owns) weights[tid] = wgt;
  const float wsum = wave_sum(l * wgt);
  if ((tid & (TS_WAVE - 1)) == 0) wave_part[1][wave] = wsum;
  __syncthreads();
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < REDUCE_THREADS / TS_WAVE; ++i) den += wave_part[1][i];

  if (sums_here) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int sp = g + j * GROUPS;
      if (sp < splits) acc += part[j] * weights[sp];
    }
    // Further splits, four loads at a time, added in split order.
    for (int sp0 = g + 4 * GROUPS; sp0 < splits; sp0 += 4 * GROUPS) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int sp = sp0 + j * GROUPS;
        part[j] = *reinterpret_cast<const f32x4*>(partial_acc + (base + (sp < splits ? sp : sp0)) * D + d4);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int sp = sp0 + j * GROUPS;
        if (sp < splits) acc += part[j] * weights[sp];
      }
    }
    *reinterpret_cast<f32x4*>(&sums[g][d4]) = acc;
  }
  __syncthreads();
  if (tid < D) {
    float num = 0.f;
#pragma unroll
    for (int i = 0; i < GROUPS; ++i) num += sums[i][tid];
    out[((size_t)token * heads + head) * D + tid] = (uint16_t)bf16_bits(num / den);
  }
}

// ---------------------------------------------------------------------------------------------
// prefill: grid (query blocks, kv_heads * head_chunks); one wavefront handles 16 consecutive
// tokens of one request's portion for up to CT query heads of one KV head.
// blocks [n, 2]: (request index in the step, first row of the block in the step).
// ---------------------------------------------------------------------------------------------
template <int CT>
__global__ void __launch_bounds__(64)
prefill_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ q, long q_stride,
               const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages,
               const int* __restrict__ block_table, int table_width, const int* __restrict__ query_start_loc,
               const int* __restrict__ context_lens, const int* __restrict__ blocks, int heads, int kv_heads,
               int block_shift, float scale_log2, int window) {
  const int lane = threadIdx.x;
  const int lane16 = lane & 15;
  const int group = lane >> 4;
  const int gsize = heads / kv_heads;
  const int head_chunks = (gsize + CT - 1) / CT;
  const int kvh = blockIdx.y / head_chunks;
  const int first_head = (blockIdx.y % head_chunks) * CT;  // within the KV head's group
  const int seq = blocks[2 * blockIdx.x];
  const int row0 = blocks[2 * blockIdx.x + 1];
  const int row_end = query_start_loc[seq + 1];
  const int ctx = context_lens[seq];
  const int pos0 = ctx - (row_end - query_start_loc[seq]) + (row0 - query_start_loc[seq]);  // position of row0
  const int cols = min(16, row_end - row0);
  const bool col_valid = lane16 < cols;
  // An invalid column sees nothing (empty range): its state stays empty and it is never stored.
  const int p_col = col_valid ? pos0 + lane16 : -1;
  const int lo_col = (window > 0 && p_col - window + 1 > 0) ? p_col - window + 1 : 0;
  const int p_last = pos0 + cols - 1;
  const int lo_first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int begin = lo_first & ~(WINDOW_KEYS - 1);
  const int end = p_last + 1;
  // A window every column of the block sees in full: no masks needed.
  const int lo_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
  auto interior = [&](int w) { return cols == 16 && w >= lo_last && w + WINDOW_KEYS - 1 <= pos0; };

  PageGeometry geo{k_pages, v_pages, block_table + (size_t)seq * table_width, table_width, kv_heads, kvh, block_shift,
                   (1 << block_shift) - 1};
  QueryFrags qf[CT];
  ColumnState st[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int hg = first_head + c;
    const bool live = col_valid && hg < gsize;
    load_query(qf[c], live ? q + (size_t)(row0 + lane16) * q_stride + (size_t)(kvh * gsize + hg) * D : nullptr, group);
    init_state(st[c]);
  }

  WindowFrags fa, fb;
  load_window(fa, geo, begin, lo_first, p_last, lane16, group);
  int w = begin;
  while (true) {
    if (w + WINDOW_KEYS < end) load_window(fb, geo, w + WINDOW_KEYS, lo_first, p_last, lane16, group);
    if (w < lo_first || w + WINDOW_KEYS > end) clear_stale_values(fa, w, lo_first, p_last, group);
#pragma unroll
    for (int c = 0; c < CT; ++c) attend(st[c], fa, qf[c], w, group, lo_col, p_col, scale_log2, interior(w));
    w += WINDOW_KEYS;
    if (w >= end) break;
    if (w + WINDOW_KEYS < end) load_window(fa, geo, w + WINDOW_KEYS, lo_first, p_last, lane16, group);
    if (w < lo_first || w + WINDOW_KEYS > end) clear_stale_values(fb, w, lo_first, p_last, group);
#pragma unroll
    for (int c = 0; c < CT; ++c) attend(st[c], fb, qf[c], w, group, lo_col, p_col, scale_log2, interior(w));
    w += WINDOW_KEYS;
    if (w >= end) break;
  }

#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int hg = first_head + c;
    const float l_total = column_sum(st[c].l);
    if (col_valid && hg < gsize) {
      const float inv = 1.f / l_total;
      uint16_t* orow = out + ((size_t)(row0 + lane16) * heads + kvh * gsize + hg) * D;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const f32x4 a = st[c].acc[n] * inv;
        *reinterpret_cast<u32x2*>(orow + 16 * n + 4 * group) = Frag4{pack2(a[0], a[1]), pack2(a[2], a[3])};
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// prefill with shared windows: one workgroup of four wavefronts per (query block, KV head, chunk
// of its query heads).  Each wavefront handles CT query heads for the block's 16 tokens; all of
// them see the same keys, so each 32-key window is fetched from the pages once per workgroup,
// staged in LDS (double-buffered; rows padded and key rows permuted so that the 16 lanes of one
// LDS pass hit distinct banks) and read from there as matrix-core operands by every wavefront.
// Windows travel global memory -> registers (a ring, two or three windows in flight) -> LDS.
// ---------------------------------------------------------------------------------------------
constexpr int K_ROW = D + 8;              // LDS stride of a key row (elements)
constexpr int V_ROW = WINDOW_KEYS + 8;    // LDS stride of a head dimension's 32 values
constexpr int K_TILE = WINDOW_KEYS * K_ROW;
constexpr int V_TILE = D * V_ROW;

// How a workgroup of four wavefronts divides a window between them: wavefront i fetches the
// keys 8 i .. 8 i + 7 (whole rows) and the values of the same eight keys (one 16-byte chunk per
// head dimension).  Eight aligned keys lie in one page, so a wavefront needs one page id per
// window, a scalar load, and its addresses are a scalar base plus a per-lane constant.
constexpr int STAGE_WAVES = 4;
constexpr int KEYS_PER_WAVE = WINDOW_KEYS / STAGE_WAVES;
static_assert(KEYS_PER_WAVE == 8, "a wavefront's keys must be one aligned group of eight");
constexpr int K_WAVE_PIECES = KEYS_PER_WAVE * (D / 8);                   // 16-byte pieces of eight key rows
constexpr int K_EACH = (K_WAVE_PIECES + TS_WAVE - 1) / TS_WAVE;          // per lane
constexpr int V_EACH = (D + TS_WAVE - 1) / TS_WAVE;                      // head dimensions per lane

struct StagedWindow {
  u32x4 k[K_EACH];
  u32x4 v[V_EACH];
};

// Issue the loads of this thread's pieces of window `w`.  Nothing here looks at what the loads
// bring, so they stay in flight until the window is staged.  A window wholly inside lo..last
// takes the scalar path; one at the edge replaces keys outside lo..last (see live_key), whose
// pages it looks up per lane.
__device__ __forceinline__ void fetch_window(StagedWindow& r, const PageGeometry& g, int w, int lo, int last, int wave,
                                             int lane) {
  const int first_key = w + KEYS_PER_WAVE * wave;  // the same in every lane of the wavefront
  if (w >= lo && w + WINDOW_KEYS - 1 <= last) {
    const long long page = g.table[__builtin_amdgcn_readfirstlane(first_key) >> g.block_shift];
    const long long head = ((page * g.kv_heads + g.kvh) << g.block_shift) * D;
    const uint16_t* kbase = g.k_pages + head + (long long)(first_key & g.block_mask) * D;
    const uint16_t* vbase = g.v_pages + head + (first_key & g.block_mask);
#pragma unroll
    for (int i = 0; i < K_EACH; ++i) {
      const int piece = min(lane + i * TS_WAVE, K_WAVE_PIECES - 1);  // spare lanes repeat the last piece
      r.k[i] = load8(kbase + 8 * piece);                             // eight rows of D are contiguous
    }
#pragma unroll
    for (int i = 0; i < V_EACH; ++i) {
      const int d = min(lane + i * TS_WAVE, D - 1);
      r.v[i] = load8(vbase + ((long long)d << g.block_shift));
    }
  } else {
#pragma unroll
    for (int i = 0; i < K_EACH; ++i) {
      const int piece = min(lane + i * TS_WAVE, K_WAVE_PIECES - 1);
      const int key = live_key(first_key + piece / (D / 8), w, lo, last);
      const long long page = g.table[key >> g.block_shift];
      r.k[i] = load8(g.k_pages + ((page * g.kv_heads + g.kvh) << g.block_shift) * D +
                     (long long)(key & g.block_mask) * D + 8 * (piece % (D / 8)));
    }
    const bool live = first_key + 7 >= lo && first_key <= last;
    const int chunk = live ? first_key : (live_key(first_key, w, lo, last) & ~7);
    const long long page = g.table[chunk >> g.block_shift];
    const uint16_t* vbase = g.v_pages + ((page * g.kv_heads + g.kvh) << g.block_shift) * D + (chunk & g.block_mask);
#pragma unroll
    for (int i = 0; i < V_EACH; ++i) {
      const int d = min(lane + i * TS_WAVE, D - 1);
      r.v[i] = load8(vbase + ((long long)d << g.block_shift));
    }
  }
}

// Write the fetched window `w` to LDS.  Values of keys outside lo..last are whatever an earlier
// owner of the page left: they are cleared here, so that a stale non-finite value cannot meet a
// zero probability (only a window that is not wholly inside lo..last needs it).
// Row of the 32-row score tile (v_mfma_f32_32x32x16_bf16) that holds key offset ko of a window.
// The accumulator gives lane half h (lanes 32 h .. 32 h + 31) the rows 8 a + 4 h + b in register
// 4 a + b; as B operand of the second product the same lane must hold, for the 16-key step s,
// the keys 16 s + 8 h .. + 7.  So registers 0..7 are the keys of step 0 and 8..15 those of step
// 1: key offset 16 (a / 2) + 8 h + 4 (a % 2) + b sits in row 8 a + 4 h + b.
__device__ __forceinline__ int wide_key_row(int ko) {
  return 8 * (2 * (ko >> 4) + ((ko >> 2) & 1)) + 4 * ((ko >> 3) & 1) + (ko & 3);
}

template <bool WIDE = false>
__device__ __forceinline__ void stage_window(uint16_t* ks, uint16_t* vs, const StagedWindow& r, int w, int lo, int last,
                                             int wave, int lane) {
#pragma unroll
  for (int i = 0; i < K_EACH; ++i) {
    const int piece = lane + i * TS_WAVE;
    if (piece < K_WAVE_PIECES) {
      // Key offset ko of the window goes to the row the score tiles read it from: tile
      // t = (ko / 4) % 2, row m = 4 (ko / 8) + ko % 4, stored at 16 t + m, so that the 16 lanes
      // of an LDS pass read 16 consecutive rows (distinct banks with the padded stride).
      const int ko = KEYS_PER_WAVE * wave + piece / (D / 8);
      const int slot = WIDE ? wide_key_row(ko) : 16 * ((ko >> 2) & 1) + ((ko >> 3) << 2) + (ko & 3);
      *reinterpret_cast<u32x4*>(ks + slot * K_ROW + 8 * (piece % (D / 8))) = r.k[i];
    }
  }
  const int chunk = w + KEYS_PER_WAVE * wave;
  const bool edge = w < lo || w + WINDOW_KEYS - 1 > last;
#pragma unroll
  for (int i = 0; i < V_EACH; ++i) {
    const int d = lane + i * TS_WAVE;
    if (d >= D) continue;
    u32x4 value = r.v[i];
    if (edge) {
      const bool live = chunk + 7 >= lo && chunk <= last;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t low = (live && chunk + 2 * e <= last) ? 0x0000ffffu : 0u;
        const uint32_t high = (live && chunk + 2 * e + 1 <= last) ? 0xffff0000u : 0u;
        value[e] &= low | high;
      }
    }
    *reinterpret_cast<u32x4*>(vs + d * V_ROW + KEYS_PER_WAVE * wave) = value;
  }
}

// The lane's operands of the staged window, in the layout load_window gives.
__device__ __forceinline__ void read_keys(KeyFrags& f, const uint16_t* ks, int lane16, int group) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const uint16_t* row = ks + (16 * t + lane16) * K_ROW;
#pragma unroll
    for (int j = 0; j < KJ; ++j) f.k[t][j] = load8(row + 32 * j + 8 * group);
    if (KTAIL) f.ktail[t] = group < 2 ? load8(row + 32 * KJ + 8 * group) : Frag8{0u, 0u, 0u, 0u};
  }
}
__device__ __forceinline__ void read_values(ValueFrags& f, const uint16_t* vs, int lane16, int group) {
#pragma unroll
  for (int n = 0; n < NT; ++n) f.v[n] = load8(vs + (16 * n + lane16) * V_ROW + 8 * group);
}

template <int CT>
__global__ void __launch_bounds__(STAGE_WAVES * TS_WAVE) __attribute__((amdgpu_waves_per_eu(TS_WAVES_PER_SIMD, TS_WAVES_PER_SIMD)))
prefill_shared_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ q, long q_stride,
                      const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages,
                      const int* __restrict__ block_table, int table_width, const int* __restrict__ query_start_loc,
                      const int* __restrict__ context_lens, const int* __restrict__ blocks, int num_blocks,
                      int pair_blocks, int heads, int kv_heads, int block_shift, float scale_log2, int window) {
  extern __shared__ __attribute__((aligned(16))) uint16_t staged[];  // [2][K_TILE] then [2][V_TILE]
  uint16_t* ks = staged;
  uint16_t* vs = staged + 2 * K_TILE;
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = threadIdx.x / TS_WAVE;
  const int lane16 = lane & 15;
  const int group = lane >> 4;
  const int gsize = heads / kv_heads;
  constexpr int HW = STAGE_WAVES;
  const int head_chunks = (gsize + HW * CT - 1) / (HW * CT);
  // Workgroup id -> (block, KV head and chunk of its query heads), the latter fastest.  Blocks
  // come heaviest first.  With pair_blocks (the host sets it when all workgroups are resident
  // at once, two per compute unit) the second half of the grid walks the lighter half of the
  // blocks backwards, so that the two workgroups a compute unit is handed in turn, i and
  // i + n / 2, are a heavy and a light one.
  const int lanes_y = kv_heads * head_chunks;
  const int y = blockIdx.x % lanes_y;
  int block = blockIdx.x / lanes_y;
  if (pair_blocks && block >= (num_blocks + 1) / 2) block = num_blocks - 1 - (block - (num_blocks + 1) / 2);
  const int kvh = y / head_chunks;
  const int first_head = ((y % head_chunks) * HW + wave) * CT;  // within the KV head's group
  const int seq = blocks[2 * block];
  const int row0 = blocks[2 * block + 1];
  const int row_end = query_start_loc[seq + 1];
  const int ctx = context_lens[seq];
  const int pos0 = ctx - (row_end - query_start_loc[seq]) + (row0 - query_start_loc[seq]);  // position of row0
  const int cols = min(16, row_end - row0);
  const bool col_valid = lane16 < cols;
  const int p_col = col_valid ? pos0 + lane16 : -1;
  const int lo_col = (window > 0 && p_col - window + 1 > 0) ? p_col - window + 1 : 0;
  const int p_last = pos0 + cols - 1;
  const int lo_first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int begin = lo_first & ~(WINDOW_KEYS - 1);
  const int end = p_last + 1;
  // A window every column of the block sees in full: no masks needed.
  const int lo_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
  auto interior = [&](int w) { return cols == 16 && w >= lo_last && w + WINDOW_KEYS - 1 <= pos0; };

  PageGeometry geo{k_pages, v_pages, block_table + (size_t)seq * table_width, table_width, kv_heads, kvh, block_shift,
                   (1 << block_shift) - 1};
  QueryFrags qf[CT];
  ColumnState st[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int hg = first_head + c;
    load_query(qf[c], (col_valid && hg < gsize) ? q + (size_t)(row0 + lane16) * q_stride + (size_t)(kvh * gsize + hg) * D
                                                : nullptr, group);
    init_state(st[c]);
  }
  const bool wave_live = first_head < gsize;

  // Windows travel global memory -> registers -> LDS.  A ring of P register sets keeps the
  // loads of P windows in flight, so a load has P - 1 rounds of computing to arrive in; LDS
  // holds two windows (the one being read, the next being written).
  constexpr int P = (K_EACH + V_EACH) * CT <= 4 ? 3 : 2;
  StagedWindow ring[P];
  // Every round issues its fetch, past the last window too (that window again, dropped): with a
  // fetch that may or may not have been issued the compiler cannot count the loads in flight
  // and waits for all of them before each staging.
  const int last_window = (end - 1) & ~(WINDOW_KEYS - 1);
#pragma unroll
  for (int u = 0; u < P; ++u)
    fetch_window(ring[u], geo, min(begin + u * WINDOW_KEYS, last_window), lo_first, p_last, wave, lane);
  stage_window(ks, vs, ring[0], begin, lo_first, p_last, wave, lane);
  __syncthreads();
  int buf = 0;
  int w = begin;
  while (w < end) {
#pragma unroll
    for (int u = 0; u < P; ++u) {
      // ring[u] held window w, which is staged: refill it with the window P rounds ahead.
      fetch_window(ring[u], geo, min(w + P * WINDOW_KEYS, last_window), lo_first, p_last, wave, lane);
      if (wave_live) {
        // Keys first, values only once the probabilities stand: the two sets of operands are
        // never in registers together.
        Frag8 prob[CT];
        float alpha[CT];
        {
          KeyFrags kf;
          read_keys(kf, ks + buf * K_TILE, lane16, group);
          // One branch for all heads of the wavefront: the masks' comparisons are formed only
          // where a window needs them, and neither path copies its scores to meet the other.
          if (interior(w)) {
#pragma unroll
            for (int c = 0; c < CT; ++c)
              prob[c] = softmax_window<false>(st[c], score_tile(kf, 0, qf[c]), score_tile(kf, 1, qf[c]), w, group,
                                              lo_col, p_col, scale_log2, alpha[c]);
          } else {
#pragma unroll
            for (int c = 0; c < CT; ++c)
              prob[c] = softmax_window<true>(st[c], score_tile(kf, 0, qf[c]), score_tile(kf, 1, qf[c]), w, group,
                                             lo_col, p_col, scale_log2, alpha[c]);
          }
        }
        ValueFrags vf;
        read_values(vf, vs + buf * V_TILE, lane16, group);
#pragma unroll
        for (int c = 0; c < CT; ++c) accumulate(st[c], vf, prob[c], alpha[c]);
      }
      if (w + WINDOW_KEYS < end)  // the other LDS window was last read a round ago
        stage_window(ks + (buf ^ 1) * K_TILE, vs + (buf ^ 1) * V_TILE, ring[(u + 1) % P], w + WINDOW_KEYS, lo_first,
                     p_last, wave, lane);
      __syncthreads();
      buf ^= 1;
      w += WINDOW_KEYS;
      if (w >= end) break;
    }
  }

#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int hg = first_head + c;
    const float l_total = column_sum(st[c].l);
    if (col_valid && hg < gsize) {
      const float inv = 1.f / l_total;
      uint16_t* orow = out + ((size_t)(row0 + lane16) * heads + kvh * gsize + hg) * D;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const f32x4 a = st[c].acc[n] * inv;
        *reinterpret_cast<u32x2*>(orow + 16 * n + 4 * group) = Frag4{pack2(a[0], a[1]), pack2(a[2], a[3])};
      }
    }
  }
}

template <int CT>
static int launch_prefill_shared(hipStream_t stream, uint16_t* out, const uint16_t* q, long q_stride,
                                 const uint16_t* k_pages, const uint16_t* v_pages, const int* block_table,
                                 int table_width, const int* query_start_loc, const int* context_lens,
                                 const int* blocks, int num_blocks, int heads, int kv_heads, int shift,
                                 float scale_log2, int window) {
  constexpr size_t lds = (size_t)2 * (K_TILE + V_TILE) * sizeof(uint16_t);
  static_assert(lds <= 160 * 1024, "the staged windows must fit in LDS");
  if (lds > 48 * 1024) {
    static bool raised = false;  // per process; the attribute belongs to the kernel
    if (!raised) {
      if (hipFuncSetAttribute((const void*)prefill_shared_kernel<CT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds) != hipSuccess)
        return TS_ERR_LAUNCH;
      raised = true;
    }
  }
  constexpr int HW = STAGE_WAVES;
  const int gsize = heads / kv_heads;
  const int chunks = (gsize + HW * CT - 1) / (HW * CT);
  const long long total = (long long)num_blocks * kv_heads * chunks;
  if (total > 0x7fffffffLL) return TS_ERR_SHAPE;
  // Two workgroups fit a compute unit; when the whole grid is resident at once the hardware
  // cannot even out the blocks' unequal lengths by handing out work as units free up, so
  // heavy and light blocks are paired instead (see the kernel).
  static int compute_units = 0;
  if (compute_units == 0) {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return TS_ERR_LAUNCH;
    compute_units = prop.multiProcessorCount;
  }
  const int pair_blocks = total <= 2LL * compute_units ? 1 : 0;
  hipLaunchKernelGGL((prefill_shared_kernel<CT>), dim3((unsigned)total), dim3(HW * TS_WAVE), lds, stream, out, q,
                     q_stride, k_pages, v_pages, block_table, table_width, query_start_loc, context_lens, blocks,
                     num_blocks, pair_blocks, heads, kv_heads, shift, scale_log2, window);
  return ts_launch_status();
}


// ---------------------------------------------------------------------------------------------
// prefill, 32 tokens per wavefront (head sizes 32, 64, 96, 128; three or more query heads per
// KV head): one workgroup per (block of 32 rows, KV head, some of its query heads), one head per
// wavefront: four wavefronts that also fetch the windows, or five to seven and one more that
// does nothing but fetch (see WIDE_PIECES below).  S^T = K Q^T is a 32 x 32 tile of v_mfma_f32_32x32x16_bf16
// (rows: the window's 32 keys, columns: the 32 tokens), O^T = V^T P^T four such tiles.  A column's
// 32 scores lie in two lanes (l and l ^ 32), 16 registers each, so the softmax's maximum and sum
// are taken inside a lane and crossed once; per score it costs under half the vector
// instructions of the 16-column kernels, and a key row read from LDS serves 32 tokens.  Windows
// are staged as in prefill_shared_kernel (the same LDS image but for the order of the key rows,
// see wide_key_row).
// ---------------------------------------------------------------------------------------------
#if TS_HEAD_DIM % 32 == 0 && TS_HEAD_DIM <= 128
#define TS_WIDE_PREFILL 1
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int WIDE_ROWS = 32;
constexpr int KJ16 = D / 16;  // 16-deep steps of the first product
constexpr int NT32 = D / 32;  // 32-wide tiles of the head dimension (second product)

// Keys and values of a window travel separately in this kernel (the keys of a window are needed
// one round before its values), so the fetched pieces are kept apart.
struct StagedKeys {
  u32x4 k[K_EACH];
};
struct StagedValues {
  u32x4 v[V_EACH];
};

// The two halves of fetch_window: this wavefront's eight key rows, or the eight keys' values, of
// window `w` (keys outside lo..last are replaced, see live_key).
// `page` is the page of the wavefront's eight keys of window `w` (page_of_chunk), looked up a round
// earlier so that nothing waits for it here; a window at the edge of lo..last looks its pages up
// per lane instead.
__device__ __forceinline__ int page_of_chunk(const PageGeometry& g, int w, int wave) {
  // Clamped to the row: in a block's last window the chunk may lie past the last page (such a
  // window looks its pages up per lane, so the value is dropped, but the load stays inside).
  return g.table[min(__builtin_amdgcn_readfirstlane(w + KEYS_PER_WAVE * wave) >> g.block_shift, g.table_width - 1)];
}

// A lane's 32-bit offset as the compiler must see it for a load to take a scalar base and this
// offset as they are: widened next to the load.  Widened once before the loop (where the
// compiler would move it, the offset being the same every round) it becomes a 64-bit register
// pair, and every load needs a 64-bit addition first.
__device__ __forceinline__ size_t lane_offset(uint32_t offset) {
  asm volatile("" : "+v"(offset));
  return offset;
}

// Byte address of the first key row (or, for values, of head dimension 0's first value) of the
// chunk of eight keys that begins at `first_key` on page `page`: all of it the same in every lane,
// so it is worked out by the scalar unit, and a lane adds a 32-bit offset of its own.
__device__ __forceinline__ const char* chunk_base(const uint16_t* pages, const PageGeometry& g, long long page,
                                                  int first_key, int key_stride) {
  const long long row = ((page * g.kv_heads + g.kvh) << g.block_shift) * D;
  return reinterpret_cast<const char*>(pages) + 2 * (row + (long long)(first_key & g.block_mask) * key_stride);
}

// INSIDE: the caller knows that the window lies within lo..last, and nothing is tested.
template <bool INSIDE>
__device__ __forceinline__ void fetch_keys(StagedKeys& r, const PageGeometry& g, int w, int lo, int last, int wave,
                                           int lane, int page_id) {
  const int first_key = w + KEYS_PER_WAVE * wave;  // the same in every lane of the wavefront
  if (INSIDE || (w >= lo && w + WINDOW_KEYS - 1 <= last)) {
    const char* kbase = chunk_base(g.k_pages, g, page_id, first_key, D);
#pragma unroll
    for (int i = 0; i < K_EACH; ++i) {
      uint32_t offset = 16u * (uint32_t)min(lane + i * TS_WAVE, K_WAVE_PIECES - 1);  // spare lanes repeat the last piece
      r.k[i] = *reinterpret_cast<const u32x4*>(kbase + lane_offset(offset));
    }
  } else {
#pragma unroll
    for (int i = 0; i < K_EACH; ++i) {
      const int piece = min(lane + i * TS_WAVE, K_WAVE_PIECES - 1);
      const int key = live_key(first_key + piece / (D / 8), w, lo, last);
      const long long page = g.table[key >> g.block_shift];
      r.k[i] = load8(g.k_pages + ((page * g.kv_heads + g.kvh) << g.block_shift) * D +
                     (long long)(key & g.block_mask) * D + 8 * (piece % (D / 8)));
    }
  }
}

template <bool INSIDE>
__device__ __forceinline__ void fetch_values(StagedValues& r, const PageGeometry& g, int w, int lo, int last, int wave,
                                             int lane, int page_id) {
  const int first_key = w + KEYS_PER_WAVE * wave;
  int chunk = first_key;
  long long page = page_id;
  if (!INSIDE && !(w >= lo && w + WINDOW_KEYS - 1 <= last)) {
    const bool live = first_key + 7 >= lo && first_key <= last;
    chunk = __builtin_amdgcn_readfirstlane(live ? first_key : (live_key(first_key, w, lo, last) & ~7));
    page = g.table[chunk >> g.block_shift];
  }
  const char* vbase = chunk_base(g.v_pages, g, page, chunk, 1);
#pragma unroll
  for (int i = 0; i < V_EACH; ++i) {
    const uint32_t offset = 2u * ((uint32_t)min(lane + i * TS_WAVE, D - 1) << g.block_shift);
    r.v[i] = *reinterpret_cast<const u32x4*>(vbase + lane_offset(offset));
  }
}

// The halves of stage_window, keys in the row order of the 32-row score tile (wide_key_row).
__device__ __forceinline__ void stage_keys(uint16_t* ks, const StagedKeys& r, int wave, int lane) {
#pragma unroll
  for (int i = 0; i < K_EACH; ++i) {
    const int piece = lane + i * TS_WAVE;
    if (piece < K_WAVE_PIECES) {
      const int ko = KEYS_PER_WAVE * wave + piece / (D / 8);
      *reinterpret_cast<u32x4*>(ks + wide_key_row(ko) * K_ROW + 8 * (piece % (D / 8))) = r.k[i];
    }
  }
}

template <bool INSIDE>
__device__ __forceinline__ void stage_values(uint16_t* vs, const StagedValues& r, int w, int lo, int last, int wave,
                                             int lane) {
  const int chunk = w + KEYS_PER_WAVE * wave;
  const bool edge = !INSIDE && (w < lo || w + WINDOW_KEYS - 1 > last);
#pragma unroll
  for (int i = 0; i < V_EACH; ++i) {
    const int d = lane + i * TS_WAVE;
    if (d >= D) continue;
    u32x4 value = r.v[i];
    if (edge) {  // stale values of keys outside lo..last are cleared (see stage_window)
      asm volatile("" ::: "memory");  // keeps this a branch, taken by a block's first and last windows only
      const bool live = chunk + 7 >= lo && chunk <= last;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t low = (live && chunk + 2 * e <= last) ? 0x0000ffffu : 0u;
        const uint32_t high = (live && chunk + 2 * e + 1 <= last) ? 0xffff0000u : 0u;
        value[e] &= low | high;
      }
    }
    *reinterpret_cast<u32x4*>(vs + d * V_ROW + KEYS_PER_WAVE * wave) = value;
  }
}

// How far (in powers of two) a column's scores may rise above the reference its probabilities
// are taken against before the reference is moved and the accumulators rescaled.  Probabilities
// then reach 2^8 at most, which 32-bit sums and bfloat16 operands hold as well as values up to 1;
// after a column's first windows its reference hardly ever moves again, and the rescaling of the
// D / 2 accumulator registers is skipped.
constexpr float WIDE_RESCALE_SLACK = 8.f;

// Scores of keys the lane's column must not see become -inf (in place).  Register i of lane
// half h holds the key at offset 16 (i / 8) + 8 h + 4 ((i / 4) % 2) + i % 4 of the window.
__device__ __forceinline__ void wide_mask(f32x16& s, int w, int half, int first_valid, int last_valid) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int key = w + 16 * (i >> 3) + 8 * half + 4 * ((i >> 2) & 1) + (i & 3);
    s[i] = (key >= first_valid && key <= last_valid) ? s[i] : -INFINITY;
  }
}

// S^T of the window staged at `ks` for the wavefront's 32 tokens and its head, as one
// accumulation chain on the matrix cores.
__device__ __forceinline__ void wide_scores(f32x16& s, const uint16_t* ks, const Frag8 (&qf)[KJ16], int col, int half) {
  const uint16_t* krow = ks + col * K_ROW + 8 * half;
#pragma unroll
  for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
  for (int j = 0; j < KJ16; ++j)
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(load8(krow + 16 * j)), as_bf16x8(qf[j]), s, 0, 0, 0);
}

// All four pieces of a window that lies inside lo..last, for the wavefront that feeds a
// workgroup.  Pages hold 16 keys or more there, so two neighbouring pieces lie on one page, next
// to each other: `page[h]` is the page of the window's keys 16 h .. 16 h + 15, and a half costs
// one address worked out by the scalar unit; its loads differ in their constant offsets.
__device__ __forceinline__ void fetch_keys_halves(StagedKeys (&r)[4], const PageGeometry& g, int w, int lane,
                                                  const int (&page)[2]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const char* base = chunk_base(g.k_pages, g, page[h], w + 16 * h, D);
#pragma unroll
    for (int i = 0; i < K_EACH; ++i) {
      const uint32_t offset = 16u * (uint32_t)min(lane + i * TS_WAVE, K_WAVE_PIECES - 1);
      const char* at = base + lane_offset(offset);
      r[2 * h].k[i] = *reinterpret_cast<const u32x4*>(at);
      r[2 * h + 1].k[i] = *reinterpret_cast<const u32x4*>(at + KEYS_PER_WAVE * D * 2);
    }
  }
}

__device__ __forceinline__ void fetch_values_halves(StagedValues (&r)[4], const PageGeometry& g, int w, int lane,
                                                    const int (&page)[2]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const char* base = chunk_base(g.v_pages, g, page[h], w + 16 * h, 1);
#pragma unroll
    for (int i = 0; i < V_EACH; ++i) {
      const uint32_t offset = 2u * ((uint32_t)min(lane + i * TS_WAVE, D - 1) << g.block_shift);
      const char* at = base + lane_offset(offset);
      r[2 * h].v[i] = *reinterpret_cast<const u32x4*>(at);
      r[2 * h + 1].v[i] = *reinterpret_cast<const u32x4*>(at + KEYS_PER_WAVE * 2);
    }
  }
}

// A window is fetched and staged in WINDOW_KEYS / KEYS_PER_WAVE pieces of eight keys.  In the
// self-fed form of the kernel below each of a workgroup's four wavefronts moves one piece beside
// its head's arithmetic.  In the fed form one more wavefront moves all four pieces and does
// nothing else, and up to seven wavefronts of heads do nothing but arithmetic: a wavefront issues
// at most one instruction every four cycles whatever its kind, and the address arithmetic, loads
// and LDS writes of a round cost a self-fed wavefront as much time as its matrix instructions.
// Eight wavefronts of this register size fill a compute unit (two per SIMD).  The fed form
// wants pages of 16 keys or more (see fetch_keys_halves).
constexpr int WIDE_PIECES = WINDOW_KEYS / KEYS_PER_WAVE;
constexpr int FED_MAX_HEADS = 7;
constexpr int FED_MIN_HEADS = 5;  // fewer heads beside the feeder leave SIMDs with one wavefront

template <bool FED>
__global__ void __launch_bounds__((FED ? FED_MAX_HEADS + 1 : STAGE_WAVES) * TS_WAVE)
    __attribute__((amdgpu_waves_per_eu(2, 2)))
prefill_wide_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ q, long q_stride,
                    const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages,
                    const int* __restrict__ block_table, int table_width, const int* __restrict__ query_start_loc,
                    const int* __restrict__ context_lens, const int* __restrict__ blocks, int num_blocks,
                    int pair_blocks, int group_heads, int heads, int kv_heads, int block_shift, float scale_log2,
                    int window, const int* __restrict__ ranges, float* __restrict__ partial_acc,
                    float* __restrict__ partial_ml) {
  extern __shared__ __attribute__((aligned(16))) uint16_t staged[];  // [2][K_TILE] then [2][V_TILE]
  uint16_t* ks = staged;
  uint16_t* vs = staged + 2 * K_TILE;
  const int lane = threadIdx.x & (TS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TS_WAVE);  // known to be the same in every lane
  const int col = lane & 31;
  const int half = lane >> 5;
  const int gsize = heads / kv_heads;
  // group_heads: the heads a workgroup serves, one per wavefront (self-fed: four).
  const int head_chunks = (gsize + group_heads - 1) / group_heads;
  // Workgroup id -> (block, KV head, chunk of its query heads) and the pairing of heavy and
  // light blocks: as in prefill_shared_kernel.
  const int lanes_y = kv_heads * head_chunks;
  const int y = blockIdx.x % lanes_y;
  int block = blockIdx.x / lanes_y;
  if (pair_blocks && block >= (num_blocks + 1) / 2) block = num_blocks - 1 - (block - (num_blocks + 1) / 2);
  const int kvh = y / head_chunks;
  const bool feeder = FED && wave == group_heads;  // the wavefront that only moves windows
  const bool feeds = !FED || feeder;
  const int hg = (y % head_chunks) * group_heads + wave;  // this wavefront's head within the KV head's group
  const bool wave_live = !feeder && hg < gsize;
  const int seq = blocks[2 * block];
  const int row0 = blocks[2 * block + 1];
  const int row_end = query_start_loc[seq + 1];
  const int ctx = context_lens[seq];
  const int pos0 = ctx - (row_end - query_start_loc[seq]) + (row0 - query_start_loc[seq]);  // position of row0
  const int cols = min(WIDE_ROWS, row_end - row0);
  const bool col_valid = col < cols;
  const int p_col = col_valid ? pos0 + col : -1;  // an invalid column sees nothing and is never stored
  const int lo_col = (window > 0 && p_col - window + 1 > 0) ? p_col - window + 1 : 0;
  const int p_last = pos0 + cols - 1;
  const int lo_first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  int begin = lo_first & ~(WINDOW_KEYS - 1);
  int end = p_last + 1;
  // A block whose keys are shared out over several workgroups: this one takes `count` windows
  // from the block's window `first` on and leaves its sums, not yet divided, in slot `slot` for
  // prefill_combine_kernel.  What a column may see is still decided by its own position.
  int slot = -1;
  if (ranges) {
    const int first = ranges[3 * block];
    const int count = ranges[3 * block + 1];
    slot = ranges[3 * block + 2];
    if (count > 0) {
      begin += first * WINDOW_KEYS;
      end = min(end, begin + count * WINDOW_KEYS);
    }
  }
  const int lo_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
  auto interior = [&](int w) { return cols == WIDE_ROWS && w >= lo_last && w + WINDOW_KEYS - 1 <= pos0; };
  if (begin >= end) {
    // A share that lies past the block's keys (no work list of this library's makes one): it
    // has seen nothing, and says so.  The whole workgroup leaves here, before any barrier.
    if (slot >= 0 && wave_live) {
      const size_t entry = ((size_t)slot * heads + kvh * gsize + hg) * WIDE_ROWS + col;
      for (int d = 4 * half; d < D; d += 8) *reinterpret_cast<f32x4*>(partial_acc + entry * D + d) = f32x4{0.f, 0.f, 0.f, 0.f};
      if (half == 0) {
        partial_ml[entry * 2] = -INFINITY;
        partial_ml[entry * 2 + 1] = 0.f;
      }
    }
    return;
  }

  PageGeometry geo{k_pages, v_pages, block_table + (size_t)seq * table_width, table_width, kv_heads, kvh, block_shift,
                   (1 << block_shift) - 1};
  // The queries as B operands: lane holds, for token `col`, head dimensions 16 j + 8 half .. + 7.
  Frag8 qf[KJ16];
  {
    const uint16_t* row = (col_valid && wave_live)
                              ? q + (size_t)(row0 + col) * q_stride + (size_t)(kvh * gsize + hg) * D + 8 * half
                              : nullptr;
#pragma unroll
    for (int j = 0; j < KJ16; ++j) qf[j] = row ? load8(row + 16 * j) : Frag8{0u, 0u, 0u, 0u};
  }
  float m = -INFINITY, l = 0.f;
  f32x16 acc[NT32];
#pragma unroll
  for (int t = 0; t < NT32; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;

  // A software pipeline over the windows W(i) = begin + 32 i.  Round i issues, as one stretch of
  // straight-line code, the products of two other windows beside the softmax of W(i): the
  // scores of W(i + 1) and the accumulation of W(i - 1)'s values with the probabilities of the
  // round before.  The matrix instructions and the vector instructions between them do not
  // depend on each other, so a wavefront keeps both units busy on its own (instructions issue in
  // order: a vector instruction behind a chain of dependent matrix instructions would wait for
  // the whole chain).  Meanwhile the keys of W(i + 2) and the values of W(i), fetched a round
  // ago, go to LDS, and the keys of W(i + 3) and the values of W(i + 1) are asked for.  LDS
  // holds two windows of keys and two of values.  Windows past the last are the last again
  // (loads stay unconditional, see prefill_shared_kernel); their scores are computed and dropped.
  const int rounds = (end - begin + WINDOW_KEYS - 1) / WINDOW_KEYS;
  const int last_window = (end - 1) & ~(WINDOW_KEYS - 1);
  auto window_at = [&](int i) { return min(begin + i * WINDOW_KEYS, last_window); };
  // The pieces this wavefront moves: its own one, or all of them.
  constexpr int MOVED = FED ? WIDE_PIECES : 1;
  auto piece_of = [&](int k) { return FED ? k : wave; };
  StagedKeys kr[2][MOVED];
  StagedValues vr[2][MOVED];
  // The pages of the moved pieces in the windows W(i + 1) .. W(i + 4) of round i: the feeder
  // keeps one per half window (the page of pieces 2 h and 2 h + 1), a self-fed wavefront its piece's.
  constexpr int PAGES = FED ? 2 : 1;
  auto page_piece = [&](int g) { return FED ? 2 * g : wave; };  // a piece that lies on page g of the window
  auto page_index = [&](int k) { return FED ? k / 2 : 0; };     // which of them piece k lies on
  int page1[PAGES], page2[PAGES], page3[PAGES], page4[PAGES];
  if (feeds) {
    int page0[PAGES];
#pragma unroll
    for (int g = 0; g < PAGES; ++g) {
      page0[g] = page_of_chunk(geo, window_at(0), page_piece(g));
      page1[g] = page_of_chunk(geo, window_at(1), page_piece(g));
      page2[g] = page_of_chunk(geo, window_at(2), page_piece(g));
      page3[g] = page_of_chunk(geo, window_at(3), page_piece(g));
      page4[g] = page_of_chunk(geo, window_at(4), page_piece(g));
    }
#pragma unroll
    for (int k = 0; k < MOVED; ++k) {
      const int piece = piece_of(k);
      fetch_keys<false>(kr[0][k], geo, window_at(0), lo_first, p_last, piece, lane, page0[page_index(k)]);
      fetch_keys<false>(kr[1][k], geo, window_at(1), lo_first, p_last, piece, lane, page1[page_index(k)]);
      fetch_values<false>(vr[0][k], geo, window_at(0), lo_first, p_last, piece, lane, page0[page_index(k)]);
    }
  }
  // The value windows start as zeros: the first round multiplies one of them by probabilities
  // that are all zero, and what LDS held before could be anything.
  for (int e = threadIdx.x * 8; e < 2 * V_TILE; e += blockDim.x * 8)
    *reinterpret_cast<u32x4*>(vs + e) = u32x4{0u, 0u, 0u, 0u};
  if (feeds) {
#pragma unroll
    for (int k = 0; k < MOVED; ++k) {
      stage_keys(ks, kr[0][k], piece_of(k), lane);
      stage_keys(ks + K_TILE, kr[1][k], piece_of(k), lane);
      fetch_keys<false>(kr[0][k], geo, window_at(2), lo_first, p_last, piece_of(k), lane, page2[page_index(k)]);
    }
  }
  __syncthreads();
  f32x16 s[2];  // the scores of the round's window and of the next, by parity of the round
  if (!feeder) wide_scores(s[0], ks, qf, col, half);
  __syncthreads();  // round 0 writes the window after next where these scores' keys were
  Frag8 pp0 = {0u, 0u, 0u, 0u}, pp1 = {0u, 0u, 0u, 0u};  // the probabilities of the round before

  // acc += V^T P^T for the value window staged at `vtile`.
  auto accumulate_values = [&](const uint16_t* vtile, const Frag8 p0, const Frag8 p1) __attribute__((always_inline)) {
    const uint16_t* vrow = vtile + col * V_ROW + 8 * half;
#pragma unroll
    for (int t = 0; t < NT32; ++t) {
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(load8(vrow + 32 * t * V_ROW)), as_bf16x8(p0),
                                                        acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(load8(vrow + 32 * t * V_ROW + 16)), as_bf16x8(p1),
                                                        acc[t], 0, 0, 0);
    }
  };

  // (The lambdas are inlined by force: left as functions, everything they capture would live in
  // memory.)
  // Before a window's scores (held in s[A], window at `w`) become probabilities: keys a column
  // must not see are masked, and where some column's largest score rises more than the slack
  // above its reference, the values of the window before are accumulated at once, with the
  // probabilities that belong to the old reference, the reference moves and everything so far is
  // rescaled.  Lanes whose scores stayed below the slack keep their reference (a factor of exactly
  // 1; a column that has seen nothing yet and sees nothing here must not form -inf - -inf).
  auto look = [&](auto parity, auto steady, int w) __attribute__((always_inline)) {
    constexpr int A = decltype(parity)::value;
    constexpr int B = A ^ 1;
    if (!decltype(steady)::value && !interior(w)) {
      asm volatile("" ::: "memory");  // keeps this a branch: as selects it would cost every window 64 instructions
      wide_mask(s[A], w, half, lo_col, p_col);
    }
    // The column's largest score here, over the lane's 16 and those of lane ^ 32
    // (three at a time, as a tree: a chain of eight dependent instructions would be waited for).
    float part[5];
#pragma unroll
    for (int e = 0; e < 5; ++e) part[e] = fmaxf(fmaxf(s[A][3 * e], s[A][3 * e + 1]), s[A][3 * e + 2]);
    float mx = fmaxf(fmaxf(fmaxf(part[0], part[1]), part[2]), fmaxf(fmaxf(part[3], part[4]), s[A][15]));
    float xa, xb;
    swap_rows(mx, true, xa, xb);
    mx = max_of_numbers(xa, xb) * scale_log2;  // the scale is positive: the maximum commutes with it
    const bool moves_up = mx > m + WIDE_RESCALE_SLACK;
    if (__any(moves_up)) {
      accumulate_values(vs + B * V_TILE, pp0, pp1);
      pp0 = pp1 = Frag8{0u, 0u, 0u, 0u};
      const float alpha = moves_up ? fast_exp2(m - mx) : 1.f;  // 0 for a column that had seen nothing
      m = moves_up ? mx : m;
      l *= alpha;
#pragma unroll
      for (int t = 0; t < NT32; ++t) acc[t] *= alpha;
    }
  };
  // One round.  MOVES: the wavefront fetches and stages.  COMPUTES: it has a head.  A self-fed
  // wavefront does both.  STEADY: every window the round touches, W(i) .. W(i + 5), lies whole
  // inside what every column of the block may see, so nothing is tested, clamped or masked.
  auto round = [&](auto parity, auto steady, auto moves, auto computes, int i) __attribute__((always_inline)) {
    constexpr int A = decltype(parity)::value;  // i % 2
    constexpr int B = A ^ 1;
    constexpr bool STEADY = decltype(steady)::value;
    const int w = begin + i * WINDOW_KEYS;
    auto at = [&](int k) { return STEADY ? w + k * WINDOW_KEYS : window_at(i + k); };
    if constexpr (decltype(moves)::value) {
      if constexpr (FED && STEADY) {
        fetch_keys_halves(kr[B], geo, at(3), lane, page3);
        fetch_values_halves(vr[B], geo, at(1), lane, page1);
      } else {
#pragma unroll
        for (int k = 0; k < MOVED; ++k)
          fetch_keys<STEADY>(kr[B][k], geo, at(3), lo_first, p_last, piece_of(k), lane, page3[page_index(k)]);
#pragma unroll
        for (int k = 0; k < MOVED; ++k)
          fetch_values<STEADY>(vr[B][k], geo, at(1), lo_first, p_last, piece_of(k), lane, page1[page_index(k)]);
      }
#pragma unroll
      for (int g = 0; g < PAGES; ++g) {
        page1[g] = page2[g];
        page2[g] = page3[g];
        page3[g] = page4[g];
        page4[g] = page_of_chunk(geo, at(5), page_piece(g));  // asked for now, used a round from now
      }
    }
    if (decltype(computes)::value && wave_live) {
      look(parity, steady, w);
      // From here to the end of the round's products: no branch, so that the compiler may
      // interleave the three independent strands as asked below.  The two products alternate in
      // program order: the scores are one chain of dependent matrix instructions, the values'
      // are D / 32 short ones.
      {
        const uint16_t* krow = ks + B * K_TILE + col * K_ROW + 8 * half;
        const uint16_t* vrow = vs + B * V_TILE + col * V_ROW + 8 * half;
#pragma unroll
        for (int e = 0; e < 16; ++e) s[B][e] = 0.f;
        static_assert(KJ16 == 2 * NT32, "one step of each product per turn");
#pragma unroll
        for (int j = 0; j < KJ16; ++j) {
          s[B] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(load8(krow + 16 * j)), as_bf16x8(qf[j]), s[B], 0, 0, 0);
          acc[j / 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(load8(vrow + 32 * (j / 2) * V_ROW + 16 * (j & 1))),
                                                              as_bf16x8((j & 1) ? pp1 : pp0), acc[j / 2], 0, 0, 0);
        }
      }
      const float m_use = (m == -INFINITY) ? 0.f : m;  // nothing visible so far: contribute zeros
      float sum0 = 0.f, sum1 = 0.f;
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        s[A][e] = fast_exp2(fmaf(s[A][e], scale_log2, -m_use));
        s[A][e + 1] = fast_exp2(fmaf(s[A][e + 1], scale_log2, -m_use));
        sum0 += s[A][e];
        sum1 += s[A][e + 1];
      }
      l += sum0 + sum1;
      pp0 = Frag8{pack2(s[A][0], s[A][1]), pack2(s[A][2], s[A][3]), pack2(s[A][4], s[A][5]), pack2(s[A][6], s[A][7])};
      pp1 = Frag8{pack2(s[A][8], s[A][9]), pack2(s[A][10], s[A][11]), pack2(s[A][12], s[A][13]),
                  pack2(s[A][14], s[A][15])};
      // Order asked of the scheduler: a few LDS reads ahead, then per matrix instruction (which
      // occupies its unit for 32 cycles) one more LDS read and three vector instructions (4 to 8
      // cycles each).
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);  // DS read
#pragma unroll
      for (int k = 0; k < 2 * KJ16; ++k) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        if (k < 2 * KJ16 - 4) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);  // VALU
      }
    }
    if constexpr (decltype(moves)::value) {
#pragma unroll
      for (int k = 0; k < MOVED; ++k) {
        stage_keys(ks + A * K_TILE, kr[A][k], piece_of(k), lane);
        stage_values<STEADY>(vs + A * V_TILE, vr[A][k], at(0), lo_first, p_last, piece_of(k), lane);
      }
    }
    __syncthreads();
  };
  // Rounds steady_from .. steady_to are steady: W(i) begins at or above the lowest key the last
  // column sees, and W(i + 5) ends at or below the first column's own position.  Three loops,
  // so that the steady one is a loop of its own to the compiler: general rounds up to an even
  // round at or past steady_from, steady pairs of rounds, general rounds to the end.
  const int steady_from = (lo_last - begin + WINDOW_KEYS - 1) / WINDOW_KEYS;
  // (a workgroup with a share of the block's windows ends before the block does: its last rounds
  // ask for windows past its share, which exist and are dropped.)
  const int steady_to = cols == WIDE_ROWS ? min((pos0 + 1 - begin) / WINDOW_KEYS - 6, rounds - 1) : -1;
  auto run = [&](auto moves, auto computes) __attribute__((always_inline)) {
    constexpr std::integral_constant<int, 0> even{};
    constexpr std::integral_constant<int, 1> odd{};
    int i = 0;
    for (; i < rounds && i < steady_from; i += 2) {
      round(even, std::false_type{}, moves, computes, i);
      if (i + 1 < rounds) round(odd, std::false_type{}, moves, computes, i + 1);
    }
    for (; i + 1 <= steady_to; i += 2) {
      round(even, std::true_type{}, moves, computes, i);
      round(odd, std::true_type{}, moves, computes, i + 1);
    }
    for (; i < rounds; i += 2) {
      round(even, std::false_type{}, moves, computes, i);
      if (i + 1 < rounds) round(odd, std::false_type{}, moves, computes, i + 1);
    }
  };
  // Every wavefront of the workgroup meets the same barriers, whichever of these it runs.
  if constexpr (!FED) {
    run(std::true_type{}, std::true_type{});
  } else if (feeder) {
    run(std::true_type{}, std::false_type{});
  } else {
    run(std::false_type{}, std::true_type{});
  }
  // The last window's values are still to be accumulated.
  if (wave_live) accumulate_values(vs + ((rounds - 1) & 1) * V_TILE, pp0, pp1);

  float la, lb;
  swap_rows(l, true, la, lb);
  if (slot >= 0) {
    // A share of a block: the sums as they are, with the reference they were taken against.
    // Columns past the block's rows saw nothing (m = -inf, zeros) and are written like the rest.
    if (wave_live) {
      const size_t entry = ((size_t)slot * heads + kvh * gsize + hg) * WIDE_ROWS + col;
      float* arow = partial_acc + entry * D + 4 * half;
#pragma unroll
      for (int t = 0; t < NT32; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a)
          *reinterpret_cast<f32x4*>(arow + 32 * t + 8 * a) =
              f32x4{acc[t][4 * a], acc[t][4 * a + 1], acc[t][4 * a + 2], acc[t][4 * a + 3]};
      if (half == 0) {
        partial_ml[entry * 2] = m;
        partial_ml[entry * 2 + 1] = la + lb;
      }
    }
    return;
  }
  if (col_valid && wave_live) {
    const float inv = 1.f / (la + lb);
    uint16_t* orow = out + ((size_t)(row0 + col) * heads + kvh * gsize + hg) * D + 4 * half;
#pragma unroll
    for (int t = 0; t < NT32; ++t) {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        // registers 4 a .. 4 a + 3 of tile t: head dimensions 32 t + 8 a + 4 half + 0..3
        *reinterpret_cast<u32x2*>(orow + 32 * t + 8 * a) =
            Frag4{pack2(acc[t][4 * a] * inv, acc[t][4 * a + 1] * inv), pack2(acc[t][4 * a + 2] * inv, acc[t][4 * a + 3] * inv)};
      }
    }
  }
}

// The blocks whose keys were shared out: combine[4 c ..] = (first row, rows, first slot, shares)
// of block c, whose shares lie in consecutive slots.  out = sum_s acc_s 2^(m_s - M) / sum_s l_s
// 2^(m_s - M) with M the largest reference among the shares, as in decode_reduce_kernel.
// grid (blocks to combine, heads, 4 groups of 8 rows); a thread takes four head dimensions of one
// row and asks for all of its shares' sums before it adds any (the launch is short and lives on
// how many loads are under way).
constexpr int COMBINE_ROWS = 8;
constexpr int COMBINE_THREADS = COMBINE_ROWS * (D / 4);
constexpr int PREFILL_MAX_SHARES = 16;

__global__ void __launch_bounds__(COMBINE_THREADS)
prefill_combine_kernel(uint16_t* __restrict__ out, const float* __restrict__ partial_acc,
                       const float* __restrict__ partial_ml, const int* __restrict__ combine, int heads) {
  const int row0 = combine[4 * blockIdx.x];
  const int rows = combine[4 * blockIdx.x + 1];
  const int first_slot = combine[4 * blockIdx.x + 2];
  const int shares = min(combine[4 * blockIdx.x + 3], PREFILL_MAX_SHARES);
  const int head = blockIdx.y;
  const int col = COMBINE_ROWS * blockIdx.z + threadIdx.x / (D / 4);
  const int d = 4 * (threadIdx.x % (D / 4));
  if (col >= rows) return;
  const size_t first = ((size_t)first_slot * heads + head) * WIDE_ROWS + col;
  const size_t step = (size_t)heads * WIDE_ROWS;  // from a share's entry to the next share's
  float m[PREFILL_MAX_SHARES], l[PREFILL_MAX_SHARES];
  f32x4 part[PREFILL_MAX_SHARES];
#pragma unroll
  for (int sh = 0; sh < PREFILL_MAX_SHARES; ++sh) {
    m[sh] = -INFINITY;
    l[sh] = 0.f;
    part[sh] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (sh < shares) {
      const size_t entry = first + sh * step;
      m[sh] = partial_ml[entry * 2];
      l[sh] = partial_ml[entry * 2 + 1];
      part[sh] = *reinterpret_cast<const f32x4*>(partial_acc + entry * D + d);
    }
  }
  float m_max = -INFINITY;
#pragma unroll
  for (int sh = 0; sh < PREFILL_MAX_SHARES; ++sh) m_max = fmaxf(m_max, m[sh]);
  float den = 0.f;
  f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int sh = 0; sh < PREFILL_MAX_SHARES; ++sh) {
    const float wgt = (m[sh] == -INFINITY) ? 0.f : exp2f(m[sh] - m_max);  // a share that saw nothing, or none
    den += l[sh] * wgt;
    sum += part[sh] * wgt;
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  *reinterpret_cast<u32x2*>(out + ((size_t)(row0 + col) * heads + head) * D + d) =
      Frag4{pack2(sum[0] * inv, sum[1] * inv), pack2(sum[2] * inv, sum[3] * inv)};
}

static int launch_prefill_wide(hipStream_t stream, uint16_t* out, const uint16_t* q, long q_stride,
                               const uint16_t* k_pages, const uint16_t* v_pages, const int* block_table,
                               int table_width, const int* query_start_loc, const int* context_lens,
                               const int* blocks, int num_blocks, int heads, int kv_heads, int shift,
                               float scale_log2, int window, int max_context, const int* ranges,
                               float* partial_acc, float* partial_ml, const int* combine, int num_combine) {
  constexpr size_t lds = (size_t)2 * (K_TILE + V_TILE) * sizeof(uint16_t);
  static_assert(lds <= 64 * 1024, "two workgroups' staged windows must fit in LDS");
  const int gsize = heads / kv_heads;
  static int compute_units = 0;
  if (compute_units == 0) {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return TS_ERR_LAUNCH;
    compute_units = prop.multiProcessorCount;
  }
  // Fed workgroups take the KV head's query heads in equal shares of at most seven; with fewer
  // than five heads beside the feeder a compute unit would be left half empty, and the self-fed
  // form (two workgroups of four heads a compute unit) does better.  It also does better where
  // its grid fills the device once to twice over at two workgroups a unit and the blocks are of
  // very unequal length, so that a heavy and a light one are paired on each unit (see the kernel),
  // while the fed grid, of one workgroup a unit, would leave units idle behind the heaviest block
  // (a prompt of 2,048 tokens of the 7B shape: 66 against 73 us; at 4,096 tokens fed is ahead, 151
  // against 182 us).  Blocks are of unequal length when no request has a context much longer than
  // what the step brings in all: the longest context is no longer than the step's rows.
  const int fed_chunks = (gsize + FED_MAX_HEADS - 1) / FED_MAX_HEADS;
  const int fed_heads = (gsize + fed_chunks - 1) / fed_chunks;
  const long long self_total = (long long)num_blocks * kv_heads * ((gsize + STAGE_WAVES - 1) / STAGE_WAVES);
  // (A work list with shared-out blocks was balanced for the fed form where the geometry has it.)
  const bool self_fits = !ranges && self_total > compute_units && self_total <= 2LL * compute_units &&
                         max_context > 0 && max_context <= (long long)num_blocks * WIDE_ROWS;
  const bool fed = fed_heads >= FED_MIN_HEADS && shift >= 4 && !self_fits;
  const int group_heads = fed ? fed_heads : STAGE_WAVES;
  const int chunks = (gsize + group_heads - 1) / group_heads;
  const long long total = (long long)num_blocks * kv_heads * chunks;
  if (total > 0x7fffffffLL) return TS_ERR_SHAPE;
  if (fed) {
    // One workgroup fills a compute unit; blocks come heaviest first, so units that finish early
    // take the lighter ones.
    hipLaunchKernelGGL(prefill_wide_kernel<true>, dim3((unsigned)total), dim3((group_heads + 1) * TS_WAVE), lds, stream,
                       out, q, q_stride, k_pages, v_pages, block_table, table_width, query_start_loc, context_lens,
                       blocks, num_blocks, 0, group_heads, heads, kv_heads, shift, scale_log2, window, ranges,
                       partial_acc, partial_ml);
  } else {
    const int pair_blocks = (!ranges && total <= 2LL * compute_units) ? 1 : 0;
    hipLaunchKernelGGL(prefill_wide_kernel<false>, dim3((unsigned)total), dim3(STAGE_WAVES * TS_WAVE), lds, stream, out,
                       q, q_stride, k_pages, v_pages, block_table, table_width, query_start_loc, context_lens, blocks,
                       num_blocks, pair_blocks, group_heads, heads, kv_heads, shift, scale_log2, window, ranges,
                       partial_acc, partial_ml);
  }
  const int status = ts_launch_status();
  if (status != TS_OK || num_combine == 0) return status;
  hipLaunchKernelGGL(prefill_combine_kernel, dim3(num_combine, heads, WIDE_ROWS / COMBINE_ROWS), dim3(COMBINE_THREADS), 0,
                     stream, out, partial_acc, partial_ml, combine, heads);
  return ts_launch_status();
}

// Workgroups a block of the work list becomes for this geometry (KV heads x chunks of their query
// heads) and how many of them a compute unit runs at a time, in the form launch_prefill_wide
// takes for a list with shared-out blocks: what a caller needs to balance such a list.
static void prefill_wide_shape(int heads, int kv_heads, int shift, int* per_block, int* per_unit) {
  const int gsize = heads / kv_heads;
  const int fed_chunks = (gsize + FED_MAX_HEADS - 1) / FED_MAX_HEADS;
  const int fed_heads = (gsize + fed_chunks - 1) / fed_chunks;
  const bool fed = fed_heads >= FED_MIN_HEADS && shift >= 4;
  *per_block = kv_heads * (fed ? fed_chunks : (gsize + STAGE_WAVES - 1) / STAGE_WAVES);
  *per_unit = fed ? 1 : 2;
}
#endif  // wide prefill

}  // namespace

// Decode attention for the requests seq_begin .. seq_begin + requests - 1 of the step, each of
// which brings one token.  `splits` wavefronts share each request's keys, `keys_per_split`
// (a multiple of 32) each; partial buffers must hold requests * heads * splits entries.
// max_context (device, may be null): the step's longest context; when given, keys_per_split is
// derived from it on the device so that `splits * keys_per_split` covers it.
extern "C" int TS_SYM(ts_attention_decode_d)(
    void* out, void* partial_acc, void* partial_ml, const void* q, long q_stride, const void* k_pages,
    const void* v_pages, const int* block_table, int table_width, const int* query_start_loc,
    const int* context_lens, int seq_begin, int requests, int heads, int kv_heads, int block_size,
    float scale, int window, int keys_per_split, int splits, const int* max_context, hipStream_t stream) {
  if (requests == 0) return TS_OK;
  if (!out || !partial_acc || !partial_ml || !q || !k_pages || !v_pages || !block_table ||
      !query_start_loc || !context_lens)
    return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0) return TS_ERR_SHAPE;
  if (block_size < 8 || (block_size & (block_size - 1))) return TS_ERR_SHAPE;
  if (keys_per_split < WINDOW_KEYS || keys_per_split % WINDOW_KEYS != 0 || splits < 1 || splits > DECODE_MAX_SPLITS)
    return TS_ERR_SHAPE;
  if (requests > 65535) return TS_ERR_SHAPE;
  int shift = 0;
  while ((1 << shift) < block_size) ++shift;
  const int head_tiles = (heads / kv_heads + 15) / 16;
  if (kv_heads * head_tiles > 65535) return TS_ERR_SHAPE;
  dim3 grid(splits, kv_heads * head_tiles, requests);
  // The values are read with non-temporal loads, the keys with plain ones (DECODE_ONCE).
  hipLaunchKernelGGL(decode_kernel<DECODE_ONCE>, grid, dim3(64), 0, stream, (float*)partial_acc, (float*)partial_ml,
                     (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages,
                     block_table, table_width, query_start_loc, context_lens, seq_begin, heads, kv_heads,
                     shift, scale * LOG2E, window, keys_per_split, splits, max_context);
  if (hipGetLastError() != hipSuccess) return TS_ERR_LAUNCH;
  hipLaunchKernelGGL(decode_reduce_kernel, dim3(requests, heads), dim3(REDUCE_THREADS), 0, stream, (uint16_t*)out,
                     (const float*)partial_acc, (const float*)partial_ml, query_start_loc, seq_begin, heads,
                     splits);
  return ts_launch_status();
}

// Prefill attention for `num_blocks` blocks of `block_rows` consecutive rows (16 or 32: what
// ts_attention_prefill_rows_d says for the geometry); blocks [num_blocks, 2] holds (request
// index, first row) of each, rows being token rows of the step.  Writes the rows of
// `out [T, heads * D]` the blocks cover.  max_context: the longest context among the requests, or 0
// if the caller does not know it (it only helps to choose a launch plan).
// ranges (may be null; blocks of 32 rows only): [num_blocks, 3] = (first window, windows, slot) of
// each entry of `blocks`.  An entry with slot -1 is a whole block (windows 0: all of them).  The
// others are shares of a block's windows of 32 keys, counted from the block's first window (the
// one that holds the lowest key its first row sees); a block may appear in `blocks` once per share.
// Shares leave their sums in partial_acc [slots, heads, 32, D] and partial_ml [slots, heads, 32, 2]
// (32-bit), and combine [num_combine, 4] = (first row, rows, first slot, shares <= 16) names the
// blocks to put together afterwards, a block's shares lying in consecutive slots.
// Rows per block that ts_attention_prefill_d<D> wants in `blocks` for this geometry.
extern "C" int TS_SYM(ts_attention_prefill_rows_d)(int heads, int kv_heads) {
#ifdef TS_WIDE_PREFILL
  if (kv_heads >= 1 && heads % kv_heads == 0 && heads / kv_heads >= 3) return WIDE_ROWS;
#endif
  (void)heads;
  (void)kv_heads;
  return 16;
}

// For a work list with shares (see ts_attention_prefill_d): the workgroups one entry becomes and
// how many workgroups a compute unit runs at a time; 0, 0 where blocks are not shared out.
extern "C" void TS_SYM(ts_attention_prefill_shape_d)(int heads, int kv_heads, int block_size, int* per_block,
                                                     int* per_unit) {
  *per_block = *per_unit = 0;
#ifdef TS_WIDE_PREFILL
  if (kv_heads < 1 || heads % kv_heads != 0 || heads / kv_heads < 3 || block_size < 8) return;
  int shift = 0;
  while ((1 << shift) < block_size) ++shift;
  prefill_wide_shape(heads, kv_heads, shift, per_block, per_unit);
#endif
}

extern "C" int TS_SYM(ts_attention_prefill_d)(
    void* out, const void* q, long q_stride, const void* k_pages, const void* v_pages, const int* block_table,
    int table_width, const int* query_start_loc, const int* context_lens, const int* blocks, int num_blocks,
    int block_rows, int heads, int kv_heads, int block_size, float scale, int window, int max_context,
    const int* ranges, void* partial_acc, void* partial_ml, const int* combine, int num_combine,
    hipStream_t stream) {
  if (num_blocks == 0) return TS_OK;
  if (!out || !q || !k_pages || !v_pages || !block_table || !query_start_loc || !context_lens || !blocks)
    return TS_ERR_ARG;
  if (ranges ? (!partial_acc || !partial_ml || num_combine < 0 || (num_combine > 0 && !combine)) : num_combine != 0)
    return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0) return TS_ERR_SHAPE;
  if (block_size < 8 || (block_size & (block_size - 1))) return TS_ERR_SHAPE;
  int shift = 0;
  while ((1 << shift) < block_size) ++shift;
  const int gsize = heads / kv_heads;
  if (block_rows != TS_SYM(ts_attention_prefill_rows_d)(heads, kv_heads)) return TS_ERR_ARG;
#ifdef TS_WIDE_PREFILL
  if (gsize >= 3)
    return launch_prefill_wide(stream, (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)k_pages,
                               (const uint16_t*)v_pages, block_table, table_width, query_start_loc, context_lens,
                               blocks, num_blocks, heads, kv_heads, shift, scale * LOG2E, window, max_context, ranges,
                               (float*)partial_acc, (float*)partial_ml, combine, num_combine);
#endif
  if (ranges) return TS_ERR_ARG;  // only blocks of 32 rows are shared out
  // Three or more query heads per KV head: workgroups of four wavefronts, one or two heads each,
  // share every window of keys and values through LDS.
  if (gsize >= 3) {
    if (gsize >= 5)
      return launch_prefill_shared<2>(stream, (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)k_pages,
                                         (const uint16_t*)v_pages, block_table, table_width, query_start_loc,
                                         context_lens, blocks, num_blocks, heads, kv_heads, shift, scale * LOG2E, window);
    return launch_prefill_shared<1>(stream, (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)k_pages,
                                       (const uint16_t*)v_pages, block_table, table_width, query_start_loc,
                                       context_lens, blocks, num_blocks, heads, kv_heads, shift, scale * LOG2E, window);
  }
  constexpr int CT = TS_PREFILL_HEADS;
  const int head_chunks = (gsize + CT - 1) / CT;
  if (kv_heads * head_chunks > 65535) return TS_ERR_SHAPE;
  dim3 grid(num_blocks, kv_heads * head_chunks);
  hipLaunchKernelGGL(prefill_kernel<CT>, grid, dim3(64), 0, stream, (uint16_t*)out, (const uint16_t*)q, q_stride,
                     (const uint16_t*)k_pages, (const uint16_t*)v_pages, block_table, table_width,
                     query_start_loc, context_lens, blocks, heads, kv_heads, shift, scale * LOG2E, window);
  return ts_launch_status();
}
