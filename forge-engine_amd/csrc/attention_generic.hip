// Paged grouped-query attention for a mixed batch, general sizes.
//
// One launch serves every sequence of a step: portions of prompts (many query
// tokens, some context already cached) beside single decoded tokens.  The keys
// and values of the step's own tokens are already in the pages.  For sequence
// s with q_len query tokens and ctx keys in total (ctx_before = ctx - q_len),
// query token i sits at position p = ctx_before + i and reads keys
//   max(0, p - window + 1) .. p        (window <= 0: all keys 0 .. p).
// Query head h reads kv head h / G.  Scores, softmax (online, over key tiles)
// and the weighted sum of values are float32 on the vector ALU; one rounding
// at the store.  This kernel takes any even head size up to 256, any group size,
// any page size, float32 or bfloat16 storage; faster matrix-core kernels cover the
// common bfloat16 shapes.
//
// Work split: block = (row tile, kv head, sequence); a row is one (query
// token, query head of the group) pair, 16 rows per block, so the G heads that
// share a kv head share its key/value tiles.  Thread (r = tid / 16, c = tid % 16)
// owns row r: it computes the scores of keys c, c + 16, ... of the tile and
// output dims c, c + 16, ...; the 16 lanes of a row reduce by shuffles.
// With few blocks and long contexts (a decode step of few sequences) the keys of a
// block's rows are cut into `splits` runs of whole tiles, each walked by a block of its
// own that leaves its running maximum, sum and unnormalised output in scratch; a second
// kernel with the same grid of row tiles merges the runs in order.
#include "common.h"

#define ROWS 16

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float* o) {
    const uint2 v = *(const uint2*)p;
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
};

// four consecutive elements: one vector load where the address allows it (vec), else one by one
template <typename T>
__device__ __forceinline__ void load4(const T* p, bool vec, int count, float* o) {
  if (vec) {
    Vec4<T>::load(p, o);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = i < count ? load_as_float(p + i) : 0.f;
  }
}

template <typename T, int DMAX, int TK, bool FAST_EXP>
__global__ __launch_bounds__(256) void paged_attention_generic_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ key_pages,
    const T* __restrict__ value_pages, T* __restrict__ out, long long out_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int table_stride, int kv_heads, int groups, int head_dim,
    int block_size, int num_blocks, int window, float scale, int min_q_len, int max_q_served,
    int splits, float* __restrict__ part_acc, float* __restrict__ part_ml, int total_tokens) {
  constexpr int KPT = TK / 16;    // keys per thread in a tile
  constexpr int DPT = DMAX / 16;  // output dims per thread
  extern __shared__ float smem[];
  const int D = head_dim;
  const int kstride = D + 1;
  float* Qs = smem;                   // [ROWS][D + 1]
  float* Ks = Qs + ROWS * kstride;    // [TK][D + 1]
  float* Vs = Ks + TK * kstride;      // [TK][D + 1]
  float* Ps = Vs + TK * kstride;      // [ROWS][TK]

  const int seq = blockIdx.z;
  const int hk = blockIdx.y;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int ctx = ctx_len[seq];
  const int ctx_before = ctx - q_len;
  const int rows_total = q_len * groups;
  const int split = blockIdx.x % splits;
  const int row0 = (blockIdx.x / splits) * ROWS;
  if (row0 >= rows_total || ctx_before < 0 || q_len < min_q_len || q_len > max_q_served) return;

  const int tid = threadIdx.x;
  const int r = tid / 16;
  const int c = tid % 16;
  const int my_row = row0 + r;
  const bool row_ok = my_row < rows_total;
  const int my_tok = row_ok ? my_row / groups : 0;
  const int my_g = row_ok ? my_row - my_tok * groups : 0;
  const int my_pos = ctx_before + my_tok;
  const int last_row = min(rows_total, row0 + ROWS) - 1;
  const int pos_min = ctx_before + row0 / groups;
  const int pos_max = ctx_before + last_row / groups;
  const int k_begin = window > 0 ? max(0, pos_min - window + 1) : 0;
  const int k_end = pos_max + 1;  // <= ctx

  // Q tile -> LDS as float32
  const int chunks = (D + 3) / 4;
  const bool vec = D % 4 == 0 && q_stride % 4 == 0 &&
                   ((((uintptr_t)q) | ((uintptr_t)key_pages)) & (4 * sizeof(T) - 1)) == 0;
  for (int e = tid; e < ROWS * chunks; e += 256) {
    const int rr = e / chunks;
    const int d4 = (e - rr * chunks) * 4;
    const int row = row0 + rr;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (row < rows_total) {
      const int tok = row / groups;
      const int g = row - tok * groups;
      load4(q + (size_t)(q0 + tok) * q_stride + (size_t)(hk * groups + g) * D + d4, vec, D - d4, v);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (d4 + i < D) Qs[rr * kstride + d4 + i] = v[i];
  }

  float m = -INFINITY, l = 0.f;
  float acc[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) acc[i] = 0.f;

  const int* table = block_table + (size_t)seq * table_stride;
  // this block's run of key tiles
  const int tile_first = k_begin / TK, tile_last = (k_end + TK - 1) / TK;
  const int tiles_per_split = (tile_last - tile_first + splits - 1) / splits;
  const int my_first = tile_first + split * tiles_per_split;
  const int my_last = min(tile_last, my_first + tiles_per_split);
  __shared__ int page_s[TK], slot_s[TK];   // where each key of the tile lives: page (-1: not read) and slot in it
  for (int kt = my_first * TK; kt < my_last * TK; kt += TK) {
    __syncthreads();  // previous tile consumed (and Q visible on the first pass)
    if (tid < TK) {   // one division and one look at the table per key, not per element
      const int kp = kt + tid;
      int block = -1;
      if (kp >= k_begin && kp < k_end) {
        block = table[kp / block_size];
        if (block >= num_blocks) block = -1;
      }
      page_s[tid] = block;
      slot_s[tid] = kp % block_size;
    }
    __syncthreads();
    for (int e = tid; e < TK * chunks; e += 256) {
      const int kk = e / chunks;
      const int d4 = (e - kk * chunks) * 4;
      // every load is unconditional (a key that is not read takes page 0 and its value is dropped):
      // a load under a per-thread condition is a branch, and a thread's loads would wait for one another
      const int block = page_s[kk];
      float kv[4];
      load4(key_pages + (((size_t)max(block, 0) * kv_heads + hk) * block_size + slot_s[kk]) * D + d4, vec, D - d4, kv);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (d4 + i < D) Ks[kk * kstride + d4 + i] = block >= 0 ? kv[i] : 0.f;
    }
    // values live transposed in their pages ([D][slot]): consecutive threads take consecutive keys
    for (int e = tid; e < TK * D; e += 256) {
      const int d = e / TK;
      const int kk = e - d * TK;
      const int block = page_s[kk];
      const float v = load_as_float(value_pages + (((size_t)max(block, 0) * kv_heads + hk) * D + d) * block_size + slot_s[kk]);
      Vs[kk * kstride + d] = block >= 0 ? v : 0.f;
    }
    __syncthreads();

    float s[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) s[i] = 0.f;
    const float* qrow = Qs + r * kstride;
#pragma unroll 8
    for (int d = 0; d < D; ++d) {
      const float qv = qrow[d];
#pragma unroll
      for (int i = 0; i < KPT; ++i) s[i] = fmaf(qv, Ks[(c + 16 * i) * kstride + d], s[i]);
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int kp = kt + c + 16 * i;
      const bool visible = row_ok && kp <= my_pos && (window <= 0 || kp > my_pos - window);
      s[i] = visible ? s[i] * scale : -INFINITY;
      tile_max = fmaxf(tile_max, s[i]);
    }
#pragma unroll
    for (int offset = 8; offset > 0; offset >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, offset, FE_WAVE));
    const float m_new = fmaxf(m, tile_max);
    float corr = 1.f, tile_sum = 0.f;
    if (m_new > -INFINITY) {
      corr = FAST_EXP ? __expf(m - m_new) : expf(m - m_new);
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const float p = FAST_EXP ? __expf(s[i] - m_new) : expf(s[i] - m_new);
        s[i] = p;
        tile_sum += p;
      }
    } else {
#pragma unroll
      for (int i = 0; i < KPT; ++i) s[i] = 0.f;
    }
#pragma unroll
    for (int offset = 8; offset > 0; offset >>= 1) tile_sum += __shfl_xor(tile_sum, offset, FE_WAVE);
    l = l * corr + tile_sum;
    m = m_new;
#pragma unroll
    for (int i = 0; i < KPT; ++i) Ps[r * TK + c + 16 * i] = s[i];
    __syncthreads();

#pragma unroll
    for (int i = 0; i < DPT; ++i) acc[i] *= corr;
    const float* prow = Ps + r * TK;
#pragma unroll 4
    for (int kk = 0; kk < TK; ++kk) {
      const float p = prow[kk];
      const float* vrow = Vs + kk * kstride;
#pragma unroll
      for (int i = 0; i < DPT; ++i)
        if (c + 16 * i < D) acc[i] = fmaf(p, vrow[c + 16 * i], acc[i]);
    }
  }

  if (row_ok && splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    T* orow = out + (size_t)(q0 + my_tok) * out_stride + (size_t)(hk * groups + my_g) * D;
#pragma unroll
    for (int i = 0; i < DPT; ++i)
      if (c + 16 * i < D) store_from_float(orow + c + 16 * i, acc[i] * inv);
  } else if (row_ok) {
    // this run's share of the row: [split][token][head], the output unnormalised
    const size_t row = ((size_t)split * total_tokens + q0 + my_tok) * (kv_heads * groups) + hk * groups + my_g;
#pragma unroll
    for (int i = 0; i < DPT; ++i)
      if (c + 16 * i < D) part_acc[row * D + c + 16 * i] = acc[i];
    if (c == 0) { part_ml[row * 2] = m; part_ml[row * 2 + 1] = l; }
  }
}

// The runs of a row's keys, merged in their order: the same grid of (row tile, kv head,
// sequence) and the same thread per (row, dims) as the kernel above.
template <typename T, int DMAX, bool FAST_EXP>
__global__ __launch_bounds__(256) void paged_attention_generic_merge_kernel(
    T* __restrict__ out, long long out_stride, const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    int kv_heads, int groups, int head_dim, int min_q_len, int max_q_served, int splits,
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, int total_tokens) {
  constexpr int DPT = DMAX / 16;
  const int D = head_dim;
  const int seq = blockIdx.z, hk = blockIdx.y;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int rows_total = q_len * groups;
  const int row0 = blockIdx.x * ROWS;
  if (row0 >= rows_total || ctx_len[seq] - q_len < 0 || q_len < min_q_len || q_len > max_q_served) return;
  const int r = threadIdx.x / 16, c = threadIdx.x % 16;
  const int my_row = row0 + r;
  if (my_row >= rows_total) return;
  const int tok = my_row / groups, g = my_row - tok * groups;
  const size_t heads = (size_t)kv_heads * groups;
  const size_t first = ((size_t)(q0 + tok)) * heads + hk * groups + g;
  const size_t step = (size_t)total_tokens * heads;
  float m_tot = -INFINITY;
  for (int sp = 0; sp < splits; ++sp) m_tot = fmaxf(m_tot, part_ml[(first + sp * step) * 2]);
  float l = 0.f, acc[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) acc[i] = 0.f;
  for (int sp = 0; sp < splits; ++sp) {
    const size_t row = first + sp * step;
    const float ms = part_ml[row * 2];
    const float f = ms > -INFINITY ? (FAST_EXP ? __expf(ms - m_tot) : expf(ms - m_tot)) : 0.f;
    l = fmaf(f, part_ml[row * 2 + 1], l);
#pragma unroll
    for (int i = 0; i < DPT; ++i)
      if (c + 16 * i < D) acc[i] = fmaf(f, part_acc[row * D + c + 16 * i], acc[i]);
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  T* orow = out + (size_t)(q0 + tok) * out_stride + (size_t)(hk * groups + g) * D;
#pragma unroll
  for (int i = 0; i < DPT; ++i)
    if (c + 16 * i < D) store_from_float(orow + c + 16 * i, acc[i] * inv);
}

template <typename T, int DMAX, int TK, bool FAST_EXP>
static int launch_generic(const void* q, long long q_stride, const void* key_pages, const void* value_pages,
                          void* out, long long out_stride, const int* cu_q, const int* ctx_len,
                          const int* block_table, int table_stride, int num_seqs, int max_q_len,
                          int kv_heads, int groups, int head_dim, int block_size, int num_blocks,
                          int window, float scale, int min_q_len, int max_q_served, int splits,
                          float* part_acc, float* part_ml, int total_tokens, hipStream_t stream) {
  const long long tiles = ((long long)max_q_len * groups + ROWS - 1) / ROWS;
  if (tiles * splits > 0x7fffffffLL || kv_heads > 65535 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  const size_t smem = sizeof(float) * ((size_t)(ROWS + 2 * TK) * (head_dim + 1) + ROWS * TK);
  dim3 grid((unsigned)(tiles * splits), kv_heads, num_seqs);
  paged_attention_generic_kernel<T, DMAX, TK, FAST_EXP><<<grid, 256, smem, stream>>>(
      (const T*)q, q_stride, (const T*)key_pages, (const T*)value_pages, (T*)out, out_stride, cu_q,
      ctx_len, block_table, table_stride, kv_heads, groups, head_dim, block_size, num_blocks, window,
      scale, min_q_len, max_q_served, splits, part_acc, part_ml, total_tokens);
  if (splits > 1) {
    dim3 merge_grid((unsigned)tiles, kv_heads, num_seqs);
    paged_attention_generic_merge_kernel<T, DMAX, FAST_EXP><<<merge_grid, 256, 0, stream>>>(
        (T*)out, out_stride, cu_q, ctx_len, kv_heads, groups, head_dim, min_q_len, max_q_served, splits,
        part_acc, part_ml, total_tokens);
  }
  return fe_check_launch();
}

template <typename T, bool FAST_EXP>
static int dispatch_generic(const void* q, long long q_stride, const void* key_pages, const void* value_pages,
                            void* out, long long out_stride, const int* cu_q, const int* ctx_len,
                            const int* block_table, int table_stride, int num_seqs, int max_q_len,
                            int kv_heads, int groups, int head_dim, int block_size, int num_blocks,
                            int window, float scale, int min_q_len, int max_q_served, int splits,
                            float* part_acc, float* part_ml, int total_tokens, hipStream_t stream) {
#define FE_GO(DMAX, TK)                                                                              \
  return launch_generic<T, DMAX, TK, FAST_EXP>(q, q_stride, key_pages, value_pages, out, out_stride, \
                                               cu_q, ctx_len, block_table, table_stride, num_seqs,   \
                                               max_q_len, kv_heads, groups, head_dim, block_size,    \
                                               num_blocks, window, scale, min_q_len, max_q_served, splits, \
                                               part_acc, part_ml, total_tokens, stream)
  if (head_dim <= 32) FE_GO(32, 64);
  if (head_dim <= 64) FE_GO(64, 64);
  if (head_dim <= 128) FE_GO(128, 32);
  FE_GO(256, 16);
#undef FE_GO
}

// q: [tokens, ...] with q_stride elements between tokens, heads contiguous
// ([q_heads][D]) from the token's start; out likewise with out_stride.
// cu_q: [num_seqs + 1] prefix sums of query lengths; ctx_len: [num_seqs] keys
// in the cache after this step; block_table: [num_seqs, table_stride].
// Sequences with fewer than min_q_len or more than max_q_served query tokens are skipped
// (other kernels serve them).  splits > 1 (at most 64) cuts every row's keys into that many runs
// walked by blocks of their own; it needs scratch part_acc [splits][total_tokens][q heads][head_dim]
// and part_ml [splits][total_tokens][q heads][2] floats, total_tokens being the rows of q.
// The tile of keys a block walks at a time is fe_paged_attention_generic_key_tile(head_dim) long.
extern "C" int fe_paged_attention_generic_key_tile(int head_dim) {
  return head_dim <= 64 ? 64 : (head_dim <= 128 ? 32 : 16);
}

extern "C" int fe_paged_attention_generic(const void* q, long long q_stride, const void* key_pages,
                                          const void* value_pages, void* out, long long out_stride,
                                          int dtype, const int* cu_q, const int* ctx_len,
                                          const int* block_table, int table_stride, int num_seqs,
                                          int max_q_len, int kv_heads, int groups, int head_dim,
                                          int block_size, int num_blocks, int window, float scale,
                                          int min_q_len, int max_q_served, int splits, float* part_acc,
                                          float* part_ml, int total_tokens, hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len <= 0) return FE_OK;
  if (max_q_served < max_q_len) max_q_len = max_q_served;   // the grid covers only what is served
  if (max_q_len < min_q_len) return FE_OK;
  if (head_dim < 2 || head_dim > 256 || head_dim % 2) return FE_BAD_ARGUMENT;
  if (kv_heads <= 0 || groups <= 0 || block_size <= 0 || num_blocks <= 0 || table_stride <= 0) return FE_BAD_ARGUMENT;
  if (out_stride < (long long)kv_heads * groups * head_dim) return FE_BAD_ARGUMENT;
  if (splits < 1 || splits > 64 || (splits > 1 && (!part_acc || !part_ml || total_tokens < 1))) return FE_BAD_ARGUMENT;
  if (dtype == FE_F32)
    return dispatch_generic<float, false>(q, q_stride, key_pages, value_pages, out, out_stride, cu_q, ctx_len,
                                          block_table, table_stride, num_seqs, max_q_len, kv_heads, groups,
                                          head_dim, block_size, num_blocks, window, scale, min_q_len, max_q_served,
                                          splits, part_acc, part_ml, total_tokens, stream);
  if (dtype == FE_BF16)
    return dispatch_generic<bf16_t, true>(q, q_stride, key_pages, value_pages, out, out_stride, cu_q, ctx_len,
                                          block_table, table_stride, num_seqs, max_q_len, kv_heads, groups,
                                          head_dim, block_size, num_blocks, window, scale, min_q_len, max_q_served,
                                          splits, part_acc, part_ml, total_tokens, stream);
  return FE_BAD_ARGUMENT;
}
