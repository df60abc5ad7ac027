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
  // Where each key of a tile lives: page (-1: not read) and slot in it; two tiles, the one being
  // multiplied and the one being fetched.
  __shared__ int page_s[2][TK], slot_s[2][TK];
  // Every load below is unconditional and all loads of a tile are issued before the first is used: a load
  // under a per-thread condition is a branch, and loads that wait for one another cost a trip to memory each
  // (a key that is not read takes page 0 and its value is dropped).  A tile's keys and values are fetched
  // into registers while the tile before it is multiplied out of LDS, its page ids a tile earlier still.
  constexpr int KL = TK * DMAX / 1024;     // groups of four elements a thread fetches of a tile's keys, and of its values
  const bool vec_v = block_size % 4 == 0 && (((uintptr_t)value_pages) & (4 * sizeof(T) - 1)) == 0;
  const int kt_end = my_last * TK;
  // the page of key kt + tid (threads below TK)
  auto lookup = [&](int kt) -> int {
    const int kp = kt + min(tid, TK - 1);
    const int block = table[min(max(kp, k_begin), k_end - 1) / block_size];
    return kp >= k_begin && kp < k_end && block < num_blocks ? block : -1;
  };
  float kreg[KL][4], vreg[KL][4];
  auto fetch = [&](int buf) {
    const int* page = page_s[buf];
    const int* slot = slot_s[buf];
#pragma unroll
    for (int j = 0; j < KL; ++j) {
      const int e = min(tid + j * 256, TK * chunks - 1);
      const int kk = e / chunks;
      const int d4 = (e - kk * chunks) * 4;
      load4(key_pages + (((size_t)max(page[kk], 0) * kv_heads + hk) * block_size + slot[kk]) * D + d4, vec, D - d4, kreg[j]);
    }
    // values live transposed in their pages ([D][slot]): consecutive threads take consecutive keys,
    // four slots at a time where pages hold a multiple of four
    if (vec_v) {
#pragma unroll
      for (int j = 0; j < KL; ++j) {
        const int e = min(tid + j * 256, TK / 4 * D - 1);
        const int d = e / (TK / 4);
        const int kk = (e - d * (TK / 4)) * 4;
        const int block = max(max(page[kk], page[kk + 1]), max(page[kk + 2], page[kk + 3]));
        Vec4<T>::load(value_pages + (((size_t)max(block, 0) * kv_heads + hk) * D + d) * block_size + slot[kk], vreg[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4 * KL; ++j) {
        const int e = min(tid + j * 256, TK * D - 1);
        const int d = e / TK;
        const int kk = e - d * TK;
        vreg[j / 4][j % 4] = load_as_float(value_pages + (((size_t)max(page[kk], 0) * kv_heads + hk) * D + d) * block_size + slot[kk]);
      }
    }
  };
  auto to_lds = [&](int buf) {
    const int* page = page_s[buf];
#pragma unroll
    for (int j = 0; j < KL; ++j) {
      const int e = tid + j * 256;
      if (e < TK * chunks) {
        const int kk = e / chunks;
        const int d4 = (e - kk * chunks) * 4;
        const bool read = page[kk] >= 0;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (d4 + i < D) Ks[kk * kstride + d4 + i] = read ? kreg[j][i] : 0.f;
      }
    }
    if (vec_v) {
#pragma unroll
      for (int j = 0; j < KL; ++j) {
        const int e = tid + j * 256;
        if (e < TK / 4 * D) {
          const int d = e / (TK / 4);
          const int kk = (e - d * (TK / 4)) * 4;
#pragma unroll
          for (int i = 0; i < 4; ++i) Vs[(kk + i) * kstride + d] = page[kk + i] >= 0 ? vreg[j][i] : 0.f;
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4 * KL; ++j) {
        const int e = tid + j * 256;
        if (e < TK * D) {
          const int d = e / TK;
          const int kk = e - d * TK;
          Vs[kk * kstride + d] = page[kk] >= 0 ? vreg[j / 4][j % 4] : 0.f;
        }
      }
    }
  };
  int next_block = -1;
  if (my_first < my_last) {
    next_block = lookup(my_first * TK);
    if (tid < TK) {
      page_s[0][tid] = next_block;
      slot_s[0][tid] = (my_first * TK + tid) % block_size;
    }
    __syncthreads();
    if (my_first * TK + TK < kt_end) next_block = lookup(my_first * TK + TK);
    fetch(0);
  }
  int buf = 0;
  for (int kt = my_first * TK; kt < kt_end; kt += TK, buf ^= 1) {
    __syncthreads();  // the tile before is consumed (and Q visible on the first pass)
    to_lds(buf);
    if (tid < TK) {   // one division and one look at the table per key, not per element
      page_s[buf ^ 1][tid] = next_block;
      slot_s[buf ^ 1][tid] = (kt + TK + tid) % block_size;
    }
    __syncthreads();
    if (kt + TK < kt_end) {
      if (kt + 2 * TK < kt_end) next_block = lookup(kt + 2 * TK);
      fetch(buf ^ 1);
    }

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
  // eight runs a round, every load of a round issued before the first is used (the last round reads
  // the last run again where it has fewer; those copies get the weight zero)
  float m_tot = -INFINITY;
  for (int base = 0; base < splits; base += 8) {
    float ms[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) ms[j] = part_ml[(first + min(base + j, splits - 1) * step) * 2];
#pragma unroll
    for (int j = 0; j < 8; ++j) m_tot = fmaxf(m_tot, ms[j]);
  }
  float l = 0.f, acc[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) acc[i] = 0.f;
  for (int base = 0; base < splits; base += 8) {
    float2 ml[8];
    float part[8][DPT];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const size_t row = first + min(base + j, splits - 1) * step;
      ml[j] = *(const float2*)(part_ml + row * 2);
#pragma unroll
      for (int i = 0; i < DPT; ++i) part[j][i] = part_acc[row * D + min(c + 16 * i, D - 1)];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool counts = base + j < splits && ml[j].x > -INFINITY;
      const float f = counts ? (FAST_EXP ? __expf(ml[j].x - m_tot) : expf(ml[j].x - m_tot)) : 0.f;
      l = fmaf(f, ml[j].y, l);
#pragma unroll
      for (int i = 0; i < DPT; ++i) acc[i] = fmaf(f, part[j][i], acc[i]);
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  T* orow = out + (size_t)(q0 + tok) * out_stride + (size_t)(hk * groups + g) * D;
#pragma unroll
  for (int i = 0; i < DPT; ++i)
    if (c + 16 * i < D) store_from_float(orow + c + 16 * i, acc[i] * inv);
}

// ---------------------------------------------------------------------------------------------
// Single-token sequences (decoding) on the vector ALU: the float32 mode's decode attention, and
// bfloat16 shapes that the matrix-core decode kernel does not take.
//
// block = (key run, group of up to GMAX query heads that share a kv head, kv head, sequence); 256 threads.
// Nothing of a key or value goes through LDS.  A tile of TK = 1024 / LPK keys is fetched as it lies in
// memory: LPK consecutive lanes share a key and hold four of its dims each (a thread has four keys of a
// tile), multiply them with the same dims of the GMAX queries in registers, and the LPK lanes add up by
// lane permutes.  Values lie transposed in their pages, so a thread takes four consecutive slots of one
// output dim (four dims of a tile), the TK / 4 lanes that share a dim add up once, after the last tile.
// Scores meet in LDS ([GMAX][TK]) for the softmax, which GMAX * TK threads do, a group of TK lanes a row.
// The next tile's keys are fetched once this tile's scores are formed, its values once this tile's are
// used, and page ids a tile before their data: the fetches fly while the block computes.
// Requires head_dim % 4 == 0, block_size % 4 == 0 and 16-byte aligned rows (the host checks).
template <int L> __device__ __forceinline__ float lanes_sum(float v) {   // over L consecutive lanes, every lane gets it
  static_assert(L == 4 || L == 8 || L == 16 || L == 32 || L == 64, "group of lanes");
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // lane ^ 2
  if (L >= 8) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - lane in 8
  if (L >= 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true)); // 15 - lane in 16
  if (L >= 32) v = sum_xor16(v);
  if (L >= 64) v = sum_xor32(v);
  return v;
}
template <int L> __device__ __forceinline__ float lanes_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)));
  if (L >= 8) v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true)));
  if (L >= 16) v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true)));
  if (L >= 32) v = max_xor16(v);
  if (L >= 64) v = max_xor32(v);
  return v;
}

template <typename T, int LPK, int GMAX, bool FAST_EXP>
__global__ __launch_bounds__(256) void paged_attention_rows_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ key_pages,
    const T* __restrict__ value_pages, T* __restrict__ out, long long out_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int table_stride, int kv_heads, int groups, int head_dim, int block_size, int block_shift,
    int num_blocks, int window, float scale, int splits, float* __restrict__ part_acc,
    float* __restrict__ part_ml, int total_tokens) {
  constexpr int TK = 1024 / LPK;    // keys of a tile: 64, 32, 16
  constexpr int KPP = 256 / LPK;    // keys the block covers with one fetch a thread: a thread's keys lie KPP apart
  constexpr int LPD = TK / 4;       // lanes that share an output dim
  constexpr int DPP = 256 / LPD;    // dims the block covers with one fetch a thread: a thread's dims lie DPP apart
  // A tile's scores, then its probabilities.  Two buffers that the tiles take in turn: a wave that has
  // used a tile's probabilities goes on to write the next tile's scores before the block's next barrier,
  // while a slower wave may still be reading the probabilities; in the other buffer it disturbs nobody,
  // and that buffer's last readers passed two barriers ago.
  __shared__ __align__(16) float Ps2[2][GMAX][TK];
  __shared__ float ml_s[GMAX][2];                // running maximum and sum of a row
  __shared__ float corr_s[GMAX];                 // what the tile scales a row's earlier sums by

  const int tid = threadIdx.x;
  const int seq = blockIdx.z, hk = blockIdx.y;
  const int q0 = cu_q[seq];
  if (cu_q[seq + 1] - q0 != 1) return;
  const int ctx = ctx_len[seq];
  const int split = blockIdx.x % splits;
  const int row0 = (blockIdx.x / splits) * GMAX;
  if (ctx < 1 || row0 >= groups) return;
  const int rows = min(GMAX, groups - row0);
  const int D = head_dim, chunks = D / 4;
  const int k_begin = window > 0 ? max(0, ctx - window) : 0, k_end = ctx;
  const int tile_first = k_begin / TK, tile_last = (k_end + TK - 1) / TK;
  const int tiles_per_split = (tile_last - tile_first + splits - 1) / splits;
  const int my_first = tile_first + split * tiles_per_split;
  const int my_last = min(tile_last, my_first + tiles_per_split);
  const int kt_end = my_last * TK;

  const int lane_k = tid % LPK, key0 = tid / LPK;      // keys: which four dims, which key of a pass
  const bool d_ok = lane_k < chunks;
  const int d4 = min(lane_k, chunks - 1) * 4;
  const int kq4 = (tid % LPD) * 4, dim0 = tid / LPD;   // values: which four slots of the tile, which dim of a pass

  float qr[GMAX][4];
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    Vec4<T>::load(q + (size_t)q0 * q_stride + (size_t)(hk * groups + row0 + min(g, rows - 1)) * D + d4, qr[g]);
#pragma unroll
    for (int i = 0; i < 4; ++i) qr[g][i] = d_ok && g < rows ? qr[g][i] : 0.f;
  }
  if (tid < GMAX) { ml_s[tid][0] = -INFINITY; ml_s[tid][1] = 0.f; corr_s[tid] = 1.f; }

  const int* table = block_table + (size_t)seq * table_stride;
  auto page_index = [&](int kp) { return block_shift >= 0 ? kp >> block_shift : kp / block_size; };
  // page ids of a tile: of this thread's four keys, and of its four value slots (which share a page)
  auto lookup = [&](int kt, int* pages_k, int& page_v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) pages_k[j] = table[page_index(min(max(kt + key0 + j * KPP, k_begin), k_end - 1))];
    page_v = table[page_index(min(max(kt + kq4, k_begin & ~3), (k_end - 1) & ~3))];
  };
  float kreg[4][4], vreg[4][4];
  // every fetch is unconditional: a key or slot that is not read takes an address that is there, and is dropped
  auto fetch_keys = [&](int kt, const int* pages_k) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kp = min(max(kt + key0 + j * KPP, k_begin), k_end - 1);
      const int slot = kp - page_index(kp) * block_size;
      const int page = pages_k[j] < num_blocks ? max(pages_k[j], 0) : 0;
      Vec4<T>::load(key_pages + (((size_t)page * kv_heads + hk) * block_size + slot) * D + d4, kreg[j]);
    }
  };
  auto fetch_values = [&](int kt, int page_v) {
    const int kp = min(max(kt + kq4, k_begin & ~3), (k_end - 1) & ~3);
    const int slot = kp - page_index(kp) * block_size;
    const int page = page_v < num_blocks ? max(page_v, 0) : 0;
    const T* base = value_pages + ((size_t)page * kv_heads + hk) * D * block_size + slot;
#pragma unroll
    for (int j = 0; j < 4; ++j) Vec4<T>::load(base + (size_t)min(dim0 + j * DPP, D - 1) * block_size, vreg[j]);
  };

  float acc[GMAX][4];
#pragma unroll
  for (int g = 0; g < GMAX; ++g)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[g][j] = 0.f;

  int pk[4], pv = 0, pkn[4], pvn = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) pk[j] = pkn[j] = 0;
  if (my_first * TK < kt_end) {
    lookup(my_first * TK, pk, pv);
    fetch_keys(my_first * TK, pk);
    fetch_values(my_first * TK, pv);
    if (my_first * TK + TK < kt_end) lookup(my_first * TK + TK, pkn, pvn);
  }
  int buffer = 0;
  for (int kt = my_first * TK; kt < kt_end; kt += TK, buffer ^= 1) {
    const bool more = kt + TK < kt_end;
    float (*Ps)[TK] = Ps2[buffer];
    float s[GMAX][4];
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        s[g][j] = fmaf(qr[g][3], kreg[j][3], fmaf(qr[g][2], kreg[j][2], fmaf(qr[g][1], kreg[j][1], qr[g][0] * kreg[j][0])));
    bool read[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kp = kt + key0 + j * KPP;
      read[j] = kp >= k_begin && kp < k_end && pk[j] < num_blocks && pk[j] >= 0;
    }
    if (more) {
#pragma unroll
      for (int j = 0; j < 4; ++j) pk[j] = pkn[j];
      fetch_keys(kt + TK, pk);
    }
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float total = lanes_sum<LPK>(s[g][j]);
        if (lane_k == 0) Ps[g][key0 + j * KPP] = read[j] ? total * scale : -INFINITY;
      }
    __syncthreads();
    for (int e = tid; e < GMAX * TK; e += 256) {   // a row's TK lanes stay together: 256 and 64 are multiples of TK
      const int g = e / TK, key = e - g * TK;
      const float score = Ps[g][key];
      const float m_old = ml_s[g][0], l_old = ml_s[g][1];
      const float m_new = fmaxf(m_old, lanes_max<TK>(score));
      float p = 0.f, corr = 1.f;
      if (m_new > -INFINITY) {
        corr = FAST_EXP ? __expf(m_old - m_new) : expf(m_old - m_new);
        p = FAST_EXP ? __expf(score - m_new) : expf(score - m_new);
      }
      const float tile_sum = lanes_sum<TK>(p);
      Ps[g][key] = p;
      if (key == 0) { ml_s[g][0] = m_new; ml_s[g][1] = fmaf(l_old, corr, tile_sum); corr_s[g] = corr; }
    }
    __syncthreads();
    // slots that no key in reach owns may hold anything: their values count as zero
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kp = kt + kq4 + i;
      const bool owned = kp >= k_begin && kp < k_end && pv < num_blocks && pv >= 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) vreg[j][i] = owned ? vreg[j][i] : 0.f;
    }
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      const float corr = corr_s[g];
      const float4 p = *(const float4*)&Ps[g][kq4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[g][j] = fmaf(p.w, vreg[j][3], fmaf(p.z, vreg[j][2], fmaf(p.y, vreg[j][1], fmaf(p.x, vreg[j][0], acc[g][j] * corr))));
    }
    if (more) {
      pv = pvn;
      fetch_values(kt + TK, pv);
      if (kt + 2 * TK < kt_end) lookup(kt + 2 * TK, pkn, pvn);
    }
  }
  __syncthreads();   // a run without keys: the rows' first statistics are in LDS

#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    if (g >= rows) break;
    const float m = ml_s[g][0], l = ml_s[g][1];
    const float inv = splits == 1 ? (l > 0.f ? 1.f / l : 0.f) : 1.f;
    const size_t head = (size_t)hk * groups + row0 + g;
    const size_t part_row = ((size_t)split * total_tokens + q0) * ((size_t)kv_heads * groups) + head;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float total = lanes_sum<LPD>(acc[g][j]) * inv;
      const int d = dim0 + j * DPP;
      if (tid % LPD == 0 && d < D) {
        if (splits == 1) store_from_float(out + (size_t)q0 * out_stride + head * D + d, total);
        else part_acc[part_row * D + d] = total;
      }
    }
    if (splits > 1 && tid == 0) { part_ml[part_row * 2] = m; part_ml[part_row * 2 + 1] = l; }
  }
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

// Single-token sequences only (sequences with another number of query tokens are skipped), any even
// number of dims that is a multiple of four up to 256, pages of a multiple of four slots, rows of q and
// the pages 16-byte aligned; everything else as fe_paged_attention_generic, whose merge kernel and
// scratch layout the key runs share.
extern "C" int fe_paged_attention_rows(const void* q, long long q_stride, const void* key_pages,
                                       const void* value_pages, void* out, long long out_stride, int dtype,
                                       const int* cu_q, const int* ctx_len, const int* block_table,
                                       int table_stride, int num_seqs, int kv_heads, int groups, int head_dim,
                                       int block_size, int num_blocks, int window, float scale, int splits,
                                       float* part_acc, float* part_ml, int total_tokens, hipStream_t stream) {
  if (num_seqs <= 0) return FE_OK;
  if (head_dim < 4 || head_dim > 256 || head_dim % 4 || block_size <= 0 || block_size % 4) return FE_BAD_ARGUMENT;
  if (kv_heads <= 0 || groups <= 0 || num_blocks <= 0 || table_stride <= 0) return FE_BAD_ARGUMENT;
  if (kv_heads > 65535 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (out_stride < (long long)kv_heads * groups * head_dim) return FE_BAD_ARGUMENT;
  if (splits < 1 || splits > 64 || (splits > 1 && (!part_acc || !part_ml || total_tokens < 1))) return FE_BAD_ARGUMENT;
  const size_t elem = dtype == FE_F32 ? 4 : 2;
  if (dtype != FE_F32 && dtype != FE_BF16) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)q | (uintptr_t)key_pages | (uintptr_t)value_pages) & (4 * elem - 1)) || q_stride % 4) return FE_BAD_ARGUMENT;
  int block_shift = -1;
  if ((block_size & (block_size - 1)) == 0)
    for (block_shift = 0; (1 << block_shift) < block_size; ++block_shift) {}
  const int gmax = groups <= 4 ? 4 : 8;
  const int row_tiles = (groups + gmax - 1) / gmax;
  dim3 grid((unsigned)(row_tiles * splits), kv_heads, num_seqs);
#define FE_ROWS(T, LPK, GMAX, FAST)                                                                       \
  paged_attention_rows_kernel<T, LPK, GMAX, FAST><<<grid, 256, 0, stream>>>(                              \
      (const T*)q, q_stride, (const T*)key_pages, (const T*)value_pages, (T*)out, out_stride, cu_q,       \
      ctx_len, block_table, table_stride, kv_heads, groups, head_dim, block_size, block_shift, num_blocks, \
      window, scale, splits, part_acc, part_ml, total_tokens)
#define FE_ROWS_G(T, LPK, FAST) do { if (gmax == 4) FE_ROWS(T, LPK, 4, FAST); else FE_ROWS(T, LPK, 8, FAST); } while (0)
#define FE_ROWS_D(T, FAST) do {                                      \
    if (head_dim <= 64) FE_ROWS_G(T, 16, FAST);                      \
    else if (head_dim <= 128) FE_ROWS_G(T, 32, FAST);                \
    else FE_ROWS_G(T, 64, FAST); } while (0)
  if (dtype == FE_F32) FE_ROWS_D(float, false); else FE_ROWS_D(bf16_t, true);
#undef FE_ROWS_D
#undef FE_ROWS_G
#undef FE_ROWS
  if (splits > 1) {
    dim3 merge_grid((unsigned)((groups + ROWS - 1) / ROWS), kv_heads, num_seqs);
#define FE_MERGE(T, DMAX, FAST)                                                                            \
    paged_attention_generic_merge_kernel<T, DMAX, FAST><<<merge_grid, 256, 0, stream>>>(                   \
        (T*)out, out_stride, cu_q, ctx_len, kv_heads, groups, head_dim, 1, 1, splits, part_acc, part_ml, total_tokens)
#define FE_MERGE_D(T, FAST) do {                                     \
    if (head_dim <= 32) FE_MERGE(T, 32, FAST);                       \
    else if (head_dim <= 64) FE_MERGE(T, 64, FAST);                  \
    else if (head_dim <= 128) FE_MERGE(T, 128, FAST);                \
    else FE_MERGE(T, 256, FAST); } while (0)
    if (dtype == FE_F32) FE_MERGE_D(float, false); else FE_MERGE_D(bf16_t, true);
#undef FE_MERGE_D
#undef FE_MERGE
  }
  return fe_check_launch();
}
