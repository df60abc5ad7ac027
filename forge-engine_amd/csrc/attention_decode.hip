// Paged grouped-query attention for single decoded tokens, bfloat16 cache.
//
// For every sequence of the batch that brings exactly one query token (others
// are skipped: another kernel serves them), the G query heads that share a kv
// head read that head's keys and values once.  The kernel is bound by the
// cache's bytes; everything between the loads and the output stays in
// registers:
//   * grid (key split, kv head, sequence); with few sequences the keys of one
//     (sequence, head) are split over several blocks so that the chip is full,
//     and the block that finishes last merges the splits (a counter per (sequence, head));
//   * inside a block the four waves take 32-key blocks in turn;
//   * scores transposed, S^T = K Q^T: MFMA 16x16x32 with A = 16 keys (rows) and
//     B = the G query rows padded to 16 (columns).  The 32 keys of a block feed
//     two MFMA tiles whose rows interleave in groups of four, so that lane
//     group lq ends up with the scores of the 8 consecutive keys 8lq .. 8lq+7 of
//     its query row: exactly the B operand of the second product;
//   * softmax statistics per query row in float32 (a row's keys sit in four
//     lanes: two shuffles), base-2 exponent with the scale folded in;
//   * output transposed, O^T = V^T P^T: A = 16 dims x 32 keys from the value
//     pages, which are stored transposed ([D][slot]) for this, B = P^T.
// Exactness: scores, max, sum and the weighted value sum are float32; P is
// rounded to bfloat16 for the second product; one rounding at the final store.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define KEYS 32          // keys per block of work
#define WAVES 4
#define GMAX 8           // largest group size served

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
__device__ __forceinline__ unsigned int pack_bf16(float lo, float hi) {
  const bf16x2 v = {(__bf16)lo, (__bf16)hi};   // the hardware's round-to-nearest-even conversion
  return __builtin_bit_cast(unsigned int, v);
}

// Device-scope accesses: they are served by memory that all dies share, not by a die's own L2.
__device__ __forceinline__ void store_agent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int D>
__global__ __launch_bounds__(256, D <= 128 ? 2 : 1) void paged_decode_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, long long out_stride,
    float* part_o, float* part_ml, int* __restrict__ counters, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const int* __restrict__ block_table, int table_stride,
    int kv_heads, int groups, int block_shift, int num_blocks, int window, float scale_log2) {
  const int block_size = 1 << block_shift, block_mask = block_size - 1;
  constexpr int KC = D / 32;        // MFMA k-steps over the head dim (scores)
  constexpr int DT = D / 16;        // 16-dim tiles of the output
  __shared__ float Ow[WAVES][GMAX][D];
  __shared__ float Ms[WAVES][GMAX], Ls[WAVES][GMAX];

  const int split = blockIdx.x, splits = gridDim.x;
  const int hk = blockIdx.y, seq = blockIdx.z;
  const int q0 = cu_q[seq];
  if (cu_q[seq + 1] - q0 != 1) return;
  const int ctx = ctx_len[seq];
  const int k_begin = window > 0 ? max(0, ctx - window) : 0;
  const int first = k_begin / KEYS;
  const int last = (ctx + KEYS - 1) / KEYS;               // exclusive
  const int per_split = (last - first + splits - 1) / splits;
  const int my_first = first + split * per_split;
  const int my_last = min(last, my_first + per_split);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lq = lane >> 4;

  // query rows as the B operand: lane (lr = row g, lq) holds q[g][32c + 8lq .. +8]
  bf16x8 qb[KC];
  {
    const bf16_t* qrow = q + (size_t)q0 * q_stride + (size_t)(hk * groups + (lr < groups ? lr : 0)) * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      uintx4 v = uintx4{0u, 0u, 0u, 0u};
      if (lr < groups) v = *(const uintx4*)(qrow + c * 32 + lq * 8);
      qb[c] = __builtin_bit_cast(bf16x8, v);
    }
  }

  float m_run = -INFINITY, l_run = 0.f;   // of query row lr (the same in the four lanes that share it)
  floatx4 o[DT];                          // O^T: dims 16t + 4lq + i of query row lr
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int* table = block_table + (size_t)seq * table_stride;
  // MFMA row r of key tile h (h = 0, 1) is key 8*(r/4) + 4h + r%4 of the block
  const int krow = 8 * (lr >> 2) + (lr & 3);
  // Page ids are read two blocks ahead and keys one block ahead, so that no load has to wait
  // for another load: a lane needs one key page (its key rows krow, krow + 4 share it) and one
  // value page (keys 8lq .. 8lq+7) per block.
  // Every load below is unconditional (out-of-range keys read a valid address and are masked
  // afterwards), so the loop body is straight-line code and the loads stay where they are issued.
  const int table_last = table_stride - 1;
  // Raw table entries are loaded two blocks ahead and checked only where they are used, so that
  // nothing waits for them while the block's own loads are in flight.
  auto raw_page = [&](int key) -> int { return table[min(key >> block_shift, table_last)]; };
  auto checked = [&](int id, int key) -> int { return (key < ctx && id >= 0 && id < num_blocks) ? id : 0; };
  auto fetch_keys = [&](int b, int block, uintx4 (*dst)[KC]) {
    const bool mine = b < my_last;      // past this block's share: read page 0 again (cached) instead
    block = mine ? block : 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int key = mine ? b * KEYS + krow + 4 * h : krow + 4 * h;
      const bf16_t* row = key_pages + ((((size_t)block * kv_heads + hk) << block_shift) + (key & block_mask)) * D;
#pragma unroll
      for (int c = 0; c < KC; ++c) dst[h][c] = *(const uintx4*)(row + c * 32 + lq * 8);
    }
  };
  // One block of 32 keys: its keys are in kcur (loaded a step ago), vraw is its value page; the
  // step issues its value loads, then the next block's key loads into knext (page knext_raw) and
  // the raw page ids of the block after that (into vraw and knext_raw2).  Two steps alternate the
  // roles of the register sets, so nothing is copied.
  auto step = [&](int b, uintx4 (*kcur)[KC], uintx4 (*knext)[KC], int& vraw, int knext_raw, int& knext_raw2) {
    // values (A operand of the second product): lane (lr = dim, lq) reads the 8 consecutive keys
    // 8lq .. 8lq+7 of dims 16t + lr from the transposed page
    const int vkey = b * KEYS + 8 * lq;
    const bool v_ok = vkey < ctx;
    const int vpage = checked(vraw, vkey);
    const bf16_t* vbase = value_pages + ((((size_t)vpage * kv_heads + hk) * D) << block_shift) + (vkey & block_mask);
    uintx4 va[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) va[t] = *(const uintx4*)(vbase + ((size_t)(t * 16 + lr) << block_shift));
    __builtin_amdgcn_sched_barrier(0);
    fetch_keys(b + WAVES, checked(knext_raw, (b + WAVES) * KEYS + krow), knext);
    vraw = raw_page((b + 2 * WAVES) * KEYS + 8 * lq);
    knext_raw2 = raw_page((b + 2 * WAVES) * KEYS + krow);
    __builtin_amdgcn_sched_barrier(0);

    floatx4 st[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      st[h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; ++c)
        st[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kcur[h][c]), qb[c], st[h], 0, 0, 0);
    }
    // lane (lr = query row, lq): st[h][i] = score of key b*32 + 8lq + 4h + i
    float s[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = b * KEYS + 8 * lq + j;
      const float v = st[j >> 2][j & 3] * scale_log2;
      s[j] = (key >= k_begin && key < ctx) ? v : -INFINITY;
      mx = fmaxf(mx, s[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, FE_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, FE_WAVE));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new > -INFINITY ? m_new : 0.f;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s[j] = __builtin_amdgcn_exp2f(s[j] - m_use);
      sum += s[j];
    }
    sum += __shfl_xor(sum, 16, FE_WAVE);
    sum += __shfl_xor(sum, 32, FE_WAVE);
    l_run = l_run * corr + sum;
    m_run = m_new;
    uintx4 pw;
    pw.x = pack_bf16(s[0], s[1]); pw.y = pack_bf16(s[2], s[3]);
    pw.z = pack_bf16(s[4], s[5]); pw.w = pack_bf16(s[6], s[7]);
    const bf16x8 pb = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= corr;
      const uintx4 vt = v_ok ? va[t] : uintx4{0u, 0u, 0u, 0u};
      o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vt), pb, o[t], 0, 0, 0);
    }
  };

  uintx4 k0[2][KC], k1[2][KC];
  const int b0 = my_first + wave;
  int v0 = 0, v1 = 0, kr0 = 0, kr1 = 0;      // raw page ids: values of this / the next block, keys of the next two
  if (b0 < my_last) {
    v0 = raw_page(b0 * KEYS + 8 * lq);
    fetch_keys(b0, checked(raw_page(b0 * KEYS + krow), b0 * KEYS + krow), k0);
    kr1 = raw_page((b0 + WAVES) * KEYS + krow);
    v1 = raw_page((b0 + WAVES) * KEYS + 8 * lq);
  }
  for (int b = b0; b < my_last; b += 2 * WAVES) {
    step(b, k0, k1, v0, kr1, kr0);
    if (b + WAVES >= my_last) break;
    step(b + WAVES, k1, k0, v1, kr0, kr1);
  }

  // lane (lr = query row, lq) holds O^T[16t + 4lq + i][lr]; the four waves meet in LDS
  if (lr < groups) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) Ow[wave][lr][t * 16 + lq * 4 + i] = o[t][i];
    if (lq == 0) { Ms[wave][lr] = m_run; Ls[wave][lr] = l_run; }
  }
  __syncthreads();

  for (int e = tid; e < groups * D; e += 256) {
    const int g = e / D, d = e - g * D;
    float m_tot = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) m_tot = fmaxf(m_tot, Ms[w][g]);
    float ov = 0.f, l = 0.f;
    if (m_tot > -INFINITY) {
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float f = __builtin_amdgcn_exp2f(Ms[w][g] - m_tot);
        ov += f * Ow[w][g][d];
        l += f * Ls[w][g];
      }
    }
    if (splits == 1) {
      out[(size_t)q0 * out_stride + (size_t)(hk * groups + g) * D + d] = float_to_bf16(l > 0.f ? ov / l : 0.f);
    } else {
      const size_t slot = ((size_t)seq * kv_heads + hk) * splits + split;
      store_agent(&part_o[(slot * groups + g) * D + d], ov);
      if (d == 0) {
        store_agent(&part_ml[(slot * groups + g) * 2], m_tot);        // base-2 exponent units
        store_agent(&part_ml[(slot * groups + g) * 2 + 1], l);
      }
    }
  }
  if (splits == 1) return;

  // The block that finishes last among the splits of this (sequence, kv head) merges them.  The
  // parts are written and read with device-scope accesses that go past the per-die L2 caches, the
  // barrier waits for this block's stores, then one thread counts the block in; whoever counts
  // last reads all parts.  No cache-wide fence: on this chip those serialise across all blocks
  // (measured: 0.3 us per block).  The counter goes back to zero for the next launch.
  __shared__ int is_last;
  __shared__ float scale_s[GMAX][64];   // weight of each split per query row
  __shared__ float inv_l[GMAX];
  __syncthreads();
  if (tid == 0) {
    int* counter = counters + (size_t)seq * kv_heads + hk;
    const int arrived = atomicAdd(counter, 1);
    is_last = arrived == splits - 1;
    if (is_last) atomicExch(counter, 0);
  }
  __syncthreads();
  if (!is_last) return;
  const size_t first_part = ((size_t)seq * kv_heads + hk) * splits;
  if (tid < groups) {
    const int g = tid;
    float m_tot = -INFINITY;
    for (int sp = 0; sp < splits; ++sp) m_tot = fmaxf(m_tot, load_agent(&part_ml[((first_part + sp) * groups + g) * 2]));
    float l = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const float f = m_tot > -INFINITY ? __builtin_amdgcn_exp2f(load_agent(&part_ml[((first_part + sp) * groups + g) * 2]) - m_tot) : 0.f;
      scale_s[g][sp] = f;
      l += f * load_agent(&part_ml[((first_part + sp) * groups + g) * 2 + 1]);
    }
    inv_l[g] = l > 0.f ? 1.f / l : 0.f;
  }
  __syncthreads();
  for (int e = tid; e < groups * D; e += 256) {
    const int g = e / D, d = e - g * D;
    float ov = 0.f;
    for (int sp = 0; sp < splits; ++sp) ov += scale_s[g][sp] * load_agent(&part_o[((first_part + sp) * groups + g) * D + d]);
    out[(size_t)q0 * out_stride + (size_t)(hk * groups + g) * D + d] = float_to_bf16(ov * inv_l[g]);
  }
}

// Sequences with one query token only; others are left untouched.  Pages: keys
// [blocks][kv_heads][block_size][D], values transposed [blocks][kv_heads][D][block_size];
// block_size a power of two >= 16.  splits > 1 (at most 64) needs part_o [num_seqs * kv_heads * splits * groups * head_dim] and
// part_ml [num_seqs * kv_heads * splits * groups * 2] floats, and counters [num_seqs * kv_heads]
// ints that are zero before the first launch; every launch leaves them zero again.  Launches that
// share counters must not overlap.
extern "C" int fe_paged_attention_decode(const void* q, long long q_stride, const void* key_pages,
                                         const void* value_pages, void* out, long long out_stride,
                                         float* part_o, float* part_ml, int* counters, const int* cu_q,
                                         const int* ctx_len, const int* block_table, int table_stride,
                                         int num_seqs, int kv_heads, int groups, int head_dim,
                                         int block_size, int num_blocks, int window, float scale,
                                         int splits, hipStream_t stream) {
  if (num_seqs <= 0) return FE_OK;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return FE_BAD_ARGUMENT;
  if (groups < 1 || groups > GMAX || kv_heads < 1 || kv_heads > 65535 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < 16 || (block_size & (block_size - 1)) || num_blocks < 1 || table_stride < 1) return FE_BAD_ARGUMENT;
  int block_shift = 0;
  while ((1 << block_shift) < block_size) ++block_shift;
  if (q_stride % 8 || splits < 1 || splits > 64) return FE_BAD_ARGUMENT;
  if (splits > 1 && (!part_o || !part_ml || !counters)) return FE_BAD_ARGUMENT;
  dim3 grid(splits, kv_heads, num_seqs);
  const float scale_log2 = scale * 1.4426950408889634f;
#define FE_GO(DD)                                                                                          \
  paged_decode_kernel<DD><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)key_pages,    \
      (const bf16_t*)value_pages, (bf16_t*)out, out_stride, part_o, part_ml, counters, cu_q, ctx_len, block_table,     \
      table_stride, kv_heads, groups, block_shift, num_blocks, window, scale_log2)
  if (head_dim == 64) FE_GO(64);
  else if (head_dim == 128) FE_GO(128);
  else FE_GO(256);
#undef FE_GO
  return fe_check_launch();
}
