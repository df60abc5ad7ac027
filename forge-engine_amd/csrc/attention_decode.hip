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
//
// The PREPARE variant takes the raw output of the fused q/k/v projection instead of finished
// queries and does on the way what a kernel of its own would do before it: RMSNorm over each
// q and k head, rotation by the token's position, and the write of the new key and value into
// their pages.  The new token's own key never comes back from memory: the last key split
// treats it as a fifth partial result (score q.k_new, weight 1, value v_new) beside those of
// its four waves.  The arithmetic is the stand-alone kernel's (rope_math.h), so the cache
// holds the same bits whichever kernel wrote them.
#include "common.h"
#include "rope_math.h"

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

// Two neighbouring output elements from up to N splits: all loads first (the pair of partial
// outputs as one 8-byte load), then the sums in split order.
template <int N>
__device__ __forceinline__ unsigned int merge_few(const float* part_o, const float* part_ml, size_t first_part,
                                                  int splits, int groups, int g, int dim, int d) {
  float m[N], l[N];
  unsigned long long o[N];
#pragma unroll
  for (int sp = 0; sp < N; ++sp) {
    const size_t row = (first_part + (sp < splits ? sp : 0)) * groups + g;
    m[sp] = load_agent(&part_ml[row * 2]);
    l[sp] = load_agent(&part_ml[row * 2 + 1]);
    o[sp] = __hip_atomic_load((const unsigned long long*)&part_o[row * dim + d], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  float m_tot = -INFINITY;
#pragma unroll
  for (int sp = 0; sp < N; ++sp) m_tot = fmaxf(m_tot, sp < splits ? m[sp] : -INFINITY);
  float l_tot = 0.f, ov0 = 0.f, ov1 = 0.f;
#pragma unroll
  for (int sp = 0; sp < N; ++sp) {
    const float f = (sp < splits && m_tot > -INFINITY) ? __builtin_amdgcn_exp2f(m[sp] - m_tot) : 0.f;
    l_tot += f * l[sp];
    ov0 += f * __uint_as_float((unsigned int)o[sp]);
    ov1 += f * __uint_as_float((unsigned int)(o[sp] >> 32));
  }
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  return (unsigned int)float_to_bf16(ov0 * inv) | ((unsigned int)float_to_bf16(ov1 * inv) << 16);
}

// What the PREPARE variant needs beyond the plain one: the norms' weights (null: no norm), the
// rotation's frequencies [D / 2], and the pages as writable memory.
struct Prepare {
  const float* q_weight;
  const float* k_weight;
  const float* inv_freq;
  float eps;
  // the projection's output as float32 partial sums [num_sums][rows][q_stride] instead of one
  // bfloat16 matrix (a product whose K was split over blocks): added up in order and rounded here
  const float* sums;
  int num_sums;
  long long sum_stride;
};
#define MAX_SUMS 4

// MODE 0: finished queries; 1: PREPARE from the projection's bfloat16 output; 2: PREPARE from its
// float32 partial sums.
template <int D, int MODE>
__global__ __launch_bounds__(256, D <= 128 ? 2 : 1) void paged_decode_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* key_pages,
    const bf16_t* value_pages, bf16_t* __restrict__ out, long long out_stride,
    float* part_o, float* part_ml, int* __restrict__ counters, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const int* __restrict__ block_table, int table_stride,
    int kv_heads, int groups, int block_shift, int num_blocks, int window, float scale_log2,
    Prepare prep) {
  constexpr bool PREPARE = MODE != 0, FROM_SUMS = MODE == 2;
  const int block_size = 1 << block_shift, block_mask = block_size - 1;
  constexpr int KC = D / 32;        // MFMA k-steps over the head dim (scores)
  constexpr int DT = D / 16;        // 16-dim tiles of the output
  constexpr int PARTS = WAVES + (PREPARE ? 1 : 0);   // partial results that meet in LDS
  __shared__ float Ow[PARTS][GMAX][D];
  __shared__ float Ms[PARTS][GMAX], Ls[PARTS][GMAX];

  const int split = blockIdx.x, splits = gridDim.x;
  const int hk = blockIdx.y, seq = blockIdx.z;
  const int q0 = cu_q[seq];
  if (cu_q[seq + 1] - q0 != 1) return;
  const int ctx = ctx_len[seq];
  const int cached = PREPARE ? ctx - 1 : ctx;             // keys that the loop below reads from the pages
  const int k_begin = window > 0 ? max(0, ctx - window) : 0;
  const int first = k_begin / KEYS;
  const int last = (cached + KEYS - 1) / KEYS;            // exclusive
  const int per_split = (last - first + splits - 1) / splits;
  const int my_first = first + split * per_split;
  const int my_last = min(last, my_first + per_split);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lq = lane >> 4;

  // Everything that depends on nothing but the sequence's length is requested before any of it
  // is used, every load unconditional (out-of-range indices read a valid address and the value is
  // dropped): the rotation's frequency of this thread, the projection's output (or its partial
  // sums) for this block's heads, and the page ids of the wave's first two blocks of keys.  A
  // load under a condition would become a branch, and where branches meet the compiler waits for
  // every load in flight.
  __shared__ float cos_s[PREPARE ? D / 2 : 1], sin_s[PREPARE ? D / 2 : 1];
  __shared__ __attribute__((aligned(16))) bf16_t raw_s[FROM_SUMS ? (GMAX + 2) * D : 8];
  float frequency = 0.f;
  // the norms' weights of this lane's elements too (without a norm: any valid address, not used):
  // asked for after the keys they would be answered after the keys, and the queries' preparation
  // would wait for both
  float4 q_w[PREPARE ? KC : 1][2], k_w[2];
  if constexpr (PREPARE) {
    frequency = prep.inv_freq[min(tid, D / 2 - 1)];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const float* at = prep.q_weight ? prep.q_weight + c * 32 + lq * 8 : prep.inv_freq;
      q_w[c][0] = *(const float4*)at;
      q_w[c][1] = *(const float4*)(at + 4);
    }
    const float* at = prep.k_weight ? prep.k_weight + (lane & (D / 8 - 1)) * 8 : prep.inv_freq;
    k_w[0] = *(const float4*)at;
    k_w[1] = *(const float4*)(at + 4);
  }

  // partial sums: pieces of four elements of this block's query heads, key head and value head
  constexpr int PIECE_ROUNDS = FROM_SUMS ? ((GMAX + 2) * (D / 4) + 255) / 256 : 1;
  float4 part[PIECE_ROUNDS][MAX_SUMS];
  if constexpr (FROM_SUMS) {
#pragma unroll
    for (int round = 0; round < PIECE_ROUNDS; ++round) {
      const int piece = min(tid + round * 256, (groups + 2) * (D / 4) - 1);
      const int head = piece / (D / 4), d = (piece - head * (D / 4)) * 4;
      const int column_head = head < groups ? hk * groups + head
                                            : kv_heads * groups + (head - groups) * kv_heads + hk;
      const float* src = prep.sums + (size_t)q0 * q_stride + (size_t)column_head * D + d;
#pragma unroll
      for (int i = 0; i < MAX_SUMS; ++i) part[round][i] = *(const float4*)(src + (size_t)min(i, prep.num_sums - 1) * prep.sum_stride);
    }
  }

  // query rows as the B operand: lane (lr = row g, lq) holds q[g][32c + 8lq .. +8]; rows beyond
  // the group read row 0 again, their scores and outputs are never stored
  bf16x8 qb[KC];
  if constexpr (!FROM_SUMS) {
    const bf16_t* qrow = q + (size_t)q0 * q_stride + (size_t)(hk * groups + (lr < groups ? lr : 0)) * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) qb[c] = *(const bf16x8*)(qrow + c * 32 + lq * 8);
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
  auto checked = [&](int id, int key) -> int { return (key < cached && id >= 0 && id < num_blocks) ? id : 0; };
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
    // Which of these eight keys lie inside [k_begin, cached): the values of the others are set
    // to zero below.  Their probabilities are zero anyway, but a slot that no live key owns may
    // hold anything (a NaN that an earlier request left there), and 0 * NaN is NaN.
    const int v_hi = min(max(cached - vkey, 0), 8), v_lo = min(max(k_begin - vkey, 0), 8);
    const unsigned int v_bits = ((1u << v_hi) - 1u) & ~((1u << v_lo) - 1u);
    uintx4 v_mask;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v_mask[i] = (((v_bits >> (2 * i)) & 1u) ? 0x0000ffffu : 0u) | (((v_bits >> (2 * i + 1)) & 1u) ? 0xffff0000u : 0u);
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
      s[j] = (key >= k_begin && key < cached) ? v : -INFINITY;
      mx = fmaxf(mx, s[j]);
    }
    mx = max_xor16(mx);
    mx = max_xor32(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new > -INFINITY ? m_new : 0.f;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s[j] = __builtin_amdgcn_exp2f(s[j] - m_use);
      sum += s[j];
    }
    sum = sum_xor16(sum);
    sum = sum_xor32(sum);
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
      const uintx4 vt = va[t] & v_mask;
      o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vt), pb, o[t], 0, 0, 0);
    }
  };

  uintx4 k0[2][KC], k1[2][KC];
  const int b0 = my_first + wave;
  // raw page ids: values of this / the next block, keys of the next two (valid addresses whatever b0 is)
  int v0 = raw_page(b0 * KEYS + 8 * lq);
  const int kraw0 = raw_page(b0 * KEYS + krow);
  int kr1 = raw_page((b0 + WAVES) * KEYS + krow);
  int v1 = raw_page((b0 + WAVES) * KEYS + 8 * lq);
  int kr0 = 0;
  fetch_keys(b0, checked(kraw0, b0 * KEYS + krow), k0);

  // What the requests above brought, while the keys are on their way: the rotation's cosines and
  // sines of this token once per block, and the projection's output added up and rounded.
  if constexpr (PREPARE) {
    if (tid < D / 2) {
      float sn, cs;
      sincosf((float)(ctx - 1) * frequency, &sn, &cs);
      cos_s[tid] = cs;
      sin_s[tid] = sn;
    }
  }
  if constexpr (FROM_SUMS) {
#pragma unroll
    for (int round = 0; round < PIECE_ROUNDS; ++round) {
      const int piece = tid + round * 256;
      float4 sum = part[round][0];
#pragma unroll
      for (int i = 1; i < MAX_SUMS; ++i)
        if (i < prep.num_sums) { sum.x += part[round][i].x; sum.y += part[round][i].y; sum.z += part[round][i].z; sum.w += part[round][i].w; }
      uint2 packed;
      packed.x = (uint32_t)float_to_bf16(sum.x) | ((uint32_t)float_to_bf16(sum.y) << 16);
      packed.y = (uint32_t)float_to_bf16(sum.z) | ((uint32_t)float_to_bf16(sum.w) << 16);
      if (piece < (groups + 2) * (D / 4)) *(uint2*)&raw_s[piece * 4] = packed;
    }
  }

  bool extra = false;       // this block also brings the new token's own key and value
  if constexpr (PREPARE) {
    __syncthreads();        // cos_s, sin_s, raw_s (the keys requested above stay in flight)
    if constexpr (FROM_SUMS) {
#pragma unroll
      for (int c = 0; c < KC; ++c) qb[c] = *(const bf16x8*)&raw_s[(lr < groups ? lr : 0) * D + c * 32 + lq * 8];
    }
    // Queries: chunk 4c + lq of head row lr sits in qb[c].  Norm, rotation and rounding as the
    // stand-alone kernel does them: the butterfly over chunks runs over c first, then over lq.
    float qv[KC][8];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const uintx4 raw = __builtin_bit_cast(uintx4, qb[c]);
      const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
      unpack_bf16x8(w4, qv[c]);
    }
    if (prep.q_weight) {
      float total[KC];
#pragma unroll
      for (int c = 0; c < KC; ++c) total[c] = sum_squares8(qv[c]);
#pragma unroll
      for (int offset = KC / 2; offset > 0; offset >>= 1) {
        float next[KC];
#pragma unroll
        for (int c = 0; c < KC; ++c) next[c] = total[c] + total[c ^ offset];
#pragma unroll
        for (int c = 0; c < KC; ++c) total[c] = next[c];
      }
      float sumsq = total[0];
      sumsq = sum_xor32(sumsq);
      sumsq = sum_xor16(sumsq);
      const float inv = inverse_rms(sumsq, D, prep.eps);
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const float4 wa = q_w[c][0], wb = q_w[c][1];
        const float w8[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) qv[c][e] = normalise(qv[c][e], inv, w8[e]);
      }
    }
#pragma unroll
    for (int c = 0; c < KC / 2; ++c) {
      float lo[8], hi[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float cs = cos_s[c * 32 + lq * 8 + e], sn = sin_s[c * 32 + lq * 8 + e];
        lo[e] = rotate_low(qv[c][e], qv[c + KC / 2][e], cs, sn);
        hi[e] = rotate_high(qv[c + KC / 2][e], qv[c][e], cs, sn);
      }
      uint32_t pl[4], ph[4];
      pack_bf16x8(lo, pl);
      pack_bf16x8(hi, ph);
      qb[c] = __builtin_bit_cast(bf16x8, uintx4{pl[0], pl[1], pl[2], pl[3]});
      qb[c + KC / 2] = __builtin_bit_cast(bf16x8, uintx4{ph[0], ph[1], ph[2], ph[3]});
    }

    // The new token's key and value: made by the last wave of the last split (the one with the
    // least other work), written to their pages, and kept in LDS as a partial result of their
    // own: score q.k_new, weight 1, value v_new.
    extra = split == splits - 1;
    if (extra && wave == WAVES - 1) {
      constexpr int LPH = D / 8;                 // lanes that share a head, 8 elements each
      __shared__ __attribute__((aligned(16))) bf16_t new_key[D];
      const int sub = lane & (LPH - 1);
      const int role = lane / LPH;               // 0: key, 1: value, others idle (they follow the key's path)
      const int pos = ctx - 1;
      const bf16_t* row = q + (size_t)q0 * q_stride;
      const size_t k_at = (size_t)(kv_heads * groups + hk) * D, v_at = k_at + (size_t)kv_heads * D;
      uint4 raw;
      if constexpr (FROM_SUMS) raw = *(const uint4*)&raw_s[(groups + (role == 1 ? 1 : 0)) * D + sub * 8];
      else raw = *(const uint4*)(row + (role == 1 ? v_at : k_at) + sub * 8);
      const int block = table[min(pos >> block_shift, table_last)];
      const bool writable = block >= 0 && block < num_blocks;     // the host reserves pages before the launch
      const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
      float v[8];
      unpack_bf16x8(w4, v);
      if (prep.k_weight) {
        float sumsq = sum_squares8(v);
#pragma unroll
        for (int offset = LPH / 2; offset > 0; offset >>= 1) sumsq += __shfl_xor(sumsq, offset, FE_WAVE);
        const float inv = inverse_rms(sumsq, D, prep.eps);
        const float4 wa = k_w[0], wb = k_w[1];
        const float w8[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = normalise(v[e], inv, w8[e]);
      }
      const bool low = sub * 8 < D / 2;
      float r[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float other = __shfl_xor(v[e], LPH / 2, FE_WAVE);
        const int j = (sub * 8 + e) & (D / 2 - 1);
        r[e] = low ? rotate_low(v[e], other, cos_s[j], sin_s[j]) : rotate_high(v[e], other, cos_s[j], sin_s[j]);
      }
      uint32_t k4[4];
      pack_bf16x8(r, k4);
      const size_t page = (size_t)(writable ? block : 0) * kv_heads + hk;
      if (role == 0) {
        *(uint4*)&new_key[sub * 8] = make_uint4(k4[0], k4[1], k4[2], k4[3]);
        if (writable)
          *(uint4*)(const_cast<bf16_t*>(key_pages) + ((page << block_shift) + (pos & block_mask)) * D + sub * 8) =
              make_uint4(k4[0], k4[1], k4[2], k4[3]);
      } else if (role == 1) {
        bf16_t* vdst = const_cast<bf16_t*>(value_pages) + ((page * D) << block_shift) + (pos & block_mask);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const bf16_t bits = (bf16_t)(e & 1 ? w4[e >> 1] >> 16 : w4[e >> 1] & 0xffffu);
          if (writable) vdst[(size_t)(sub * 8 + e) << block_shift] = bits;
          for (int g = 0; g < groups; ++g) Ow[WAVES][g][sub * 8 + e] = bf16_to_float(bits);
        }
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();                     // new_key is read by other lanes of this wave
      float dot = 0.f;
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const uint4 kraw = *(const uint4*)&new_key[c * 32 + lq * 8];
        const uintx4 qraw = __builtin_bit_cast(uintx4, qb[c]);
        const uint32_t kw[4] = {kraw.x, kraw.y, kraw.z, kraw.w}, qw[4] = {qraw.x, qraw.y, qraw.z, qraw.w};
        float kf[8], qf[8];
        unpack_bf16x8(kw, kf);
        unpack_bf16x8(qw, qf);
#pragma unroll
        for (int e = 0; e < 8; ++e) dot = __fmaf_rn(qf[e], kf[e], dot);
      }
      dot = sum_xor16(dot);
      dot = sum_xor32(dot);
      if (lq == 0 && lr < groups) { Ms[WAVES][lr] = dot * scale_log2; Ls[WAVES][lr] = 1.f; }
    }
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
    if (PREPARE && extra) m_tot = fmaxf(m_tot, Ms[PARTS - 1][g]);
    float ov = 0.f, l = 0.f;
    if (m_tot > -INFINITY) {
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float f = __builtin_amdgcn_exp2f(Ms[w][g] - m_tot);
        ov += f * Ow[w][g][d];
        l += f * Ls[w][g];
      }
      if (PREPARE && extra) {
        const float f = __builtin_amdgcn_exp2f(Ms[PARTS - 1][g] - m_tot);
        ov += f * Ow[PARTS - 1][g][d];
        l += f * Ls[PARTS - 1][g];
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
  // parts are written and read with device-scope accesses that go past the per-die L2 caches,
  // every wave waits until its own stores are acknowledged, the barrier gathers the waves, then
  // one thread counts the block in; whoever counts last reads all parts.  The counter is a
  // relaxed atomic: in the language's memory model nothing orders the parts before the count.
  // What orders them is this hardware: a device-scope store is acknowledged only once it is
  // visible at the memory side that all dies share, so after the wait and the barrier every part
  // of this block is visible there before its count is, and the last block's device-scope loads
  // read from there.  An acquire-release counter at device scope would say the same in the model
  // but costs a cache write-back and invalidate in every block (measured: 16.2 instead of 14.1 us
  // a launch at 8 sequences); a cache-wide fence serialises across all blocks (0.3 us per block).
  // The counter goes back to zero for the next launch.
  __shared__ int is_last;
  __shared__ float scale_s[GMAX][64];   // weight of each split per query row
  __shared__ float inv_l[GMAX];
  __builtin_amdgcn_s_waitcnt((0x0) | (0x7 << 4) | (0xF << 8));    // vmcnt(0): this wave's stores have been acknowledged
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
  if (splits <= 16) {
    // few splits: every thread reads the statistics of its row itself, together with its share
    // of the partial outputs, so that all loads are in flight at once (same sums, same order)
    for (int e = 2 * tid; e < groups * D; e += 512) {
      const int g = e / D, d = e - g * D;
      unsigned int* dst = (unsigned int*)(out + (size_t)q0 * out_stride + (size_t)(hk * groups + g) * D + d);
      if (splits <= 4) *dst = merge_few<4>(part_o, part_ml, first_part, splits, groups, g, D, d);
      else if (splits <= 8) *dst = merge_few<8>(part_o, part_ml, first_part, splits, groups, g, D, d);
      else *dst = merge_few<16>(part_o, part_ml, first_part, splits, groups, g, D, d);
    }
    return;
  }
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

static int launch_decode(const void* q, long long q_stride, const void* key_pages, const void* value_pages,
                         void* out, long long out_stride, float* part_o, float* part_ml, int* counters,
                         const int* cu_q, const int* ctx_len, const int* block_table, int table_stride,
                         int num_seqs, int kv_heads, int groups, int head_dim, int block_size,
                         int num_blocks, int window, float scale, int splits, const Prepare* prep,
                         hipStream_t stream) {
  if (num_seqs <= 0) return FE_OK;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return FE_BAD_ARGUMENT;
  if (groups < 1 || groups > GMAX || kv_heads < 1 || kv_heads > 65535 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < 16 || (block_size & (block_size - 1)) || num_blocks < 1 || table_stride < 1) return FE_BAD_ARGUMENT;
  int block_shift = 0;
  while ((1 << block_shift) < block_size) ++block_shift;
  if (q_stride % 8 || out_stride % 2 || splits < 1 || splits > 64) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)out) & 3) || (((uintptr_t)part_o) & 7)) return FE_BAD_ARGUMENT;   // pairs of outputs, pairs of partial sums
  if ((((uintptr_t)q) | ((uintptr_t)key_pages) | ((uintptr_t)value_pages)) & 15) return FE_BAD_ARGUMENT;
  if (splits > 1 && (!part_o || !part_ml || !counters)) return FE_BAD_ARGUMENT;
  dim3 grid(splits, kv_heads, num_seqs);
  const float scale_log2 = scale * 1.4426950408889634f;
  const Prepare none = {nullptr, nullptr, nullptr, 0.f, nullptr, 0, 0};
#define FE_GO(DD, MODE)                                                                                    \
  paged_decode_kernel<DD, MODE><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)key_pages, \
      (const bf16_t*)value_pages, (bf16_t*)out, out_stride, part_o, part_ml, counters, cu_q, ctx_len, block_table,     \
      table_stride, kv_heads, groups, block_shift, num_blocks, window, scale_log2, MODE ? *prep : none)
  if (prep && prep->num_sums > 0) {
    if (head_dim == 64) FE_GO(64, 2);
    else if (head_dim == 128) FE_GO(128, 2);
    else FE_GO(256, 2);
  } else if (prep) {
    if (head_dim == 64) FE_GO(64, 1);
    else if (head_dim == 128) FE_GO(128, 1);
    else FE_GO(256, 1);
  } else {
    if (head_dim == 64) FE_GO(64, 0);
    else if (head_dim == 128) FE_GO(128, 0);
    else FE_GO(256, 0);
  }
#undef FE_GO
  return fe_check_launch();
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
  return launch_decode(q, q_stride, key_pages, value_pages, out, out_stride, part_o, part_ml, counters, cu_q,
                       ctx_len, block_table, table_stride, num_seqs, kv_heads, groups, head_dim, block_size,
                       num_blocks, window, scale, splits, nullptr, stream);
}

// The same for a batch in which EVERY sequence brings one token, straight from the fused
// projection's output qkv [num_seqs rows of (kv_heads * groups + 2 * kv_heads) * head_dim, row
// stride q_stride]: q and k heads are normalised (weights [head_dim] float32, null: no norm)
// and rotated whole by position ctx_len - 1 (inv_freq [head_dim / 2]), and each sequence's new
// key and value are written to slot ctx_len - 1 of its pages.  qkv itself is not changed.
// qkv_sums > 0 (at most 4): qkv is float32 and holds that many partial sums of the projection,
// sum_stride floats apart, each [num_seqs rows, row stride q_stride]; they are added up in order
// and rounded to bfloat16 first.
extern "C" int fe_paged_attention_decode_prepare(const void* qkv, int qkv_sums, long long sum_stride,
                                                 long long q_stride, const float* q_weight,
                                                 const float* k_weight, const float* inv_freq, float eps,
                                                 void* key_pages, void* value_pages, void* out,
                                                 long long out_stride, float* part_o, float* part_ml,
                                                 int* counters, const int* cu_q, const int* ctx_len,
                                                 const int* block_table, int table_stride, int num_seqs,
                                                 int kv_heads, int groups, int head_dim, int block_size,
                                                 int num_blocks, int window, float scale, int splits,
                                                 hipStream_t stream) {
  if (!inv_freq || (!q_weight) != (!k_weight)) return FE_BAD_ARGUMENT;
  if (q_weight && ((((uintptr_t)q_weight) | ((uintptr_t)k_weight)) & 15)) return FE_BAD_ARGUMENT;
  if (q_stride < (long long)(kv_heads * groups + 2 * kv_heads) * head_dim) return FE_BAD_ARGUMENT;
  if (qkv_sums < 0 || qkv_sums > MAX_SUMS) return FE_BAD_ARGUMENT;
  if (qkv_sums > 0 && (q_stride % 4 || sum_stride % 4 || sum_stride < (long long)num_seqs * q_stride)) return FE_BAD_ARGUMENT;
  const Prepare prep = {q_weight, k_weight, inv_freq, eps, qkv_sums > 0 ? (const float*)qkv : nullptr, qkv_sums, sum_stride};
  return launch_decode(qkv, q_stride, key_pages, value_pages, out, out_stride, part_o, part_ml, counters, cu_q,
                       ctx_len, block_table, table_stride, num_seqs, kv_heads, groups, head_dim, block_size,
                       num_blocks, window, scale, splits, &prep, stream);
}
