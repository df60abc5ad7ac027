// Paged grouped-query attention for portions of prompts (two or more query
// tokens of one sequence in a step), bfloat16 cache, on the matrix cores.
//
// Block = 64 query tokens of one query head of one sequence, four waves of 16
// rows; keys and values are walked in tiles of 64, shared by the waves in LDS.
// Long walks take blocks of eight waves (KG = 2): two groups of four waves with
// LDS buffers of their own walk every other tile each and merge their results
// at the end, which halves the chain of dependent tiles that the longest block
// of a launch is (one prompt of 2,048 tokens: all blocks are resident at once
// and the one with 32 tiles sets the time).
//   S^T = K Q^T    MFMA 16x16x32, A = 16 keys from LDS, B = 16 query rows held
//                  in registers for the whole kernel.  The 32 keys of a block
//                  feed two MFMA tiles whose rows interleave in groups of four,
//                  so lane group lq gets the scores of keys 8lq .. 8lq+7 of
//                  its query row: already the B operand of the next product;
//   softmax        float32, online over tiles, base-2 exponent with the scale
//                  folded in; a row's keys sit in four lanes (two shuffles);
//                  the causal (and window) mask only on tiles that cross it;
//   O^T += V^T P^T MFMA 16x16x32, A = 16 dims x 32 keys from LDS (the value
//                  pages are stored transposed, [D][slot], for this), B = P^T
//                  (bfloat16, straight from the score registers).
// Query token i of the step sits at position ctx_before + i and sees keys
// max(0, p - window + 1) .. p.  Sequences with fewer than two query tokens are
// skipped (the decode kernel serves them).  Sums and statistics are float32; P
// is rounded to bfloat16 for the second product, as the reference rounds its
// probabilities (src/forge_engine/qwen3.py:200).
//
// A tile reaches LDS by `global_load_lds_dwordx4`, which writes 64 lanes x 16
// bytes at consecutive LDS addresses without passing through registers: no
// staging registers (four waves fit a SIMD) and no LDS store instructions.
// Which global bytes a lane loads is free, which LDS address they land at is
// not; hence
//   keys    LDS unit u = 16-byte chunk position u % CH of key row u / CH holds
//           chunk (u % CH) ^ swizzle(row) of that row (conflict-free reads for the
//           interleaved rows of the MFMA operand, coalesced 256-byte rows in memory);
//   values  LDS unit u = dim u % D of key chunk u / D (8 keys): the 16 lanes that
//           read one chunk of 16 dims hit 16 neighbouring units.
// A wave loads the 16 keys 16w .. 16w+15 of a tile and their values: one page a
// wave and tile (pages hold at least 16 keys), its id fetched a tile ahead by a
// scalar load.  One LDS buffer for keys and one for values, two barriers a tile:
// once every wave has its scores, the tile's values and the next tile's keys are
// requested and fly during the softmax; they are waited for before the second
// product.
//
// Keys at or beyond the context read the bytes of the last key instead (their
// scores are masked; their probabilities are zero).  A slot that no live key owns
// may hold anything (a NaN that an earlier request left there), and 0 * NaN is NaN:
// in the tiles that cross the context or the window's lower edge the values of such
// slots are set to zero in LDS before the second product (and below a window the
// values' loads are moved up to the first visible key's chunk, so that no page is
// read that was given back).
#include "common.h"
#include <algorithm>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

#define BN 64        // keys per tile
#define XCDS 8
#define RESCALE_MARGIN 8.f   // base-2 units a row's maximum may exceed the exponents' reference point

__device__ __forceinline__ unsigned int pack_bf16(float lo, float hi) {
  const bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(unsigned int, v);
}

// rows 8a + b (+ 4h) are read together: 4a + b is distinct for them
__device__ __forceinline__ int key_swizzle(int row, int chunks) { return (((row >> 3) & 3) * 4 + (row & 3)) & (chunks - 1); }

// wait until at most n of this wave's vector memory operations are outstanding (n < 16)
#define FE_WAIT_VMEM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (0x7 << 4) | (0xF << 8))

__device__ __forceinline__ void load_to_lds(const void* global, void* lds) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                   (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// every lane gets the sum (the largest) of v over the wave, without a trip through LDS
__device__ __forceinline__ int wave_total(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);    // lane ^ 1
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);    // lane ^ 2
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);   // 7 - lane within 8
  v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);   // 15 - lane within 16
  auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
  v = (int)(r[0] + r[1]);
  r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
  return __builtin_amdgcn_readfirstlane((int)(r[0] + r[1]));
}
__device__ __forceinline__ int wave_most(int v) {
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));
  auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
  v = max((int)r[0], (int)r[1]);
  r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
  return __builtin_amdgcn_readfirstlane(max((int)r[0], (int)r[1]));
}

template <int D, int KG>
__global__ __launch_bounds__(256 * KG, 4) void paged_prefill_kernel(   // four waves a SIMD: at most 128 registers
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, long long out_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int table_stride, int kv_heads, int groups, int block_shift, int num_blocks, int window,
    float scale_log2, int num_seqs, int heads_per_xcd) {
  const int block_mask = (1 << block_shift) - 1;
  constexpr int BM = 64;
  constexpr int KC = D / 32;            // MFMA k-steps over the head dim (scores)
  constexpr int DT = D / 16;            // 16-dim tiles of the output
  constexpr int CH = D / 8;             // 16-byte chunks per key row
  constexpr int KI = BN * CH / 256;     // key load instructions per wave and tile
  constexpr int VI = 8 * D / 256;       // value load instructions per wave and tile
  __shared__ __attribute__((aligned(16))) uintx4 lds[KG * (BN * CH + 8 * D)];   // per key group: a tile of keys, a tile of values

  // The grid is heads x tile slots, a slot being a place for one 64-row tile of some sequence
  // (slots >= the tiles there are: the host knows the step's query tokens, not how they are spread
  // over the sequences), so a step whose work sits in one long portion among single tokens launches
  // few blocks that do nothing.  Slots go round by round: first the last tile of every sequence
  // (the longest walk over its keys), then the tile before it of every sequence that has one, and
  // so on, so that long walks start early and the blocks a CU holds at a time are a mix.
  // Block id b runs on XCD b % 8; with eight heads or more an XCD, with its own L2, takes a run of
  // neighbouring heads, which share keys and values, for every slot.
  const int heads = kv_heads * groups;
  int head, slot;
  if (heads_per_xcd > 0) {
    const int local = blockIdx.x / XCDS;
    head = (blockIdx.x % XCDS) * heads_per_xcd + local % heads_per_xcd;
    slot = local / heads_per_xcd;
  } else {
    head = blockIdx.x % heads;
    slot = blockIdx.x / heads;
  }
  if (head >= heads) return;
  int seq = 0, q_tile = -1;
  if (num_seqs <= FE_WAVE) {
    // lane s looks at sequence s; tiles before round r: the sum over sequences of min(tiles, r)
    const int me = threadIdx.x & (FE_WAVE - 1);
    const int len = cu_q[min(me, num_seqs - 1) + 1] - cu_q[min(me, num_seqs - 1)];
    const int tiles = me < num_seqs && len >= 2 ? (len + BM - 1) / BM : 0;
    if (slot >= wave_total(tiles)) return;
    int lo = 0, hi = wave_most(tiles);            // the round is in [lo, hi)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (wave_total(min(tiles, mid)) <= slot) lo = mid; else hi = mid;
    }
    const int rank = slot - wave_total(min(tiles, lo));          // among the sequences with a tile in this round
    const unsigned long long in_round = __ballot(tiles > lo);
    const int before_me = __builtin_popcountll(in_round & ((1ull << me) - 1ull));
    const unsigned long long mine = __ballot(tiles > lo && before_me == rank);
    seq = __builtin_amdgcn_readfirstlane(__builtin_ctzll(mine));
    q_tile = __builtin_amdgcn_readfirstlane(__shfl(tiles, seq, FE_WAVE)) - 1 - lo;
  } else {
    // more sequences than lanes: sequence by sequence, every other one's tiles in rising order
    for (int first = 0; seq < num_seqs; ++seq) {
      const int len = cu_q[seq + 1] - cu_q[seq];
      const int tiles = len >= 2 ? (len + BM - 1) / BM : 0;
      if (slot < first + tiles) { q_tile = (seq & 1) ? slot - first : tiles - 1 - (slot - first); break; }
      first += tiles;
    }
    if (q_tile < 0) return;
  }
  const int hk = head / groups;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int row0 = q_tile * BM;
  if (q_len < 2 || row0 >= q_len) return;
  const int ctx = ctx_len[seq];
  const int before = ctx - q_len;
  const int* table = block_table + (size_t)seq * table_stride;

  const int tid = threadIdx.x, lane = tid & 63;
  const int kg = __builtin_amdgcn_readfirstlane(tid >> 8);          // key group: walks tiles tile_first + kg, + KG, ...
  const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);  // within the group: 16 rows, a quarter of the loads
  uintx4* Ks = lds + kg * (BN * CH + 8 * D);
  uintx4* Vs = Ks + BN * CH;
  const int lr = lane & 15, lq = lane >> 4;
  const int krow = 8 * (lr >> 2) + (lr & 3);   // MFMA row r of key tile h is key 8*(r/4) + 4h + r%4 of its 32-key block

  // this wave's query rows as B operands: lane (lr = row, lq) holds q[row][32c + 8lq .. +8]
  bf16x8 qb[KC];
  const int row = row0 + wave * 16 + lr;
  const int row_pos = before + row;
  {
    const bf16_t* qrow = q + (size_t)(q0 + min(row, q_len - 1)) * q_stride + (size_t)head * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const uintx4 v = *(const uintx4*)(qrow + c * 32 + lq * 8);
      qb[c] = __builtin_bit_cast(bf16x8, row < q_len ? v : uintx4{0u, 0u, 0u, 0u});
    }
  }
  float m_run = -INFINITY;
  floatx4 l_sum = floatx4{0.f, 0.f, 0.f, 0.f};     // every entry: the row's sum of probabilities so far
  const bf16x8 ones = __builtin_bit_cast(bf16x8, uintx4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
  floatx4 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int last_row = min(q_len, row0 + BM) - 1;
  const int pos_lo = before + row0, pos_hi = before + last_row;
  const int wave_lo = pos_lo + wave * 16;
  const int k_first = window > 0 ? max(0, pos_lo - window + 1) : 0;
  const int tile_first = k_first / BN, tile_last = pos_hi / BN;   // inclusive
  const int last_key = ctx - 1;

  // the page of this wave's 16 keys of a tile (uniform over the wave)
  // Keys below the first visible one (a window) may lie in pages that were given back: the loads
  // of values are moved up to the 16-key group and 8-key chunk of the first visible key, which
  // hold this request's own keys; the keys' loads may read anything, their scores are replaced.
  const int low_group = k_first & ~15, low_chunk = k_first & ~7;
  auto page_of = [&](int tile) -> int {
    const int key = max(min(tile * BN + 16 * wave, last_key), low_group);
    const int id = table[key >> block_shift];
    return (id >= 0 && id < num_blocks) ? id : 0;
  };
  // per-lane constants of the loaders
  int k_row[KI], k_chunk[KI], v_dim[VI], v_first[VI];
#pragma unroll
  for (int i = 0; i < KI; ++i) {
    const int u = (wave * KI + i) * 64 + lane;
    k_row[i] = u / CH;
    k_chunk[i] = (u % CH) ^ key_swizzle(u / CH, CH);
  }
#pragma unroll
  for (int i = 0; i < VI; ++i) {
    const int u = (wave * VI + i) * 64 + lane;
    v_dim[i] = u % D;
    v_first[i] = (u / D) * 8;         // first key of the chunk within the tile
  }
  // A tile that lies wholly inside [first visible key's group, context) needs no clamping: the
  // address of a load is then a part that is uniform over the wave (page, kv head, where the wave's
  // 16 keys start in the page; scalar arithmetic) plus a part that never changes (the lane's place
  // among those 16 keys), so the tiles of the steady state cost no vector instructions for their
  // addresses.  The tiles at the edges take the general path.
  unsigned int k_lane[KI], v_lane[VI];
#pragma unroll
  for (int i = 0; i < KI; ++i) k_lane[i] = (unsigned int)((k_row[i] & 15) * D + k_chunk[i] * 8);
#pragma unroll
  for (int i = 0; i < VI; ++i) v_lane[i] = (unsigned int)((v_dim[i] << block_shift) + (v_first[i] & 15));
  auto inner = [&](int tile) -> bool { return tile * BN + BN <= ctx && tile * BN >= low_group; };
  auto load_keys = [&](int tile, int page) {
    const size_t base = ((size_t)page * kv_heads + hk) << block_shift;
    if (inner(tile)) {
      const bf16_t* from = key_pages + (base + ((tile * BN + 16 * wave) & block_mask)) * D;
#pragma unroll
      for (int i = 0; i < KI; ++i) load_to_lds(from + k_lane[i], &Ks[(wave * KI + i) * 64]);
      return;
    }
#pragma unroll
    for (int i = 0; i < KI; ++i) {
      const int key = min(tile * BN + k_row[i], last_key);
      load_to_lds(key_pages + (base + (key & block_mask)) * D + k_chunk[i] * 8, &Ks[(wave * KI + i) * 64]);
    }
  };
  auto load_values = [&](int tile, int page) {
    const size_t base = ((size_t)page * kv_heads + hk) * D;
    if (inner(tile)) {
      const bf16_t* from = value_pages + (base << block_shift) + ((tile * BN + 16 * wave) & block_mask);
#pragma unroll
      for (int i = 0; i < VI; ++i) load_to_lds(from + v_lane[i], &Vs[(wave * VI + i) * 64]);
      return;
    }
#pragma unroll
    for (int i = 0; i < VI; ++i) {
      const int key = max(min(tile * BN + v_first[i], last_key & ~7), low_chunk);
      load_to_lds(value_pages + ((base + v_dim[i]) << block_shift) + (key & block_mask), &Vs[(wave * VI + i) * 64]);
    }
  };

  // every group makes the same number of rounds (the barriers are the block's); a group without a
  // tile in a round only waits
  const int rounds = (tile_last - tile_first + KG) / KG;
  int tile = tile_first + kg;
  int page = page_of(min(tile, tile_last));
  if (tile <= tile_last) load_keys(tile, page);
  int page_next = tile + KG <= tile_last ? page_of(tile + KG) : 0;
  FE_WAIT_VMEM(0);
  __syncthreads();               // the first tile's keys are in LDS
  for (int round = 0; round < rounds; ++round, tile += KG) {
    const bool active = tile <= tile_last;
    const bool more = tile + KG <= tile_last;
    const int key_base = tile * BN;
    const bool mine = active && key_base <= wave_lo + 15;     // some key of the tile is visible to this wave's rows
    floatx4 st[2][2];
    if (mine) {
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int c = 0; c < KC; ++c) {
            const int r = blk * 32 + krow + 4 * h;
            const bf16x8 ka = __builtin_bit_cast(bf16x8, Ks[r * CH + ((c * 4 + lq) ^ key_swizzle(r, CH))]);
            st[blk][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                ka, qb[c], c == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : st[blk][h], 0, 0, 0);
          }
    }
    // Every wave has its scores, and multiplied the tile before: both buffers are free.  This
    // tile's values and the next tile's keys are requested now and fly during the softmax.
    __syncthreads();
    if (active) load_values(tile, page);
    if (more) {
      load_keys(tile + KG, page_next);
      page = page_next;
      if (tile + 2 * KG <= tile_last) page_next = page_of(tile + 2 * KG);
    }
    bf16x8 pb[2];
    if (mine) {
      // lane (lr = query row, lq): st[blk][h][i] = score of key key_base + 32 blk + 8lq + 4h + i
      const bool edge = key_base + BN - 1 > wave_lo || (window > 0 && key_base < pos_hi - window + 1);
      float s[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) s[j] = st[j >> 3][(j >> 2) & 1][j & 3];
      if (edge) {          // one branch a tile, not one a score: the tiles in the middle of a walk skip all of it
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int key = key_base + 32 * (j >> 3) + 8 * lq + (j & 7);
          const bool visible = key <= row_pos && (window <= 0 || key > row_pos - window);
          s[j] = visible ? s[j] : -INFINITY;
        }
      }
      // the largest of the lane's 16 scores as a tree (three-operand maxima), then across the four lanes of the row
      float mx = fmaxf(fmaxf(fmaxf(fmaxf(s[0], s[1]), s[2]), fmaxf(fmaxf(s[3], s[4]), s[5])),
                       fmaxf(fmaxf(fmaxf(s[6], s[7]), s[8]), fmaxf(fmaxf(s[9], s[10]), s[11])));
      mx = fmaxf(fmaxf(mx, fmaxf(fmaxf(s[12], s[13]), s[14])), s[15]);
      mx = max_xor16(mx);
      mx = max_xor32(mx);
      // The reference point of the exponents moves only when the row's maximum has outgrown it by more
      // than RESCALE_MARGIN (base-2 units): until then the probabilities of this tile are at most
      // 2^RESCALE_MARGIN instead of at most 1, which float32 sums and bfloat16 operands hold as well,
      // and the 32 products that rescale the output, and the wave's vote on them, are left out.  The
      // quotient at the end does not depend on the reference point.
      const float m_new = fmaxf(m_run, mx * scale_log2);   // the scale is positive
      const bool moved = m_new > m_run + RESCALE_MARGIN;   // (from -infinity: any finite maximum moves it)
      const float m_next = moved ? m_new : m_run;
      const float m_use = m_next > -INFINITY ? m_next : 0.f; // a row with nothing visible yet
      const float corr = moved ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) s[j] = __builtin_amdgcn_exp2f(fmaf(s[j], scale_log2, -m_use));
      m_run = m_next;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        uintx4 pw;
        pw.x = pack_bf16(s[8 * blk + 0], s[8 * blk + 1]); pw.y = pack_bf16(s[8 * blk + 2], s[8 * blk + 3]);
        pw.z = pack_bf16(s[8 * blk + 4], s[8 * blk + 5]); pw.w = pack_bf16(s[8 * blk + 6], s[8 * blk + 7]);
        pb[blk] = __builtin_bit_cast(bf16x8, pw);
      }
      if (__any(moved)) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[t][i] *= corr;
#pragma unroll
        for (int i = 0; i < 4; ++i) l_sum[i] *= corr;
      }
    }
    FE_WAIT_VMEM(0);
    if (__builtin_expect(active && (key_base + BN > ctx || key_base < k_first), 0)) {
      // The tile holds slots at or beyond the context (the 8-key chunk of the last key has them
      // behind it; later chunks are copies of that chunk) or below the first visible key.  Their
      // probabilities are zero, but a slot that no live key owns may hold anything (a NaN that
      // an earlier request left there), and 0 * NaN is NaN: every wave sets them to zero in the
      // part of the tile that it loaded itself, before the barrier hands the tile to the others.
      // At most twice per block (its first and its last tile); one 4-byte word (two keys) at a
      // time, so that the rare path needs no registers of the common one.
      const int above = ctx - key_base, below = k_first - key_base;   // keys of the tile inside [below, above) count
      unsigned int* words = (unsigned int*)Vs;
      for (int i = 0; i < VI; ++i) {
        const int u = (wave * VI + i) * 64 + lane;
        const int first_key = (u / D) * 8;
#pragma unroll 1
        for (int j = 0; j < 4; ++j) {
          const int k0 = first_key + 2 * j;
          const unsigned int keep = ((k0 >= below && k0 < above) ? 0x0000ffffu : 0u) |
                                    ((k0 + 1 >= below && k0 + 1 < above) ? 0xffff0000u : 0u);
          if (keep != 0xffffffffu) words[u * 4 + j] &= keep;
        }
      }
    }
    __syncthreads();             // the values (and the next keys) are in LDS
    if (mine) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          const bf16x8 va = __builtin_bit_cast(bf16x8, Vs[(blk * 4 + lq) * D + t * 16 + lr]);
          o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[blk], o[t], 0, 0, 0);
        }
      // the rows' sums of probabilities as one more output tile whose "values" are all one: the matrix
      // pipe has room, the vector pipe (16 additions and two exchanges a tile) has not; and the sum is
      // then of the probabilities as the product above sees them, rounded to bfloat16
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) l_sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[blk], l_sum, 0, 0, 0);
    }
  }

  float l_run = l_sum[0];
  if constexpr (KG == 2) {
    // the second group hands its running maximum, sum and output to the first through LDS (the
    // tiles' buffers are free now), value by value with the lanes side by side
    __syncthreads();
    float* hand = (float*)lds;
    const int slot = wave * 64 + lane;
    if (kg == 1) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) hand[(t * 4 + i) * 256 + slot] = o[t][i];
      hand[(DT * 4) * 256 + slot] = m_run;
      hand[(DT * 4 + 1) * 256 + slot] = l_run;
    }
    __syncthreads();
    if (kg == 1) return;
    const float m_other = hand[(DT * 4) * 256 + slot], l_other = hand[(DT * 4 + 1) * 256 + slot];
    const float m_all = fmaxf(m_run, m_other);
    const float f_mine = m_run > -INFINITY ? __builtin_amdgcn_exp2f(m_run - m_all) : 0.f;
    const float f_other = m_other > -INFINITY ? __builtin_amdgcn_exp2f(m_other - m_all) : 0.f;
    l_run = l_run * f_mine + l_other * f_other;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] = o[t][i] * f_mine + hand[(t * 4 + i) * 256 + slot] * f_other;
  }

  // lane (lr = query row, lq) holds O^T[16t + 4lq + i][row]: four consecutive dims per store
  if (row < q_len) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    bf16_t* orow = out + (size_t)(q0 + row) * out_stride + (size_t)head * D;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      uint2 w;
      w.x = pack_bf16(o[t][0] * inv, o[t][1] * inv);
      w.y = pack_bf16(o[t][2] * inv, o[t][3] * inv);
      *(uint2*)(orow + t * 16 + lq * 4) = w;
    }
  }
}

// Pages: keys [blocks][kv_heads][block_size][D], values transposed [blocks][kv_heads][D][block_size];
// block_size a power of two >= 16; head_dim 64 or 128.  Sequences with fewer than two query tokens
// are skipped.  key_groups: 1 or 2 groups of four waves a block (see the top of the file), 0 lets the launch
// choose, from total_q: the query tokens of all sequences together (the rows of q; the grid is laid out for
// num_seqs sequences of max_q_len tokens, of which a step with one long portion fills a fraction).
extern "C" int fe_paged_attention_prefill(const void* q, long long q_stride, const void* key_pages,
                                                 const void* value_pages, void* out, long long out_stride,
                                                 const int* cu_q, const int* ctx_len, const int* block_table,
                                                 int table_stride, int num_seqs, int max_q_len, int kv_heads,
                                                 int groups, int head_dim, int block_size, int num_blocks,
                                                 int window, float scale, int key_groups, int total_q,
                                                 hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len < 2) return FE_OK;
  if (head_dim != 64 && head_dim != 128) return FE_BAD_ARGUMENT;
  if (groups < 1 || kv_heads < 1 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < 16 || (block_size & (block_size - 1)) || num_blocks < 1 || table_stride < 1 || q_stride % 8 || out_stride % 4) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)key_pages) | ((uintptr_t)value_pages) | ((uintptr_t)q)) & 15) return FE_BAD_ARGUMENT;
  const float scale_log2 = scale * 1.4426950408889634f;
  int block_shift = 0;
  while ((1 << block_shift) < block_size) ++block_shift;
  const int heads = kv_heads * groups;
  const int heads_per_xcd = heads >= XCDS ? (heads + XCDS - 1) / XCDS : 0;
  if (total_q < 1) return FE_BAD_ARGUMENT;
  // places for 64-row tiles: a sequence of n tokens has at most n / 64 + 1, and the grid does not
  // depend on how the tokens are spread over the sequences (a captured launch serves every spread)
  const long long slots = std::min<long long>((long long)num_seqs * ((max_q_len + 63) / 64), total_q / 64 + num_seqs);
  const long long blocks = (heads_per_xcd ? (long long)heads_per_xcd * XCDS : heads) * slots;
  if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  const unsigned grid = (unsigned)blocks;
  // Two key groups a block where the launch would leave the chip underfilled (all its blocks
  // resident at once: then the longest walk sets the time, and halving it pays; measured: one
  // prompt of 2,048 tokens 72 -> 66 us, of 512 tokens 18 -> 14 us) and the portions span at least
  // two tiles; with more blocks than that one group is faster (eight prompts of 1,024 tokens:
  // 126 against 141 us).
  if (key_groups < 0 || key_groups > 2) return FE_BAD_ARGUMENT;
  // (counted by the tiles that the tokens can fill, not by the grid: a captured launch is laid out
  // for more sequences than a step brings, and a block without a tile ends at once)
  const long long filled = std::min<long long>(slots, (total_q + 63) / 64);
  if (key_groups == 0) key_groups = ((long long)heads * filled <= 1024 && max_q_len >= 128) ? 2 : 1;
#define FE_GO(DD, GG)                                                                                            \
  paged_prefill_kernel<DD, GG><<<grid, 256 * GG, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)key_pages, \
      (const bf16_t*)value_pages, (bf16_t*)out, out_stride, cu_q, ctx_len, block_table, table_stride,            \
      kv_heads, groups, block_shift, num_blocks, window, scale_log2, num_seqs, heads_per_xcd)
  if (head_dim == 64 && key_groups == 1) FE_GO(64, 1);
  else if (head_dim == 64) FE_GO(64, 2);
  else if (key_groups == 1) FE_GO(128, 1);
  else FE_GO(128, 2);
#undef FE_GO
  return fe_check_launch();
}
