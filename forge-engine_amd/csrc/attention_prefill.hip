// Paged grouped-query attention for portions of prompts (two or more query
// tokens of one sequence in a step), bfloat16 cache, on the matrix cores.
//
// Block = 64 or 128 query tokens of one query head of one sequence, four waves of
// RM = 1 or 2 sets of 16 rows; keys and values are walked in tiles of 64, shared by
// the waves in LDS.  With two sets of rows a fragment read from LDS feeds two MFMAs
// (with one, the LDS reads bound a tile and not the matrix pipe), at the price of
// twice the registers: two waves a SIMD instead of four.  Launches that leave the
// chip underfilled take blocks of eight waves (KG = 2): two groups of four waves with
// LDS buffers of their own walk every other tile each and merge their results at the
// end, which halves the chain of dependent tiles that the longest block of a launch is.
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
// scalar load.  Blocks of 64 rows: one LDS buffer for keys and one for values, two
// barriers a tile: once every wave has its scores, the tile's values and the next
// tile's keys are requested and fly during the softmax; they are waited for before
// the second product.  Blocks of 128 rows: two buffers each, one barrier a tile, the
// next tile requested a whole tile ahead.  In both the MFMA operands are read from
// LDS by inline assembly, three fragments ahead of their use, with the waits counted
// by hand.
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
#define ROWS2_MIN_LEN 256              // blocks of 128 rows: for portions of at least this many tokens ...
#define ROWS2_MIN_BLOCKS 768           // ... and launches of at least this many such blocks (three a CU)
#define KEY_GROUPS_MAX_BLOCKS 704      // two key groups a block: in launches of up to this many blocks of 64 rows
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

// 16 bytes from LDS byte address `at` + 256 * STEP; nothing waits for them here
template <int STEP>
__device__ __forceinline__ uintx4 lds_read16(unsigned int at) {
  uintx4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(STEP * 256) : "memory");
  return v;
}
// ... with a step that is a constant only once the loop around the call is unrolled
__device__ __forceinline__ uintx4 lds_read16_step(unsigned int at, int step) {
  switch (step) {
#define FE_CASE(I) case I: return lds_read16<I>(at);
#define FE_CASE8(I) FE_CASE(I) FE_CASE(I + 1) FE_CASE(I + 2) FE_CASE(I + 3) FE_CASE(I + 4) FE_CASE(I + 5) FE_CASE(I + 6) FE_CASE(I + 7)
    FE_CASE8(0) FE_CASE8(8) FE_CASE8(16) FE_CASE8(24) FE_CASE8(32) FE_CASE8(40) FE_CASE8(48) FE_CASE8(56)
#undef FE_CASE8
#undef FE_CASE
  }
  return uintx4{0u, 0u, 0u, 0u};
}
// wait until at most PENDING of this wave's LDS reads are outstanding; `v` is what the wait is for.
// (LDS reads return in order.  Whatever else the compiler has under way on the same counter, its own LDS
// accesses or a scalar load, makes such a wait stricter, never weaker; and its own waits, which do not
// know of the reads above, likewise.)
template <int PENDING>
__device__ __forceinline__ void lds_arrived(uintx4& v) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(PENDING));
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

template <int D, int KG, int RM>
__global__ __launch_bounds__(256 * KG, RM == 1 ? 4 : 2 / KG) void paged_prefill_kernel(   // RM = 1: four waves a SIMD (128 registers), RM = 2: two
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, long long out_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int table_stride, int kv_heads, int groups, int block_shift, int num_blocks, int window,
    float scale_log2, int num_seqs, int heads_per_xcd) {
  const int block_mask = (1 << block_shift) - 1;
  constexpr int BM = 64 * RM;
  constexpr int KC = D / 32;            // MFMA k-steps over the head dim (scores)
  constexpr int DT = D / 16;            // 16-dim tiles of the output
  constexpr int CH = D / 8;             // 16-byte chunks per key row
  constexpr int KI = BN * CH / 256;     // key load instructions per wave and tile
  constexpr int VI = 8 * D / 256;       // value load instructions per wave and tile
  constexpr int STAGES = RM;            // blocks of 128 rows keep two tiles of keys and values (see the walk below)
  __shared__ __attribute__((aligned(16))) uintx4 lds[KG * STAGES * (BN * CH + 8 * D)];   // per key group: STAGES x (a tile of keys, a tile of values)

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
    const int rank = slot - wave_total(min(tiles, lo));          // among the sequences that have a tile in round lo
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
  uintx4* group_lds = lds + kg * STAGES * (BN * CH + 8 * D);
  const int lr = lane & 15, lq = lane >> 4;
  const int krow = 8 * (lr >> 2) + (lr & 3);   // MFMA row r of key tile h is key 8*(r/4) + 4h + r%4 of its 32-key block

  // this wave's query rows, RM sets of 16, as B operands: lane (lr = row, lq) holds q[row][32c + 8lq .. +8]
  bf16x8 qb[RM][KC];
  int row[RM], row_pos[RM];
#pragma unroll
  for (int rm = 0; rm < RM; ++rm) {
    row[rm] = row0 + (wave * RM + rm) * 16 + lr;
    row_pos[rm] = before + row[rm];
    const bf16_t* qrow = q + (size_t)(q0 + min(row[rm], q_len - 1)) * q_stride + (size_t)head * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const uintx4 v = *(const uintx4*)(qrow + c * 32 + lq * 8);
      qb[rm][c] = __builtin_bit_cast(bf16x8, row[rm] < q_len ? v : uintx4{0u, 0u, 0u, 0u});
    }
  }
  float m_run[RM];
  floatx4 l_sum[RM];                               // every entry: the row's sum of probabilities so far
  const bf16x8 ones = __builtin_bit_cast(bf16x8, uintx4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
  floatx4 o[RM][DT];
#pragma unroll
  for (int rm = 0; rm < RM; ++rm) {
    m_run[rm] = -INFINITY;
    l_sum[rm] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < DT; ++t) o[rm][t] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  const int last_row = min(q_len, row0 + BM) - 1;
  const int pos_lo = before + row0, pos_hi = before + last_row;
  const int wave_lo = pos_lo + wave * 16 * RM;      // the position of the wave's first row; its last: + 16 RM - 1
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
  // what a lane's load instruction i brings: LDS unit u = (wave * KI + i) * 64 + lane of the keys is chunk
  // position u % CH of key row u / CH; unit u of the values is dim u % D of the 8-key chunk u / D
  auto key_row = [&](int i, int ln) { return ((wave * KI + i) * 64 + ln) / CH; };
  auto key_chunk = [&](int i, int ln) { const int u = (wave * KI + i) * 64 + ln; return (u % CH) ^ key_swizzle(u / CH, CH); };
  auto value_dim = [&](int i, int ln) { return ((wave * VI + i) * 64 + ln) % D; };
  auto value_first = [&](int i, int ln) { return (((wave * VI + i) * 64 + ln) / D) * 8; };      // first key of the chunk within the tile
  // (the tiles at the edges work these out again, from a lane number that the compiler cannot trace back:
  // kept for the whole walk they would take sixteen registers that its steady state does not use)
  auto lane_again = [&]() { int ln = lane; asm volatile("" : "+v"(ln)); return ln; };
  // A tile that lies wholly inside [first visible key's group, context) needs no clamping: the
  // address of a load is then a part that is uniform over the wave (page, kv head, where the wave's
  // 16 keys start in the page; scalar arithmetic) plus a part that never changes (the lane's place
  // among those 16 keys), so the tiles of the steady state cost no vector instructions for their
  // addresses.  The tiles at the edges take the general path.
  unsigned int k_lane[KI], v_lane[VI];
#pragma unroll
  for (int i = 0; i < KI; ++i) k_lane[i] = (unsigned int)((key_row(i, lane) & 15) * D + key_chunk(i, lane) * 8);
#pragma unroll
  for (int i = 0; i < VI; ++i) v_lane[i] = (unsigned int)((value_dim(i, lane) << block_shift) + (value_first(i, lane) & 15));
  auto inner = [&](int tile) -> bool { return tile * BN + BN <= ctx && tile * BN >= low_group; };
  auto load_keys = [&](int tile, int page, uintx4* Ks) {
    const size_t base = ((size_t)page * kv_heads + hk) << block_shift;
    if (inner(tile)) {
      const bf16_t* from = key_pages + (base + ((tile * BN + 16 * wave) & block_mask)) * D;
#pragma unroll
      for (int i = 0; i < KI; ++i) load_to_lds(from + k_lane[i], &Ks[(wave * KI + i) * 64]);
      return;
    }
    const int ln = lane_again();
#pragma unroll
    for (int i = 0; i < KI; ++i) {
      const int key = min(tile * BN + key_row(i, ln), last_key);
      load_to_lds(key_pages + (base + (key & block_mask)) * D + key_chunk(i, ln) * 8, &Ks[(wave * KI + i) * 64]);
    }
  };
  auto load_values = [&](int tile, int page, uintx4* Vs) {
    const size_t base = ((size_t)page * kv_heads + hk) * D;
    if (inner(tile)) {
      const bf16_t* from = value_pages + (base << block_shift) + ((tile * BN + 16 * wave) & block_mask);
#pragma unroll
      for (int i = 0; i < VI; ++i) load_to_lds(from + v_lane[i], &Vs[(wave * VI + i) * 64]);
      return;
    }
    const int ln = lane_again();
#pragma unroll
    for (int i = 0; i < VI; ++i) {
      const int key = max(min(tile * BN + value_first(i, ln), last_key & ~7), low_chunk);
      load_to_lds(value_pages + ((base + value_dim(i, ln)) << block_shift) + (key & block_mask), &Vs[(wave * VI + i) * 64]);
    }
  };

  // The softmax of one tile for one set of rows, in SOFTMAX_ITEMS pieces of a few instructions each:
  // the scores become the probabilities in place, then the second product's B operands, rounded to
  // bfloat16.
  // lane (lr = query row, lq): st[rm][blk][h][i] = score of key key_base + 32 blk + 8lq + 4h + i
  constexpr int SOFTMAX_ITEMS = 24;
  float item_mx[RM], item_m_use[RM], corr[RM];
  bool moved[RM];
#pragma unroll
  for (int rm = 0; rm < RM; ++rm) { item_mx[rm] = 0.f; item_m_use[rm] = 0.f; corr[rm] = 1.f; moved[rm] = false; }
  auto is_edge = [&](int key_base) { return key_base + BN - 1 > wave_lo || (window > 0 && key_base < pos_hi - window + 1); };
  auto mask_edges = [&](int key_base, floatx4 (&st)[RM][2][2]) {   // one branch a tile, not one a score: the tiles in the middle of a walk skip all of it
#pragma unroll
    for (int rm = 0; rm < RM; ++rm)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int key = key_base + 32 * (j >> 3) + 8 * lq + (j & 7);
        const bool visible = key <= row_pos[rm] && (window <= 0 || key > row_pos[rm] - window);
        if (!visible) st[rm][j >> 3][(j >> 2) & 1][j & 3] = -INFINITY;
      }
  };
  auto softmax_item = [&](int rm, int item, floatx4 (&st)[RM][2][2], uintx4 (&pw)[RM][2]) {
    auto s = [&](int j) -> float { return st[rm][j >> 3][(j >> 2) & 1][j & 3]; };
    if (item == 0) {
      // the largest of the lane's 16 scores as a tree (three-operand maxima) ...
      item_mx[rm] = fmaxf(fmaxf(fmaxf(fmaxf(s(0), s(1)), s(2)), fmaxf(fmaxf(s(3), s(4)), s(5))), fmaxf(s(6), s(7)));
    } else if (item == 1) {
      const float other = fmaxf(fmaxf(fmaxf(fmaxf(s(8), s(9)), s(10)), fmaxf(fmaxf(s(11), s(12)), s(13))), fmaxf(s(14), s(15)));
      item_mx[rm] = fmaxf(item_mx[rm], other);
    } else if (item == 2) {
      item_mx[rm] = max_xor32(max_xor16(item_mx[rm]));       // ... then across the four lanes of the row
    } else if (item == 3) {
      // The reference point of the exponents moves only when the row's maximum has outgrown it by more
      // than RESCALE_MARGIN (base-2 units): until then the probabilities of this tile are at most
      // 2^RESCALE_MARGIN instead of at most 1, which float32 sums and bfloat16 operands hold as well,
      // and the 32 products that rescale the output, and the wave's vote on them, are left out.  The
      // quotient at the end does not depend on the reference point.
      const float m_new = fmaxf(m_run[rm], item_mx[rm] * scale_log2);   // the scale is positive
      moved[rm] = m_new > m_run[rm] + RESCALE_MARGIN;                   // (from -infinity: any finite maximum moves it)
      const float m_next = moved[rm] ? m_new : m_run[rm];
      item_m_use[rm] = m_next > -INFINITY ? m_next : 0.f;               // a row with nothing visible yet
      corr[rm] = moved[rm] ? __builtin_amdgcn_exp2f(m_run[rm] - item_m_use[rm]) : 1.f;
      m_run[rm] = m_next;
    } else if (item < 20) {
      const int j = item - 4;
      st[rm][j >> 3][(j >> 2) & 1][j & 3] = __builtin_amdgcn_exp2f(fmaf(s(j), scale_log2, -item_m_use[rm]));
    } else {
      const int blk = (item - 20) >> 1, half = (item - 20) & 1, j = 8 * blk + 4 * half;
      const unsigned int lo = pack_bf16(s(j), s(j + 1)), hi = pack_bf16(s(j + 2), s(j + 3));
      if (half == 0) { pw[rm][blk].x = lo; pw[rm][blk].y = hi; } else { pw[rm][blk].z = lo; pw[rm][blk].w = hi; }
    }
  };
  auto softmax = [&](int key_base, floatx4 (&st)[RM][2][2], uintx4 (&pw)[RM][2]) {
    if (is_edge(key_base)) mask_edges(key_base, st);
#pragma unroll
    for (int rm = 0; rm < RM; ++rm)
#pragma unroll
      for (int item = 0; item < SOFTMAX_ITEMS; ++item) softmax_item(rm, item, st, pw);
  };
  // what was summed so far moves to the new reference points of the exponents
  auto any_moved = [&]() { bool any = false; for (int rm = 0; rm < RM; ++rm) any = any || moved[rm]; return __any(any); };
  auto rescale = [&]() {
#pragma unroll
    for (int rm = 0; rm < RM; ++rm) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[rm][t][i] *= corr[rm];
#pragma unroll
      for (int i = 0; i < 4; ++i) l_sum[rm][i] *= corr[rm];
      moved[rm] = false;
      corr[rm] = 1.f;
    }
  };
  // The tile holds slots at or beyond the context (the 8-key chunk of the last key has them
  // behind it; later chunks are copies of that chunk) or below the first visible key.  Their
  // probabilities are zero, but a slot that no live key owns may hold anything (a NaN that
  // an earlier request left there), and 0 * NaN is NaN: every wave sets them to zero in the
  // part of the tile that it loaded itself, before the barrier hands the tile to the others.
  // At most twice per block (its first and its last tile); one 4-byte word (two keys) at a
  // time, so that the rare path needs no registers of the common one.
  auto has_unowned = [&](int key_base) { return key_base + BN > ctx || key_base < k_first; };
  auto zero_unowned = [&](int key_base, uintx4* Vt) {
    const int above = ctx - key_base, below = k_first - key_base;   // keys of the tile inside [below, above) count
    unsigned int* words = (unsigned int*)Vt;
    const int ln = lane_again();
    for (int i = 0; i < VI; ++i) {
      const int u = (wave * VI + i) * 64 + ln;
      const int first_key = (u / D) * 8;
#pragma unroll 1
      for (int j = 0; j < 4; ++j) {
        const int k0 = first_key + 2 * j;
        const unsigned int keep = ((k0 >= below && k0 < above) ? 0x0000ffffu : 0u) |
                                  ((k0 + 1 >= below && k0 + 1 < above) ? 0xffff0000u : 0u);
        if (keep != 0xffffffffu) words[u * 4 + j] &= keep;
      }
    }
  };
  // the rows' sums of probabilities as one more output tile whose "values" are all one: the matrix
  // pipe has room, the vector pipe (16 additions and two exchanges a tile) has not; and the sum is
  // then of the probabilities as the second product sees them, rounded to bfloat16
  auto row_sums = [&](uintx4 (&pw)[RM][2]) {
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int rm = 0; rm < RM; ++rm)
        l_sum[rm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, __builtin_bit_cast(bf16x8, pw[rm][blk]), l_sum[rm], 0, 0, 0);
  };
  // The two products of a tile.  S^T: the fragment of keys (blk, h, c) holds 16 keys (rows 32 blk + 4 h +
  // krow of the tile, the interleaved order) x 32 dims (step c) and serves the wave's RM sets of rows;
  // O^T += V^T P^T: the fragment of values (t, blk) holds 16 dims (16 t + lr) x 32 keys (chunk 4 blk + lq).
  // Every fragment is requested AHEAD fragments before the MFMAs that use it,
  // in an order in which the MFMAs on one accumulator stand apart, and with the waits written out (the
  // compiler, left to itself, requests four fragments and waits for all that is under way).  A lane's
  // address is a part that the lane keeps (for the keys one for each step c: the swizzle mixes c in) plus
  // a multiple of 256 bytes that is a constant of the instruction.
  constexpr int AHEAD = 3, RING = AHEAD + 1;       // (five ahead in the blocks of 128 rows: no faster)
  unsigned int key_at[KC], value_at;
#pragma unroll
  for (int c = 0; c < KC; ++c) key_at[c] = (unsigned int)((krow * CH + ((c * 4 + lq) ^ key_swizzle(krow, CH))) * 16);
  value_at = (unsigned int)((lq * D + lr) * 16);
  auto lds_address = [](const uintx4* p) { return (unsigned int)(size_t)(const __attribute__((address_space(3))) char*)p; };
  auto wait_ring = [&](uintx4& v, int pending) {
    if (pending >= 5) lds_arrived<5>(v); else if (pending == 4) lds_arrived<4>(v); else if (pending == 3) lds_arrived<3>(v);
    else if (pending == 2) lds_arrived<2>(v); else if (pending == 1) lds_arrived<1>(v); else lds_arrived<0>(v);
  };
  static_assert(AHEAD <= 5, "wait_ring");
  auto scores_ahead = [&](const uintx4* Kt, floatx4 (&st)[RM][2][2]) {
    constexpr int FRAGMENTS = 4 * KC;                 // step c outermost
    const unsigned int base = lds_address(Kt);
    // rows 32 blk + 4 h + krow: 64 D and 8 D bytes further
    auto fragment = [&](int f) -> uintx4 { return lds_read16_step(base + key_at[f >> 2], (((f >> 1) & 1) * 64 * D + (f & 1) * 8 * D) / 256); };
    uintx4 ring[RING];
#pragma unroll
    for (int f = 0; f < AHEAD; ++f) ring[f] = fragment(f);
#pragma unroll
    for (int f = 0; f < FRAGMENTS; ++f) {
      if (f + AHEAD < FRAGMENTS) ring[(f + AHEAD) % RING] = fragment(f + AHEAD);
      wait_ring(ring[f % RING], FRAGMENTS - 1 - f < AHEAD ? FRAGMENTS - 1 - f : AHEAD);
      const bf16x8 ka = __builtin_bit_cast(bf16x8, ring[f % RING]);
      const int c = f >> 2, blk = (f >> 1) & 1, h = f & 1;
#pragma unroll
      for (int rm = 0; rm < RM; ++rm)
        st[rm][blk][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            ka, qb[rm][c], c == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : st[rm][blk][h], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto weighted_ahead = [&](const uintx4* Vt, uintx4 (&pw)[RM][2]) {
    constexpr int FRAGMENTS = 2 * DT;                 // block outermost
    const unsigned int base = lds_address(Vt) + value_at;
    // chunk 4 blk + lq of the keys, dims 16 t + lr: 64 D and 256 bytes further
    auto fragment = [&](int f) -> uintx4 { return lds_read16_step(base, ((f / DT) * 64 * D + (f % DT) * 256) / 256); };
    uintx4 ring[RING];
#pragma unroll
    for (int f = 0; f < AHEAD; ++f) ring[f] = fragment(f);
#pragma unroll
    for (int f = 0; f < FRAGMENTS; ++f) {
      if (f + AHEAD < FRAGMENTS) ring[(f + AHEAD) % RING] = fragment(f + AHEAD);
      wait_ring(ring[f % RING], FRAGMENTS - 1 - f < AHEAD ? FRAGMENTS - 1 - f : AHEAD);
      const bf16x8 va = __builtin_bit_cast(bf16x8, ring[f % RING]);
      const int t = f % DT, blk = f / DT;
#pragma unroll
      for (int rm = 0; rm < RM; ++rm)
        o[rm][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, __builtin_bit_cast(bf16x8, pw[rm][blk]), o[rm][t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    row_sums(pw);
  };

  // every group makes the same number of rounds (the barriers are the block's); a group without a
  // tile in a round only waits
  const int rounds = (tile_last - tile_first + KG) / KG;
  if constexpr (STAGES == 1) {
    // One buffer for keys and one for values, two barriers a tile: once every wave has its scores,
    // the tile's values and the next tile's keys are requested and fly during the softmax; they are
    // waited for before the second product.  Four waves a SIMD, of several blocks, fill the waits.
    uintx4* Kt = group_lds;
    uintx4* Vt = Kt + BN * CH;
    int tile = tile_first + kg;
    int page = page_of(min(tile, tile_last));
    if (tile <= tile_last) load_keys(tile, page, Kt);
    int page_next = tile + KG <= tile_last ? page_of(tile + KG) : 0;
    FE_WAIT_VMEM(0);
    __syncthreads();               // the first tile's keys are in LDS
    for (int round = 0; round < rounds; ++round, tile += KG) {
      const bool active = tile <= tile_last;
      const bool more = tile + KG <= tile_last;
      const int key_base = tile * BN;
      const bool mine = active && key_base <= wave_lo + 16 * RM - 1;     // some key of the tile is visible to this wave's rows
      floatx4 st[RM][2][2];
      if (mine) scores_ahead(Kt, st);
      // Every wave has its scores, and multiplied the tile before: both buffers are free.
      __syncthreads();
      if (active) load_values(tile, page, Vt);
      if (more) {
        load_keys(tile + KG, page_next, Kt);
        page = page_next;
        if (tile + 2 * KG <= tile_last) page_next = page_of(tile + 2 * KG);
      }
      uintx4 pw[RM][2];
      if (mine) {
        softmax(key_base, st, pw);
        if (any_moved()) rescale();
      }
      FE_WAIT_VMEM(0);
      if (__builtin_expect(active && has_unowned(key_base), 0)) zero_unowned(key_base, Vt);
      __syncthreads();             // the values (and the next keys) are in LDS
      if (mine) weighted_ahead(Vt, pw);
    }
  } else {
    // Two buffers each for keys and values, one barrier a tile: behind it (every wave is done with
    // the tile before, whose buffers the loads overwrite) the next tile's keys and values are
    // requested, and have this whole tile's time to arrive.  With two waves a SIMD there is
    // little else to fill a wait with: the fragments are read from LDS some MFMAs ahead of their use.
    // (Measured and dropped: the next tile's scores issued between the pieces of this tile's softmax,
    // so that a wave keeps both pipes busy by itself.  The two tiles' registers do not fit beside
    // the accumulators of 128 rows: spilled, or moved to and from the accumulation registers with
    // one wave a SIMD, the walk took twice as long.)
    constexpr int TILE_UNITS = BN * CH + 8 * D;
    int tile = tile_first + kg;
    int page = page_of(min(tile, tile_last));
    if (tile <= tile_last) {
      load_keys(tile, page, group_lds);
      load_values(tile, page, group_lds + BN * CH);
    }
    int page_next = tile + KG <= tile_last ? page_of(tile + KG) : 0;
    for (int round = 0; round < rounds; ++round, tile += KG) {
      const bool active = tile <= tile_last;
      const bool more = tile + KG <= tile_last;
      const int key_base = tile * BN;
      const bool mine = active && key_base <= wave_lo + 16 * RM - 1;
      uintx4* Kt = group_lds + (round & 1) * TILE_UNITS;
      uintx4* Vt = Kt + BN * CH;
      FE_WAIT_VMEM(0);
      if (__builtin_expect(active && has_unowned(key_base), 0)) zero_unowned(key_base, Vt);
      __syncthreads();             // this tile's keys and values are in LDS; the other buffers are free
      if (more) {
        uintx4* Kn = group_lds + ((round + 1) & 1) * TILE_UNITS;
        load_keys(tile + KG, page_next, Kn);
        load_values(tile + KG, page_next, Kn + BN * CH);
        if (tile + 2 * KG <= tile_last) page_next = page_of(tile + 2 * KG);
      }
      if (mine) {
        floatx4 st[RM][2][2];
        uintx4 pw[RM][2];
        scores_ahead(Kt, st);
        softmax(key_base, st, pw);
        if (any_moved()) rescale();
        weighted_ahead(Vt, pw);
      }
    }
  }

  float l_run[RM];
#pragma unroll
  for (int rm = 0; rm < RM; ++rm) l_run[rm] = l_sum[rm][0];
  if constexpr (KG == 2) {
    // the second group hands its running maximum, sum and output to the first through LDS (the
    // tiles' buffers are free now), value by value with the lanes side by side, one set of rows at a time
    float* hand = (float*)lds;
    const int slot = wave * 64 + lane;
#pragma unroll
    for (int rm = 0; rm < RM; ++rm) {
      __syncthreads();
      if (kg == 1) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) hand[(t * 4 + i) * 256 + slot] = o[rm][t][i];
        hand[(DT * 4) * 256 + slot] = m_run[rm];
        hand[(DT * 4 + 1) * 256 + slot] = l_run[rm];
      }
      __syncthreads();
      if (kg == 0) {
        const float m_other = hand[(DT * 4) * 256 + slot], l_other = hand[(DT * 4 + 1) * 256 + slot];
        const float m_all = fmaxf(m_run[rm], m_other);
        const float f_mine = m_run[rm] > -INFINITY ? __builtin_amdgcn_exp2f(m_run[rm] - m_all) : 0.f;
        const float f_other = m_other > -INFINITY ? __builtin_amdgcn_exp2f(m_other - m_all) : 0.f;
        l_run[rm] = l_run[rm] * f_mine + l_other * f_other;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[rm][t][i] = o[rm][t][i] * f_mine + hand[(t * 4 + i) * 256 + slot] * f_other;
      }
    }
    if (kg == 1) return;
  }

  // lane (lr = query row, lq) holds O^T[16t + 4lq + i][row]: four consecutive dims per store
#pragma unroll
  for (int rm = 0; rm < RM; ++rm) {
    if (row[rm] >= q_len) continue;
    const float inv = l_run[rm] > 0.f ? 1.f / l_run[rm] : 0.f;
    bf16_t* orow = out + (size_t)(q0 + row[rm]) * out_stride + (size_t)head * D;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      uint2 w;
      w.x = pack_bf16(o[rm][t][0] * inv, o[rm][t][1] * inv);
      w.y = pack_bf16(o[rm][t][2] * inv, o[rm][t][3] * inv);
      *(uint2*)(orow + t * 16 + lq * 4) = w;
    }
  }
}

// Pages: keys [blocks][kv_heads][block_size][D], values transposed [blocks][kv_heads][D][block_size];
// block_size a power of two >= 16; head_dim 64 or 128.  Sequences with fewer than two query tokens
// are skipped.  key_groups: 1 or 2 groups of four waves a block (see the top of the file); row_sets: 1 or 2
// sets of 16 query rows a wave (blocks of 64 or 128 rows); 0 lets the launch choose either, from total_q:
// the query tokens of all sequences together (the rows of q; the grid is laid out for num_seqs sequences
// of max_q_len tokens, of which a step with one long portion fills a fraction).
extern "C" int fe_paged_attention_prefill(const void* q, long long q_stride, const void* key_pages,
                                                 const void* value_pages, void* out, long long out_stride,
                                                 const int* cu_q, const int* ctx_len, const int* block_table,
                                                 int table_stride, int num_seqs, int max_q_len, int kv_heads,
                                                 int groups, int head_dim, int block_size, int num_blocks,
                                                 int window, float scale, int key_groups, int row_sets, int total_q,
                                                 hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len < 2) return FE_OK;
  if (head_dim != 64 && head_dim != 128) return FE_BAD_ARGUMENT;
  if (groups < 1 || kv_heads < 1 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < 16 || (block_size & (block_size - 1)) || num_blocks < 1 || table_stride < 1 || q_stride % 8 || out_stride % 4) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)key_pages) | ((uintptr_t)value_pages) | ((uintptr_t)q)) & 15) return FE_BAD_ARGUMENT;
  if (key_groups < 0 || key_groups > 2 || row_sets < 0 || row_sets > 2 || total_q < 1) return FE_BAD_ARGUMENT;
  const float scale_log2 = scale * 1.4426950408889634f;
  int block_shift = 0;
  while ((1 << block_shift) < block_size) ++block_shift;
  const int heads = kv_heads * groups;
  const int heads_per_xcd = heads >= XCDS ? (heads + XCDS - 1) / XCDS : 0;
  // Tiles of `rows` query rows: a sequence of n tokens has at most n / rows + 1, and the grid does not
  // depend on how the tokens are spread over the sequences (a captured launch serves every spread);
  // `filled`: the tiles that the tokens can fill (a captured launch is laid out for more sequences
  // than a step brings, and a block without a tile ends at once).
  auto slots_of = [&](int rows) { return std::min<long long>((long long)num_seqs * ((max_q_len + rows - 1) / rows), total_q / rows + num_seqs); };
  auto filled_of = [&](int rows) { return std::min<long long>(slots_of(rows), (total_q + rows - 1) / rows); };
  // Two sets of rows a wave (a fragment of keys or values read from LDS then feeds two MFMAs, and the
  // LDS reads are what bounds the tile with one) where blocks of 128 rows still fill the chip some times
  // over.  Measured, 32 heads of 128, microseconds with blocks of 64 rows and one key group / two key
  // groups / 128 rows and one key group: one prompt of 1,024 tokens 24 / 22 / 29, of 2,048 50 / 55 / 54,
  // of 3,072 103 / 103 / 85, of 8,192 585 / 626 / 510; eight of 1,024 98 / 127 / 93; two of 1,024 29 / 34 / 32.
  if (row_sets == 0) row_sets = (max_q_len >= ROWS2_MIN_LEN && (long long)heads * filled_of(128) >= ROWS2_MIN_BLOCKS) ? 2 : 1;
  const int rows = 64 * row_sets;
  const long long slots = slots_of(rows);
  const long long blocks = (heads_per_xcd ? (long long)heads_per_xcd * XCDS : heads) * slots;
  if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  const unsigned grid = (unsigned)blocks;
  // Two key groups a block where the launch would leave the chip underfilled (its blocks are resident
  // all at once or nearly: then the longest walk sets the time, and halving it pays: 256 tokens behind
  // 4,096 cached ones 72 -> 53 us, one prompt of 512 tokens 13.5 -> 12.5 us) and the portions span at
  // least two tiles.
  if (key_groups == 0) key_groups = (row_sets == 1 && (long long)heads * filled_of(64) <= KEY_GROUPS_MAX_BLOCKS && max_q_len >= 128) ? 2 : 1;
#define FE_GO(DD, GG, RR)                                                                                            \
  paged_prefill_kernel<DD, GG, RR><<<grid, 256 * GG, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)key_pages, \
      (const bf16_t*)value_pages, (bf16_t*)out, out_stride, cu_q, ctx_len, block_table, table_stride,            \
      kv_heads, groups, block_shift, num_blocks, window, scale_log2, num_seqs, heads_per_xcd)
#define FE_GO_D(DD)                                          \
  if (key_groups == 1 && row_sets == 1) FE_GO(DD, 1, 1);      \
  else if (row_sets == 1) FE_GO(DD, 2, 1);                    \
  else if (key_groups == 1) FE_GO(DD, 1, 2);                  \
  else FE_GO(DD, 2, 2)
  if (head_dim == 64) { FE_GO_D(64); } else { FE_GO_D(128); }
#undef FE_GO_D
#undef FE_GO
  return fe_check_launch();
}
