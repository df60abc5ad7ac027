// Paged grouped-query attention for portions of prompts (two or more query
// tokens of one sequence in a step), bfloat16 cache, on the matrix cores.
//
// Block = 64 or 128 query tokens of one query head of one sequence; its four
// waves take 16 or 32 query rows each.  Keys and values are walked in tiles of
// 64, loaded once per block into LDS and shared by the four waves; keys as
// stored ([key][D]), values as stored too: their pages are transposed
// ([D][slot]), which is the operand layout of the second product.
//   S^T = K Q^T    MFMA 16x16x32, A = 16 keys from LDS, B = 16 query rows held
//                  in registers for the whole kernel.  The 32 keys of a block
//                  feed two MFMA tiles whose rows interleave in groups of four,
//                  so lane group lq gets the scores of keys 8lq .. 8lq+7 of
//                  its query row: already the B operand of the next product;
//   softmax        float32, online over tiles, base-2 exponent with the scale
//                  folded in; a row's keys sit in four lanes (two shuffles);
//                  the causal (and window) mask only on tiles that cross it;
//   O^T += V^T P^T MFMA 16x16x32, A = 16 dims x 32 keys from LDS, B = P^T
//                  (bfloat16, straight from the score registers).
// Query token i of the step sits at position ctx_before + i and sees keys
// max(0, p - window + 1) .. p.  Sequences with fewer than two query tokens are
// skipped (the decode kernel serves them).  Sums and statistics are float32; P
// is rounded to bfloat16 for the second product, as the reference rounds its
// probabilities (src/forge_engine/qwen3.py:200).
//
// The grid is one-dimensional and aware of the eight XCDs: consecutive block
// ids land on different XCDs, so block id l works on item (l % 8) * n/8 + l / 8
// of a list ordered by (sequence, head, pair of row tiles): one XCD, with its
// own L2, gets neighbouring heads, which share keys and values.  A block takes
// row tile i from the end and then row tile i from the start, so that all
// blocks of a sequence walk about the same number of key tiles.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define BN 64        // keys per tile
#define KPAD 0       // key rows are not padded: their 16-byte chunks are swizzled instead (see key_swizzle)
#define VPAD 8       // bf16 padding of a value row (one dim, 64 keys) in LDS
#define XCDS 8

// Chunk c (16 bytes) of key row r lives at chunk position c ^ swizzle(r) of the row.  The 16 lanes
// that read one chunk index together hold rows 8a + b (+ 4h), a < 4, b < 4, which a padded row
// stride cannot spread over all banks (rows 8 apart always collide); 4a + b is distinct for them.
__device__ __forceinline__ int key_swizzle(int row, int chunks) { return (((row >> 3) & 3) * 4 + (row & 3)) & (chunks - 1); }

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
__device__ __forceinline__ unsigned int pack_bf16(float lo, float hi) {
  const bf16x2 v = {(__bf16)lo, (__bf16)hi};   // the hardware's round-to-nearest-even conversion
  return __builtin_bit_cast(unsigned int, v);
}

template <int D, int RT>
__global__ __launch_bounds__(256, RT == 1 ? 2 : 1) void paged_prefill_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, long long out_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int table_stride, int kv_heads, int groups, int block_shift, int num_blocks, int window,
    float scale_log2, int pairs, int items_per_xcd, int total_items) {
  const int block_size = 1 << block_shift, block_mask = block_size - 1;
  constexpr int BM = 64 * RT;     // query rows per tile of rows
  constexpr int KC = D / 32;      // MFMA k-steps over the head dim (scores)
  constexpr int DT = D / 16;      // 16-dim tiles of the output
  constexpr int CH = D / 8;       // 16-byte pieces per key row
  // two LDS stages of (keys [BN][D + KPAD], values [D][BN + VPAD]): one is multiplied while the
  // next tile is written into the other, so a tile costs one barrier
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  typedef bf16_t KeyTile[BN][D + KPAD];
  typedef bf16_t ValueTile[D][BN + VPAD];
  KeyTile* Ks = (KeyTile*)lds_raw;
  ValueTile* Vt = (ValueTile*)(lds_raw + 2 * sizeof(KeyTile));

  const int heads = kv_heads * groups;
  const int item = (blockIdx.x % XCDS) * items_per_xcd + blockIdx.x / XCDS;
  if (item >= total_items) return;   // the list is padded to a multiple of the XCD count
  const int seq = item / (heads * pairs);
  const int rest = item - seq * heads * pairs;
  const int head = rest / pairs;
  const int pair = rest - head * pairs;
  const int hk = head / groups;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  if (q_len < 2) return;
  // A block takes two row tiles of its (sequence, head): number `pair` from the end, the longer
  // walk over the keys, then number `pair` from the start: every block of a sequence walks about
  // the same number of key tiles, whatever the causal mask cuts away.
  const int q_tiles = (q_len + BM - 1) / BM;
  if (2 * pair >= q_tiles) return;
  const int ctx = ctx_len[seq];
  const int before = ctx - q_len;
  const int* table = block_table + (size_t)seq * table_stride;
  const int table_last = table_stride - 1;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lq = lane >> 4;
  const int krow = 8 * (lr >> 2) + (lr & 3);   // MFMA row r of key tile h is key 8*(r/4) + 4h + r%4 of its 32-key block

  // loaders: keys piece p -> (key p / CH, 16 bytes p % CH); values piece p -> (dim p / 8, the 8
  // keys (p % 8) * 8 .. of the tile), read from the transposed page of those keys.  A lane reads
  // the page ids it needs for a tile two tiles before the tile's data loads are issued; the data
  // loads are unconditional (a key beyond the context reads page 0 and is masked later).
  constexpr int LOADS = BN * CH / 256;
  struct TileIds { int k[LOADS]; int v; };   // this lane's pages of a tile: one per key piece, one for its value pieces
  auto page_at = [&](int key) -> int {
    const int id = table[min(key >> block_shift, table_last)];
    return (key < ctx && id >= 0 && id < num_blocks) ? id : 0;
  };
  auto load_pages = [&](int tile, TileIds& ids) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) ids.k[i] = page_at(tile * BN + (tid + i * 256) / CH);
    ids.v = page_at(tile * BN + (tid % 8) * 8);
  };
  auto load_tile = [&](int tile, const TileIds& ids, uintx4* kreg, uintx4* vreg) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int p = tid + i * 256;
      {
        const int key = tile * BN + p / CH;
        kreg[i] = *(const uintx4*)(key_pages + ((((size_t)ids.k[i] * kv_heads + hk) << block_shift) + (key & block_mask)) * D + (p % CH) * 8);
      }
      {
        const int key = tile * BN + (p % 8) * 8;     // p % 8 == tid % 8: 256 is a multiple of 8
        const uintx4 v = *(const uintx4*)(value_pages + ((((size_t)ids.v * kv_heads + hk) * D + p / 8) << block_shift) + (key & block_mask));
        vreg[i] = (tile * BN + BN <= ctx || key < ctx) ? v : uintx4{0u, 0u, 0u, 0u};
      }
    }
  };
  auto store_tile = [&](int stage, const uintx4* kreg, const uintx4* vreg) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int p = tid + i * 256;
      *(uintx4*)&Ks[stage][p / CH][((p % CH) ^ key_swizzle(p / CH, CH)) * 8] = kreg[i];
      *(uintx4*)&Vt[stage][p / 8][(p % 8) * 8] = vreg[i];
    }
  };

  for (int turn = 0; turn < 2; ++turn) {
    const int q_tile = turn == 0 ? q_tiles - 1 - pair : pair;
    if (turn == 1 && q_tile == q_tiles - 1 - pair) break;   // the middle tile of an odd count
    const int row0 = q_tile * BM;

    // this wave's query rows as B operands: lane (lr = row, lq) holds q[row][32c + 8lq .. +8]
    bf16x8 qb[RT][KC];
    int row_pos[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int row = row0 + (wave * RT + rt) * 16 + lr;
      row_pos[rt] = before + row;
      const bf16_t* qrow = q + (size_t)(q0 + min(row, q_len - 1)) * q_stride + (size_t)head * D;
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const uintx4 v = *(const uintx4*)(qrow + c * 32 + lq * 8);
        qb[rt][c] = __builtin_bit_cast(bf16x8, row < q_len ? v : uintx4{0u, 0u, 0u, 0u});
      }
    }
    float m_run[RT], l_run[RT];   // running maximum (in units of the base-2 exponent) and sum
    floatx4 o[RT][DT];            // O^T: dims 16t + 4lq + i of query row lr
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      m_run[rt] = -INFINITY;
      l_run[rt] = 0.f;
#pragma unroll
      for (int t = 0; t < DT; ++t) o[rt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    const int last_row = min(q_len, row0 + BM) - 1;
    const int pos_lo = before + row0, pos_hi = before + last_row;
    const int wave_lo = pos_lo + wave * RT * 16;      // position of this wave's first row
    const int k_first = window > 0 ? max(0, pos_lo - window + 1) : 0;
    const int tile_first = k_first / BN, tile_last = pos_hi / BN;   // inclusive

    // One tile, already in LDS stage `stage`: the next tile goes from the other register set
    // (kreg, vreg) into the other stage and the loads of the tile three further on are issued
    // into those registers; then this tile is multiplied.  The caller's barrier follows.
    auto do_tile = [&](int tile, int stage, uintx4* kreg, uintx4* vreg, TileIds& ids) __attribute__((always_inline)) {
      if (tile + 1 <= tile_last) {
        store_tile(stage ^ 1, kreg, vreg);
        if (tile + 3 <= tile_last) {
          load_tile(tile + 3, ids, kreg, vreg);
          if (tile + 5 <= tile_last) load_pages(tile + 5, ids);
        }
      }

      const int key_base = tile * BN;
      if (key_base > wave_lo + RT * 16 - 1) return;   // every key of the tile lies after this wave's rows
      floatx4 st[RT][2][2];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int c = 0; c < KC; ++c) {
            const int row = blk * 32 + krow + 4 * h;
            const bf16x8 ka = *(const bf16x8*)&Ks[stage][row][((c * 4 + lq) ^ key_swizzle(row, CH)) * 8];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              st[rt][blk][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  ka, qb[rt][c], c == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : st[rt][blk][h], 0, 0, 0);
          }
      // lane (lr = query row, lq): st[rt][blk][h][i] = score of key key_base + 32 blk + 8lq + 4h + i
      const bool edge = key_base + BN - 1 > wave_lo || (window > 0 && key_base < pos_hi - window + 1);
      bf16x8 pb[RT][2];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        float s[16];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          float v = st[rt][j >> 3][(j >> 2) & 1][j & 3];
          if (edge) {
            const int key = key_base + 32 * (j >> 3) + 8 * lq + (j & 7);
            const bool visible = key <= row_pos[rt] && (window <= 0 || key > row_pos[rt] - window);
            v = visible ? v : -INFINITY;
          }
          s[j] = v;
          mx = fmaxf(mx, v);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, FE_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, FE_WAVE));
        const float m_new = fmaxf(m_run[rt], mx * scale_log2);   // the scale is positive
        const float m_use = m_new > -INFINITY ? m_new : 0.f;     // a row with nothing visible yet
        const float corr = __builtin_amdgcn_exp2f(m_run[rt] - m_use);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          s[j] = __builtin_amdgcn_exp2f(fmaf(s[j], scale_log2, -m_use));
          sum += s[j];
        }
        sum += __shfl_xor(sum, 16, FE_WAVE);
        sum += __shfl_xor(sum, 32, FE_WAVE);
        l_run[rt] = l_run[rt] * corr + sum;
        m_run[rt] = m_new;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          uintx4 pw;
          pw.x = pack_bf16(s[8 * blk + 0], s[8 * blk + 1]); pw.y = pack_bf16(s[8 * blk + 2], s[8 * blk + 3]);
          pw.z = pack_bf16(s[8 * blk + 4], s[8 * blk + 5]); pw.w = pack_bf16(s[8 * blk + 6], s[8 * blk + 7]);
          pb[rt][blk] = __builtin_bit_cast(bf16x8, pw);
        }
        if (__any(corr != 1.f)) {      // the maximum moved for some row of this wave
#pragma unroll
          for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[rt][t][i] *= corr;
        }
      }
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          const bf16x8 va = *(const bf16x8*)&Vt[stage][t * 16 + lr][blk * 32 + lq * 8];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            o[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[rt][blk], o[rt][t], 0, 0, 0);
        }
    };

    // register sets: set 0 carries the tiles at even distance from the first, set 1 the odd ones
    uintx4 k0[LOADS], v0[LOADS], k1[LOADS], v1[LOADS];
    TileIds ids0, ids1;
    load_pages(tile_first, ids0);
    load_tile(tile_first, ids0, k0, v0);
    if (tile_first + 1 <= tile_last) {
      load_pages(tile_first + 1, ids1);
      load_tile(tile_first + 1, ids1, k1, v1);
    }
    if (tile_first + 2 <= tile_last) load_pages(tile_first + 2, ids0);
    if (tile_first + 3 <= tile_last) load_pages(tile_first + 3, ids1);
    __syncthreads();              // the previous row tile's reads of LDS are done
    store_tile(0, k0, v0);
    if (tile_first + 2 <= tile_last) {
      load_tile(tile_first + 2, ids0, k0, v0);
      if (tile_first + 4 <= tile_last) load_pages(tile_first + 4, ids0);
    }
    __syncthreads();
    for (int tile = tile_first; tile <= tile_last; tile += 2) {
      do_tile(tile, 0, k1, v1, ids1);
      __syncthreads();
      if (tile + 1 > tile_last) break;
      do_tile(tile + 1, 1, k0, v0, ids0);
      __syncthreads();
    }

    // lane (lr = query row, lq) holds O^T[16t + 4lq + i][row]: four consecutive dims per store
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int row = row0 + (wave * RT + rt) * 16 + lr;
      if (row >= q_len) continue;
      const float inv = l_run[rt] > 0.f ? 1.f / l_run[rt] : 0.f;
      bf16_t* orow = out + (size_t)(q0 + row) * out_stride + (size_t)head * D;
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        uint2 w;
        w.x = pack_bf16(o[rt][t][0] * inv, o[rt][t][1] * inv);
        w.y = pack_bf16(o[rt][t][2] * inv, o[rt][t][3] * inv);
        *(uint2*)(orow + t * 16 + lq * 4) = w;
      }
    }
  }
}

// Pages: keys [blocks][kv_heads][block_size][D], values transposed [blocks][kv_heads][D][block_size];
// block_size a power of two >= 16.  rows_per_block: 0 (the default, 64), 64 or 128.
extern "C" int fe_paged_attention_prefill(const void* q, long long q_stride, const void* key_pages,
                                          const void* value_pages, void* out, long long out_stride,
                                          const int* cu_q, const int* ctx_len, const int* block_table,
                                          int table_stride, int num_seqs, int max_q_len, int kv_heads,
                                          int groups, int head_dim, int block_size, int num_blocks,
                                          int window, float scale, int rows_per_block,
                                          hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len < 2) return FE_OK;
  if (head_dim != 64 && head_dim != 128) return FE_BAD_ARGUMENT;
  if (groups < 1 || kv_heads < 1 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < 16 || (block_size & (block_size - 1)) || num_blocks < 1 || table_stride < 1 || q_stride % 8 || out_stride % 4) return FE_BAD_ARGUMENT;
  const float scale_log2 = scale * 1.4426950408889634f;
  if (rows_per_block != 0 && rows_per_block != 64 && rows_per_block != 128) return FE_BAD_ARGUMENT;
  // long portions: 128-row blocks halve the reads of keys and values
  const int rt = rows_per_block ? rows_per_block / 64 : 1;   // 64-row blocks keep two blocks on a unit
  int block_shift = 0;
  while ((1 << block_shift) < block_size) ++block_shift;
  const int q_tiles = (max_q_len + 64 * rt - 1) / (64 * rt);
  const int pairs = (q_tiles + 1) / 2;      // a block takes a late and an early tile of rows
  const long long items = (long long)num_seqs * kv_heads * groups * pairs;
  const long long per_xcd = (items + XCDS - 1) / XCDS;
  if (per_xcd * XCDS > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  const unsigned grid = (unsigned)(per_xcd * XCDS);
#define FE_GO(DD, RR) {                                                                                      \
  static bool ready_##DD##_##RR = false;                                                                       \
  const int lds_bytes = 2 * (BN * (DD + KPAD) + DD * (BN + VPAD)) * (int)sizeof(bf16_t);                       \
  if (!ready_##DD##_##RR) {                                                                                    \
    if (hipFuncSetAttribute((const void*)paged_prefill_kernel<DD, RR>,                                         \
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)              \
      return FE_LAUNCH_FAILED;                                                                                 \
    ready_##DD##_##RR = true;                                                                                  \
  }                                                                                                            \
  paged_prefill_kernel<DD, RR><<<grid, 256, lds_bytes, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)key_pages, \
      (const bf16_t*)value_pages, (bf16_t*)out, out_stride, cu_q, ctx_len, block_table, table_stride,          \
      kv_heads, groups, block_shift, num_blocks, window, scale_log2, pairs, (int)per_xcd, (int)items); }
  if (head_dim == 64) { if (rt == 2) FE_GO(64, 2) else FE_GO(64, 1) }
  else { if (rt == 2) FE_GO(128, 2) else FE_GO(128, 1) }
#undef FE_GO
  return fe_check_launch();
}
