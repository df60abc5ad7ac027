// Paged grouped-query attention for portions of prompts (two or more query
// tokens of one sequence in a step), bfloat16 cache, on the matrix cores.
//
// Block = 64 query tokens of one query head of one sequence (grid: query tile,
// query head, sequence); its four waves take 16 query rows each.  Keys and
// values are walked in tiles of 64 (whole 16-key runs of pages), loaded once
// per block into LDS and shared by the four waves:
//   S = Q K^T   MFMA 16x16x32, A = query rows (registers, loaded once),
//               B = keys from LDS, row-major [key][D + pad];
//   softmax     float32, online over tiles, base-2 exponent with the scale
//               folded in; the causal (and window) mask only where a tile
//               crosses a row's limits;
//   O += P V    MFMA 16x16x32 with keys as the k dim: A = P (bfloat16, through
//               a per-wave LDS tile to change from the score layout to the
//               operand layout), B = values from LDS stored transposed
//               [d][key + pad] so that each lane reads 8 consecutive keys.
// Query token i of the step sits at position ctx_before + i and sees keys
// max(0, p - window + 1) .. p.  Sequences with fewer than two query tokens are
// skipped (the decode kernel serves them).  Sums and statistics are float32;
// P is rounded to bfloat16 for the second product, as the reference rounds its
// probabilities (src/forge_engine/qwen3.py:200).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define BM 64        // query rows per block
#define BN 64        // keys per tile
#define KPAD 8       // bf16 padding of a key row in LDS
#define VPAD 8       // bf16 padding of a transposed value row in LDS
#define PPAD 8

template <int D>
__global__ __launch_bounds__(256) void paged_prefill_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, long long out_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int table_stride, int kv_heads, int groups, int block_size, int num_blocks, int window,
    float scale_log2) {
  constexpr int KC = D / 32;      // MFMA k-steps over the head dim (scores)
  constexpr int DT = D / 16;      // 16-wide tiles of the head dim (output)
  constexpr int CH = D / 8;       // 16-byte chunks per key row
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BN][D + KPAD];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D][BN + VPAD];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4][16][BN + PPAD];

  const int seq = blockIdx.z, head = blockIdx.y, hk = head / groups;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int row0 = blockIdx.x * BM;
  if (q_len < 2 || row0 >= q_len) return;
  const int ctx = ctx_len[seq];
  const int before = ctx - q_len;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lq = lane >> 4;

  // this wave's 16 query rows as the A operand: lane (lr = row, lq) holds q[row][32c + 8lq .. +8]
  const int my_row = row0 + wave * 16 + lr;          // A-operand row of this lane
  bf16x8 qa[KC];
  {
    const bf16_t* qrow = q + (size_t)(q0 + min(my_row, q_len - 1)) * q_stride + (size_t)head * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      uintx4 v = uintx4{0u, 0u, 0u, 0u};
      if (my_row < q_len) v = *(const uintx4*)(qrow + c * 32 + lq * 8);
      qa[c] = __builtin_bit_cast(bf16x8, v);
    }
  }
  // score/output layout: lane (lr, lq) holds rows 4lq + i (i < 4) at column lr
  int row_pos[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) row_pos[i] = before + row0 + wave * 16 + lq * 4 + i;
  float m_run[4], l_run[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m_run[i] = -INFINITY; l_run[i] = 0.f; }
  floatx4 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int last_row = min(q_len, row0 + BM) - 1;
  const int pos_lo = before + row0, pos_hi = before + last_row;
  const int k_first = window > 0 ? max(0, pos_lo - window + 1) : 0;
  const int tile_first = k_first / BN, tile_last = pos_hi / BN;   // inclusive
  const int* table = block_table + (size_t)seq * table_stride;

  // loader mapping.  keys: chunk p -> (key p / CH, 16-byte piece p % CH): rows are read whole.
  // values: chunk p -> (key p % BN, piece p / BN): a wave's 64 lanes hold 64 keys of one piece,
  // so the transposed 2-byte stores of a piece land side by side.
  constexpr int LOADS = BN * CH / 256;
  uintx4 kreg[LOADS], vreg[LOADS];
  auto load_tile = [&](int tile) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int p = tid + i * 256;
      {
        const int key = tile * BN + p / CH;
        uintx4 v = uintx4{0u, 0u, 0u, 0u};
        if (key < ctx) {
          const int block = table[key / block_size];
          if (block >= 0 && block < num_blocks)
            v = *(const uintx4*)(key_pages + (((size_t)block * kv_heads + hk) * block_size + key % block_size) * D + (p % CH) * 8);
        }
        kreg[i] = v;
      }
      {
        const int key = tile * BN + p % BN;
        uintx4 v = uintx4{0u, 0u, 0u, 0u};
        if (key < ctx) {
          const int block = table[key / block_size];
          if (block >= 0 && block < num_blocks)
            v = *(const uintx4*)(value_pages + (((size_t)block * kv_heads + hk) * block_size + key % block_size) * D + (p / BN) * 8);
        }
        vreg[i] = v;
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int p = tid + i * 256;
      *(uintx4*)&Ks[p / CH][(p % CH) * 8] = kreg[i];
      const int key = p % BN, d0 = (p / BN) * 8;
      const unsigned int w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        Vt[d0 + 2 * e][key] = (bf16_t)(w[e] & 0xffffu);
        Vt[d0 + 2 * e + 1][key] = (bf16_t)(w[e] >> 16);
      }
    }
  };

  load_tile(tile_first);
  for (int tile = tile_first; tile <= tile_last; ++tile) {
    __syncthreads();            // the previous tile's LDS reads are done
    store_tile();
    __syncthreads();
    if (tile < tile_last) load_tile(tile + 1);   // flies while this tile multiplies

    // scores of this wave's 16 rows against the tile's 64 keys
    floatx4 s[BN / 16];
#pragma unroll
    for (int st = 0; st < BN / 16; ++st) {
      s[st] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const bf16x8 kb = *(const bf16x8*)&Ks[st * 16 + lr][c * 32 + lq * 8];
        s[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[c], kb, s[st], 0, 0, 0);
      }
    }
    const int key_base = tile * BN;
    // mask only if the tile reaches beyond some row's position or before its window
    const bool edge = key_base + BN - 1 > pos_lo + wave * 16 || (window > 0 && key_base < pos_hi - window + 1);
    float corr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mx = -INFINITY;
#pragma unroll
      for (int st = 0; st < BN / 16; ++st) {
        float v = s[st][i] * scale_log2;
        if (edge) {
          const int key = key_base + st * 16 + lr;
          const bool visible = key <= row_pos[i] && (window <= 0 || key > row_pos[i] - window);
          v = visible ? v : -INFINITY;
        }
        s[st][i] = v;
        mx = fmaxf(mx, v);
      }
#pragma unroll
      for (int offset = 8; offset > 0; offset >>= 1) mx = fmaxf(mx, __shfl_xor(mx, offset, FE_WAVE));
      const float m_new = fmaxf(m_run[i], mx);
      const float m_use = m_new > -INFINITY ? m_new : 0.f;    // a row with nothing visible yet
      corr[i] = __builtin_amdgcn_exp2f(m_run[i] - m_use);
      float sum = 0.f;
#pragma unroll
      for (int st = 0; st < BN / 16; ++st) {
        const float p = __builtin_amdgcn_exp2f(s[st][i] - m_use);
        s[st][i] = p;
        sum += p;
      }
#pragma unroll
      for (int offset = 8; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, FE_WAVE);
      l_run[i] = l_run[i] * corr[i] + sum;
      m_run[i] = m_new;
    }
    // P: score layout -> LDS -> operand layout (rows = lr, 8 consecutive keys per lane)
#pragma unroll
    for (int st = 0; st < BN / 16; ++st)
#pragma unroll
      for (int i = 0; i < 4; ++i) Ps[wave][lq * 4 + i][st * 16 + lr] = float_to_bf16(s[st][i]);
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= corr[i];
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
#pragma unroll
    for (int kk = 0; kk < BN / 32; ++kk) {
      const bf16x8 pa = *(const bf16x8*)&Ps[wave][lr][kk * 32 + lq * 8];
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        const bf16x8 vb = *(const bf16x8*)&Vt[t * 16 + lr][kk * 32 + lq * 8];
        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vb, o[t], 0, 0, 0);
      }
    }
  }

  // lane holds O[row 4lq + i][d = 16t + lr]
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = row0 + wave * 16 + lq * 4 + i;
    if (row >= q_len) continue;
    const float inv = l_run[i] > 0.f ? 1.f / l_run[i] : 0.f;
    bf16_t* orow = out + (size_t)(q0 + row) * out_stride + (size_t)head * D;
#pragma unroll
    for (int t = 0; t < DT; ++t) orow[t * 16 + lr] = float_to_bf16(o[t][i] * inv);
  }
}

extern "C" int fe_paged_attention_prefill(const void* q, long long q_stride, const void* key_pages,
                                          const void* value_pages, void* out, long long out_stride,
                                          const int* cu_q, const int* ctx_len, const int* block_table,
                                          int table_stride, int num_seqs, int max_q_len, int kv_heads,
                                          int groups, int head_dim, int block_size, int num_blocks,
                                          int window, float scale, hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len < 2) return FE_OK;
  if (head_dim != 64 && head_dim != 128) return FE_BAD_ARGUMENT;
  if (groups < 1 || kv_heads < 1 || (long long)kv_heads * groups > 65535 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < 16 || block_size % 16 || num_blocks < 1 || table_stride < 1 || q_stride % 8) return FE_BAD_ARGUMENT;
  dim3 grid((max_q_len + BM - 1) / BM, kv_heads * groups, num_seqs);
  const float scale_log2 = scale * 1.4426950408889634f;
#define FE_GO(DD)                                                                                           \
  paged_prefill_kernel<DD><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)key_pages,    \
      (const bf16_t*)value_pages, (bf16_t*)out, out_stride, cu_q, ctx_len, block_table, table_stride,         \
      kv_heads, groups, block_size, num_blocks, window, scale_log2)
  if (head_dim == 64) FE_GO(64);
  else FE_GO(128);
#undef FE_GO
  return fe_check_launch();
}
