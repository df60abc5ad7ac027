// Paged grouped-query attention for single decoded tokens, bfloat16 cache.
//
// For every sequence of the batch that brings exactly one query token (others
// are skipped: they belong to the prefill kernel), the G query heads that share
// a kv head read that head's keys and values once.  The kernel is bound by the
// cache's bytes, so the work is laid out for streaming:
//   * grid (key split, kv head, sequence); with few sequences the keys of one
//     (sequence, head) are split over several blocks so that the chip is full,
//     and a second small kernel merges the splits;
//   * inside a block, the four waves take 16-key tiles in turn; a tile of keys
//     is 16 rows of D contiguous bfloat16 in its page;
//   * scores: MFMA 16x16x32 (A = the G query rows padded to 16, B = keys);
//     softmax statistics in float32, online over tiles;
//   * values: plain FMAs (the reduction runs over keys, which are not
//     contiguous per lane in the page layout, and there is bandwidth to spare).
// Exactness: scores, max, sum and the weighted value sum are float32; one
// rounding at the final store.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define TILE 16          // keys per tile
#define WAVES 4

__device__ __forceinline__ void unpack8(const uintx4 v, float* f) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

// D: head size (64, 128, 256); GT: upper bound of the group size handled (1, 2, 4, 8).
template <int D, int GT>
__global__ __launch_bounds__(256) void paged_decode_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, long long out_stride,
    float* __restrict__ part_o, float* __restrict__ part_ml, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const int* __restrict__ block_table, int table_stride,
    int kv_heads, int groups, int block_size, int num_blocks, int window, float scale) {
  constexpr int KC = D / 32;        // MFMA k-steps over the head dim
  constexpr int LPK = D / 8;        // lanes that cover one value row with 16-byte loads
  constexpr int KPI = 64 / LPK;     // value rows per load instruction
  __shared__ float Ps[WAVES][16][TILE + 1];
  __shared__ float Cs[WAVES][16];
  __shared__ float Ow[WAVES][GT][D];
  __shared__ float Ms[WAVES][GT], Ls[WAVES][GT];

  const int split = blockIdx.x, splits = gridDim.x;
  const int hk = blockIdx.y, seq = blockIdx.z;
  const int q0 = cu_q[seq];
  if (cu_q[seq + 1] - q0 != 1) return;
  const int ctx = ctx_len[seq];
  const int k_begin = window > 0 ? max(0, ctx - window) : 0;
  const int tile_first = k_begin / TILE;
  const int tile_last = (ctx + TILE - 1) / TILE;          // exclusive
  const int per_split = (tile_last - tile_first + splits - 1) / splits;
  const int my_first = tile_first + split * per_split;
  const int my_last = min(tile_last, my_first + per_split);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lq = lane >> 4;
  const int kq = lane / LPK, dl = lane % LPK;

  // query rows as the A operand: lane (lr = row, lq) holds q[row][32*c + 8*lq .. +8]
  bf16x8 qa[KC];
  {
    const bf16_t* qrow = q + (size_t)q0 * q_stride + (size_t)(hk * groups + (lr < groups ? lr : 0)) * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      uintx4 v = uintx4{0u, 0u, 0u, 0u};
      if (lr < groups) v = *(const uintx4*)(qrow + c * 32 + lq * 8);
      qa[c] = __builtin_bit_cast(bf16x8, v);
    }
  }

  float m_run[4], l_run[4];   // rows 4*lq + i, replicated over the 16 lanes of the group
#pragma unroll
  for (int i = 0; i < 4; ++i) { m_run[i] = -INFINITY; l_run[i] = 0.f; }
  float acc[GT][8];           // this lane's keys (kq) x its 8 dims (dl), all rows
#pragma unroll
  for (int g = 0; g < GT; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;

  const int* table = block_table + (size_t)seq * table_stride;
  for (int t = my_first + wave; t < my_last; t += WAVES) {
    const int key0 = t * TILE;
    const int block = table[key0 / block_size];
    const bool page_ok = block >= 0 && block < num_blocks;
    const size_t tile_off = (((size_t)(page_ok ? block : 0) * kv_heads + hk) * block_size + (key0 % block_size)) * D;
    // issue this tile's loads: keys (MFMA B operand) and values (16 bytes per lane)
    uintx4 kb[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      kb[c] = uintx4{0u, 0u, 0u, 0u};
      if (page_ok) kb[c] = *(const uintx4*)(key_pages + tile_off + (size_t)lr * D + c * 32 + lq * 8);
    }
    uintx4 vb[TILE / KPI];
#pragma unroll
    for (int j = 0; j < TILE / KPI; ++j) {
      vb[j] = uintx4{0u, 0u, 0u, 0u};
      if (page_ok) vb[j] = *(const uintx4*)(value_pages + tile_off + (size_t)(j * KPI + kq) * D + dl * 8);
    }
    floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KC; ++c)
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[c], __builtin_bit_cast(bf16x8, kb[c]), s, 0, 0, 0);
    // lane holds s[i] = score(row 4*lq + i, key key0 + lr)
    const int key = key0 + lr;
    const bool visible = page_ok && key >= k_begin && key < ctx;
    float p[4], corr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = visible ? s[i] * scale : -INFINITY;
      float mx = v;
#pragma unroll
      for (int offset = 8; offset > 0; offset >>= 1) mx = fmaxf(mx, __shfl_xor(mx, offset, FE_WAVE));
      const float m_new = fmaxf(m_run[i], mx);
      if (m_new > -INFINITY) {
        corr[i] = __expf(m_run[i] - m_new);
        p[i] = __expf(v - m_new);
      } else {
        corr[i] = 1.f;
        p[i] = 0.f;
      }
      float sum = p[i];
#pragma unroll
      for (int offset = 8; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, FE_WAVE);
      l_run[i] = l_run[i] * corr[i] + sum;
      m_run[i] = m_new;
    }
    // hand the probabilities and corrections to the value lanes through LDS
#pragma unroll
    for (int i = 0; i < 4; ++i) Ps[wave][lq * 4 + i][lr] = p[i];
    if (lr == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) Cs[wave][lq * 4 + i] = corr[i];
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      const float cg = Cs[wave][g];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] *= cg;
    }
#pragma unroll
    for (int j = 0; j < TILE / KPI; ++j) {
      float v[8];
      unpack8(vb[j], v);
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        const float pg = Ps[wave][g][j * KPI + kq];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(pg, v[e], acc[g][e]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // add up the key groups of the wave (lanes that differ in kq hold the same dims)
#pragma unroll
  for (int g = 0; g < GT; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float v = acc[g][e];
#pragma unroll
      for (int offset = LPK; offset < 64; offset <<= 1) v += __shfl_xor(v, offset, FE_WAVE);
      acc[g][e] = v;
    }
  if (kq == 0) {
#pragma unroll
    for (int g = 0; g < GT; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) Ow[wave][g][dl * 8 + e] = acc[g][e];
  }
  if (lr == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (lq * 4 + i < GT) { Ms[wave][lq * 4 + i] = m_run[i]; Ls[wave][lq * 4 + i] = l_run[i]; }
  }
  __syncthreads();

  // merge the four waves; write the result, or this split's partial result
  for (int e = tid; e < groups * D; e += 256) {
    const int g = e / D, d = e - g * D;
    float m_tot = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) m_tot = fmaxf(m_tot, Ms[w][g]);
    float o = 0.f, l = 0.f;
    if (m_tot > -INFINITY) {
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float f = __expf(Ms[w][g] - m_tot);
        o += f * Ow[w][g][d];
        l += f * Ls[w][g];
      }
    }
    if (splits == 1) {
      out[(size_t)q0 * out_stride + (size_t)(hk * groups + g) * D + d] = float_to_bf16(l > 0.f ? o / l : 0.f);
    } else {
      const size_t slot = ((size_t)seq * kv_heads + hk) * splits + split;
      part_o[(slot * groups + g) * D + d] = o;
      if (d == 0) {
        part_ml[(slot * groups + g) * 2] = m_tot;
        part_ml[(slot * groups + g) * 2 + 1] = l;
      }
    }
  }
}

// Merge the splits of one (sequence, kv head): grid (kv head, sequence).
__global__ __launch_bounds__(256) void paged_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    long long out_stride, const int* __restrict__ cu_q, int kv_heads, int groups, int head_dim,
    int splits) {
  const int hk = blockIdx.x, seq = blockIdx.y;
  const int q0 = cu_q[seq];
  if (cu_q[seq + 1] - q0 != 1) return;
  const size_t first = ((size_t)seq * kv_heads + hk) * splits;
  for (int e = threadIdx.x; e < groups * head_dim; e += blockDim.x) {
    const int g = e / head_dim, d = e - g * head_dim;
    float m_tot = -INFINITY;
    for (int s = 0; s < splits; ++s) m_tot = fmaxf(m_tot, part_ml[((first + s) * groups + g) * 2]);
    float o = 0.f, l = 0.f;
    if (m_tot > -INFINITY) {
      for (int s = 0; s < splits; ++s) {
        const float f = __expf(part_ml[((first + s) * groups + g) * 2] - m_tot);
        o += f * part_o[((first + s) * groups + g) * head_dim + d];
        l += f * part_ml[((first + s) * groups + g) * 2 + 1];
      }
    }
    out[(size_t)q0 * out_stride + (size_t)(hk * groups + g) * head_dim + d] = float_to_bf16(l > 0.f ? o / l : 0.f);
  }
}

template <int D>
static int launch_decode(int gt, dim3 grid, const void* q, long long q_stride, const void* kp, const void* vp,
                         void* out, long long out_stride, float* part_o, float* part_ml, const int* cu_q,
                         const int* ctx_len, const int* table, int table_stride, int kv_heads, int groups,
                         int block_size, int num_blocks, int window, float scale, hipStream_t stream) {
#define FE_GO(GT)                                                                                          \
  paged_decode_kernel<D, GT><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)kp,        \
      (const bf16_t*)vp, (bf16_t*)out, out_stride, part_o, part_ml, cu_q, ctx_len, table, table_stride,      \
      kv_heads, groups, block_size, num_blocks, window, scale)
  if (gt <= 1) FE_GO(1);
  else if (gt <= 2) FE_GO(2);
  else if (gt <= 4) FE_GO(4);
  else FE_GO(8);
#undef FE_GO
  return fe_check_launch();
}

// Sequences with one query token only; others are left untouched.  splits > 1
// needs part_o [num_seqs * kv_heads * splits * groups * head_dim] and part_ml
// [num_seqs * kv_heads * splits * groups * 2] floats.
extern "C" int fe_paged_attention_decode(const void* q, long long q_stride, const void* key_pages,
                                         const void* value_pages, void* out, long long out_stride,
                                         float* part_o, float* part_ml, const int* cu_q,
                                         const int* ctx_len, const int* block_table, int table_stride,
                                         int num_seqs, int kv_heads, int groups, int head_dim,
                                         int block_size, int num_blocks, int window, float scale,
                                         int splits, hipStream_t stream) {
  if (num_seqs <= 0) return FE_OK;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return FE_BAD_ARGUMENT;
  if (groups < 1 || groups > 8 || kv_heads < 1 || kv_heads > 65535 || num_seqs > 65535) return FE_BAD_ARGUMENT;
  if (block_size < TILE || block_size % TILE || num_blocks < 1 || table_stride < 1) return FE_BAD_ARGUMENT;
  if (q_stride % 8 || splits < 1 || splits > 1024) return FE_BAD_ARGUMENT;
  if (splits > 1 && (!part_o || !part_ml)) return FE_BAD_ARGUMENT;
  dim3 grid(splits, kv_heads, num_seqs);
  int status;
  if (head_dim == 64)
    status = launch_decode<64>(groups, grid, q, q_stride, key_pages, value_pages, out, out_stride, part_o, part_ml, cu_q, ctx_len, block_table, table_stride, kv_heads, groups, block_size, num_blocks, window, scale, stream);
  else if (head_dim == 128)
    status = launch_decode<128>(groups, grid, q, q_stride, key_pages, value_pages, out, out_stride, part_o, part_ml, cu_q, ctx_len, block_table, table_stride, kv_heads, groups, block_size, num_blocks, window, scale, stream);
  else
    status = launch_decode<256>(groups, grid, q, q_stride, key_pages, value_pages, out, out_stride, part_o, part_ml, cu_q, ctx_len, block_table, table_stride, kv_heads, groups, block_size, num_blocks, window, scale, stream);
  if (status != FE_OK || splits == 1) return status;
  dim3 merge_grid(kv_heads, num_seqs);
  paged_decode_merge_kernel<<<merge_grid, 256, 0, stream>>>(part_o, part_ml, (bf16_t*)out, out_stride, cu_q,
                                                            kv_heads, groups, head_dim, splits);
  return fe_check_launch();
}
