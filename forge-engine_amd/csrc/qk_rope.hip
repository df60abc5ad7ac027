// Fused per-head RMSNorm of q and k, rotary position encoding, and the write of
// k and v into the paged cache.  Input is the fused projection output
// qkv[T, (Hq + 2*Hkv) * D]; q is normalised and rotated in place, k is
// normalised, rotated and written to its page, v is copied to its page.
//
//   y      = x * rsqrt(mean_D(x^2) + eps) * w           (skipped if w is null)
//   angle  = float(position) * inv_freq[j],  j < R/2     (R = rotary_dim <= D)
//   out[j]       = y[j] * cos(angle) - y[j + R/2] * sin(angle)
//   out[j + R/2] = y[j + R/2] * cos(angle) + y[j] * sin(angle)
//   dims >= R pass through.  All arithmetic in float32, one rounding at the store.
//
// Cache layout per layer: keys pages[block][kv_head][slot][D]; values transposed,
// pages[block][kv_head][D][slot], so that the attention kernels read 8 consecutive
// keys of one dim in one piece (the matrix cores reduce over keys there).  The
// token at position p of sequence s lives in block table[s][p / block_size],
// slot p % block_size.
#include "common.h"
#include "rope_math.h"
#include <algorithm>

// One block serves `heads_per_block` heads of one token (4 waves, a head per wave at a time).
// The cosines and sines of the token's angles are computed once per block into LDS: with many
// tokens a block takes all heads of its token, so the (accurate, slow for large angles) sincosf
// runs once per (token, frequency) instead of once per head.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_write_kernel(
    T* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ inv_freq, const int* __restrict__ positions,
    const int* __restrict__ token_seq, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ key_pages, T* __restrict__ value_pages, int q_heads, int kv_heads,
    int head_dim, int rotary_dim, int block_size, int num_blocks, float eps, int write_kv,
    int heads_per_block, int groups_per_token) {
  __shared__ float cos_s[256], sin_s[256];
  __shared__ float stage[4][512];
  const int lane = threadIdx.x & (FE_WAVE - 1);
  const int wave = threadIdx.x / FE_WAVE;
  const int t = blockIdx.x / groups_per_token;
  const int group = blockIdx.x - t * groups_per_token;
  const int heads_all = q_heads + 2 * kv_heads;
  const int head_end = min(heads_all, (group + 1) * heads_per_block);
  const int pos = positions[t];
  const int half = head_dim / 2;
  const int rhalf = rotary_dim / 2;
  for (int j = threadIdx.x; j < rhalf; j += blockDim.x) {
    float sn, cs;
    sincosf((float)pos * inv_freq[j], &sn, &cs);
    cos_s[j] = cs;
    sin_s[j] = sn;
  }
  __syncthreads();

  for (int head = group * heads_per_block + wave; head < head_end; head += 4) {
    T* x = qkv + ((size_t)t * heads_all + head) * head_dim;
    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;
    const int kv_head = is_q ? 0 : (is_k ? head - q_heads : head - q_heads - kv_heads);

    T* dst = x;  // q stays in place
    if (!is_q) {
      if (!write_kv) continue;
      const int seq = token_seq[t];
      const int block = block_table[(size_t)seq * table_stride + pos / block_size];
      if (block < 0 || block >= num_blocks) continue;  // host reserves pages before the launch
      const size_t page = ((size_t)block * kv_heads + kv_head) * block_size * head_dim;
      if (!is_k) {  // value: copy into the transposed page
        T* vdst = value_pages + page + (pos % block_size);
        for (int d = lane; d < head_dim; d += FE_WAVE) vdst[(size_t)d * block_size] = x[d];
        continue;
      }
      dst = key_pages + page + (size_t)(pos % block_size) * head_dim;
    }

    const float* w = is_q ? q_weight : k_weight;
    // Each lane owns pairs (j, j + half) for j = lane, lane + 64, ...; head_dim <= 512.
    float lo[4], hi[4];
    float sumsq = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = lane + i * FE_WAVE;
      lo[i] = 0.f; hi[i] = 0.f;
      if (j < half) {
        lo[i] = load_as_float(x + j);
        hi[i] = load_as_float(x + j + half);
        sumsq += lo[i] * lo[i] + hi[i] * hi[i];
      }
    }
    float inv = 1.f;
    if (w) {
      sumsq = wave_sum(sumsq);
      inv = rsqrtf(sumsq / (float)head_dim + eps);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = lane + i * FE_WAVE;
      if (j < half) {
        if (w) {
          lo[i] = lo[i] * inv * w[j];
          hi[i] = hi[i] * inv * w[j + half];
        }
      }
    }
    // Rotation pairs are (j, j + rhalf) for j < rhalf.  With rotary_dim == head_dim
    // the partner of lo[i] is hi[i] and everything stays in registers.
    if (rotary_dim == head_dim) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = lane + i * FE_WAVE;
        if (j < half) {
          const float sn = sin_s[j], cs = cos_s[j];
          const float a = lo[i], b = hi[i];
          store_from_float(dst + j, a * cs - b * sn);
          store_from_float(dst + j + half, b * cs + a * sn);
        }
      }
    } else {
      // Partial rotation: partners may sit in other lanes, so the normalised head
      // goes through a per-wave LDS buffer (LDS operations of one wave are ordered).
      float* buf = stage[wave];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = lane + i * FE_WAVE;
        if (j < half) { buf[j] = lo[i]; buf[j + half] = hi[i]; }
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
      for (int d = lane; d < head_dim; d += FE_WAVE) {
        float v = buf[d];
        if (d < rotary_dim) {
          const int j = d < rhalf ? d : d - rhalf;
          const float sn = sin_s[j], cs = cos_s[j];
          v = d < rhalf ? buf[d] * cs - buf[d + rhalf] * sn : buf[d] * cs + buf[d - rhalf] * sn;
        }
        store_from_float(dst + d, v);
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();      // the buffer is written again for the wave's next head
    }
  }
}

// The same for bfloat16 heads of 16 * 2^n elements that are rotated whole (rotary_dim == head_dim):
// head_dim / 8 lanes share a head, each with 8 consecutive elements (one 16-byte load and store),
// so a wave works on 512 / head_dim heads at once; the partner of element j, j + head_dim / 2,
// sits in the lane head_dim / 16 further on (one shuffle per element).
#define VEC_ROUNDS 3   // rounds of 2048 / head_dim heads that a block of the kernel below takes at most
template <int LPH>    // lanes per head
__global__ __launch_bounds__(256) void qk_norm_rope_write_vec_kernel(
    bf16_t* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ inv_freq, const int* __restrict__ positions,
    const int* __restrict__ token_seq, const int* __restrict__ block_table, int table_stride,
    bf16_t* __restrict__ key_pages, bf16_t* __restrict__ value_pages, int q_heads, int kv_heads,
    int block_size, int num_blocks, float eps, int write_kv, int heads_per_block, int groups_per_token,
    int tokens, int values_apart) {
  constexpr int D = LPH * 8;
  constexpr int HALF = D / 2;
  constexpr int HEADS_AT_ONCE = 256 / LPH;
  const int heads_all = q_heads + 2 * kv_heads;
  if (values_apart && (int)blockIdx.x >= tokens * groups_per_token) {
    // Values of 16 neighbouring tokens and one kv head, turned through LDS: a token's value is
    // a row of the projection's output and a column of its page ([D][slot]), so written token
    // by token every element is a 2-byte store of its own, 2 * block_size bytes from the next.
    // Here 16 lanes write 16 neighbouring slots of one dim (tokens of one sequence follow one
    // another in the batch), which the memory system takes as one piece.
    constexpr int PITCH = D + 8;            // elements; rows stay 16-byte aligned, columns spread over the banks
    __shared__ __attribute__((aligned(16))) bf16_t rows[16][PITCH];
    __shared__ long long slot_at[16];       // element offset of [page][kv_head][0][slot], or -1
    const int vb = blockIdx.x - tokens * groups_per_token;
    const int kv_head = vb % kv_heads;
    const int t0 = (vb / kv_heads) * 16;
    if (threadIdx.x < 16) {
      const int t = t0 + threadIdx.x;
      long long at = -1;
      if (t < tokens) {
        const int pos = positions[t];
        const int block = block_table[(size_t)token_seq[t] * table_stride + pos / block_size];
        if (block >= 0 && block < num_blocks)       // host reserves pages before the launch
          at = ((long long)block * kv_heads + kv_head) * block_size * D + pos % block_size;
      }
      slot_at[threadIdx.x] = at;
    }
    for (int piece = threadIdx.x; piece < 16 * LPH; piece += 256) {
      const int row = piece / LPH, sub = piece % LPH;
      const int t = min(t0 + row, tokens - 1);
      *(uint4*)&rows[row][sub * 8] =
          *(const uint4*)(qkv + ((size_t)t * heads_all + q_heads + kv_heads + kv_head) * D + sub * 8);
    }
    __syncthreads();
    const int row = threadIdx.x & 15;
    const long long at = slot_at[row];
    if (at < 0) return;
    for (int d = threadIdx.x >> 4; d < D; d += 16) value_pages[at + (long long)d * block_size] = rows[row][d];
    return;
  }
  __shared__ float cos_s[HALF], sin_s[HALF];
  const int t = blockIdx.x / groups_per_token;
  const int group = blockIdx.x - t * groups_per_token;
  const int head_end = min(values_apart ? q_heads + kv_heads : heads_all, (group + 1) * heads_per_block);
  const int sub = threadIdx.x % LPH;          // which 8 elements of the head
  const int first = sub * 8;
  const bool low = first < HALF;              // elements of the first half pair with the second
  // A block's time is a chain of trips to memory, not bytes: the heads' elements, which depend on
  // nothing, are asked for before the position is (and with it the sines and cosines), for all of the
  // block's up to ROUNDS rounds of heads, in straight-line code (a loop around the rounds made the
  // compiler wait for every load where the loop's branches meet).  At 256 tokens 6.6 -> 5.3 us, at
  // 8,192 tokens 54 -> 47.
  const int head_first = group * heads_per_block + threadIdx.x / LPH;
  constexpr int ROUNDS = VEC_ROUNDS;         // the host gives a block at most this many rounds of heads
  uint4 raws[ROUNDS];
#pragma unroll
  for (int round = 0; round < ROUNDS; ++round) {
    const int head = min(head_first + round * HEADS_AT_ONCE, heads_all - 1);    // a round past the end reads the last head again
    raws[round] = *(const uint4*)(qkv + ((size_t)t * heads_all + head) * D + first);
  }
  const int pos = positions[t];
  const int block = write_kv ? block_table[(size_t)token_seq[t] * table_stride + pos / block_size] : -1;
  for (int j = threadIdx.x; j < HALF; j += blockDim.x) {
    float sn, cs;
    sincosf((float)pos * inv_freq[j], &sn, &cs);
    cos_s[j] = cs;
    sin_s[j] = sn;
  }
  __syncthreads();
#pragma unroll
  for (int round = 0; round < ROUNDS; ++round) {
    const int head = head_first + round * HEADS_AT_ONCE;
    if (head >= head_end) break;
    bf16_t* x = qkv + ((size_t)t * heads_all + head) * D + first;
    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;
    if (!is_q && !write_kv) continue;
    const uint4 raw = raws[round];
    size_t page = 0;
    int slot = 0;
    if (!is_q) {
      const int kv_head = is_k ? head - q_heads : head - q_heads - kv_heads;
      if (block < 0 || block >= num_blocks) continue;  // host reserves pages before the launch
      page = ((size_t)block * kv_heads + kv_head) * block_size * D;
      slot = pos % block_size;
      if (!is_k) {   // value: into the transposed page, element d at [d][slot]
        const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
        bf16_t* vdst = value_pages + page + slot;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          vdst[(size_t)(first + e) * block_size] = (bf16_t)(e & 1 ? w4[e >> 1] >> 16 : w4[e >> 1] & 0xffffu);
        continue;
      }
    }
    float v[8];
    {
      const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
      unpack_bf16x8(w4, v);
    }
    const float* w = is_q ? q_weight : k_weight;
    if (w) {
      float sumsq = sum_squares8(v);
#pragma unroll
      for (int offset = LPH / 2; offset > 0; offset >>= 1) sumsq += __shfl_xor(sumsq, offset, FE_WAVE);
      const float inv = inverse_rms(sumsq, D, eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = normalise(v[e], inv, w[first + e]);
    }
    uint32_t o4[4];
    float r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float other = __shfl_xor(v[e], LPH / 2, FE_WAVE);     // element first + e -/+ HALF
      const int j = (first + e) & (HALF - 1);
      r[e] = low ? rotate_low(v[e], other, cos_s[j], sin_s[j]) : rotate_high(v[e], other, cos_s[j], sin_s[j]);
    }
    pack_bf16x8(r, o4);
    bf16_t* dst = is_q ? x : key_pages + page + (size_t)slot * D + first;
    *(uint4*)dst = make_uint4(o4[0], o4[1], o4[2], o4[3]);
  }
}

extern "C" int fe_qk_norm_rope_write(void* qkv, int dtype, const float* q_weight, const float* k_weight,
                                     const float* inv_freq, const int* positions, const int* token_seq,
                                     const int* block_table, int table_stride, void* key_pages,
                                     void* value_pages, int tokens, int q_heads, int kv_heads,
                                     int head_dim, int rotary_dim, int block_size, int num_blocks,
                                     float eps, int write_kv, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (q_heads < 0 || kv_heads < 0 || head_dim <= 0 || head_dim % 2 || head_dim > 512) return FE_BAD_ARGUMENT;
  if (rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2) return FE_BAD_ARGUMENT;
  if (rotary_dim > 0 && !inv_freq) return FE_BAD_ARGUMENT;
  if (write_kv && (block_size <= 0 || num_blocks <= 0 || !block_table || !key_pages || !value_pages)) return FE_BAD_ARGUMENT;
  const long long work = (long long)tokens * (q_heads + 2 * kv_heads);
  if (work <= 0 || work > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  // few tokens: four heads a block, so that the launch has many blocks; many tokens: a block per
  // token, so that the angles' sines and cosines are computed once per token (the vector kernel:
  // one round of heads a block with few tokens, with many up to VEC_ROUNDS rounds, 48 heads of 128)
  const int heads_all = q_heads + 2 * kv_heads;
  const bool vec = dtype == FE_BF16 && rotary_dim == head_dim && (head_dim == 64 || head_dim == 128 || head_dim == 256) &&
                   ((((uintptr_t)qkv) | ((uintptr_t)key_pages)) & 15) == 0;
  // the vector kernel works on 2048 / head_dim heads at once
  const int heads_per_block = vec ? std::min(heads_all, (tokens >= 256 ? VEC_ROUNDS : 1) * (2048 / head_dim))
                                  : (tokens >= 256 ? heads_all : 4);
  const int groups_per_token = (heads_all + heads_per_block - 1) / heads_per_block;
  long long blocks = (long long)tokens * groups_per_token;
  if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  if (vec) {
    // with many tokens the values go to blocks of their own that write 16 slots of a page at a time
    const int values_apart = write_kv && kv_heads > 0 && tokens >= 256;
    if (values_apart) blocks += (long long)((tokens + 15) / 16) * kv_heads;
    if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
#define FE_GO(LPH)                                                                                          \
  qk_norm_rope_write_vec_kernel<LPH><<<(unsigned)blocks, 256, 0, stream>>>(                                   \
      (bf16_t*)qkv, q_weight, k_weight, inv_freq, positions, token_seq, block_table, table_stride,            \
      (bf16_t*)key_pages, (bf16_t*)value_pages, q_heads, kv_heads, block_size, num_blocks, eps, write_kv,     \
      heads_per_block, groups_per_token, tokens, values_apart)
    if (head_dim == 64) FE_GO(8);
    else if (head_dim == 128) FE_GO(16);
    else FE_GO(32);
#undef FE_GO
    return fe_check_launch();
  }
  if (dtype == FE_F32)
    qk_norm_rope_write_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(
        (float*)qkv, q_weight, k_weight, inv_freq, positions, token_seq, block_table, table_stride,
        (float*)key_pages, (float*)value_pages, q_heads, kv_heads, head_dim, rotary_dim, block_size,
        num_blocks, eps, write_kv, heads_per_block, groups_per_token);
  else if (dtype == FE_BF16)
    qk_norm_rope_write_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(
        (bf16_t*)qkv, q_weight, k_weight, inv_freq, positions, token_seq, block_table, table_stride,
        (bf16_t*)key_pages, (bf16_t*)value_pages, q_heads, kv_heads, head_dim, rotary_dim, block_size,
        num_blocks, eps, write_kv, heads_per_block, groups_per_token);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}
