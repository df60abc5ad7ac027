// The arithmetic of a head's RMSNorm and rotation for bfloat16 heads whose size is a power of
// two, written once with explicit fused multiply-adds: two kernels prepare queries and keys
// (the stand-alone one and the decode attention kernel that does it on the way), and what one
// writes into the cache must be bit for bit what the other would have written.
//
// A head is handled as chunks of 8 consecutive elements.  The sum of squares is formed per
// chunk (in element order) and the chunks are then combined as a butterfly over the chunk
// index, largest distance first: chunk_total[i] += chunk_total[i ^ offset] for offset =
// chunks / 2, ..., 1.  Addition is commutative, so every chunk ends with the same total, and
// a kernel may run the butterfly over lanes, over registers, or over both.
#pragma once
#include "common.h"

__device__ __forceinline__ void unpack_bf16x8(const uint32_t w[4], float v[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(w[e] << 16);
    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
  }
}

__device__ __forceinline__ float sum_squares8(const float v[8]) {
  float s = v[0] * v[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) s = __fmaf_rn(v[e], v[e], s);
  return s;
}

// 1 / sqrt(mean of squares + eps) for a head of `dim` elements, dim a power of two (the
// division is exact as a multiplication).
__device__ __forceinline__ float inverse_rms(float sum_squares, int dim, float eps) {
  return rsqrtf(__fmaf_rn(sum_squares, 1.f / (float)dim, eps));
}

__device__ __forceinline__ float normalise(float v, float inv, float weight) { return (v * inv) * weight; }

// Element j < dim/2 and its partner j + dim/2 under the angle of j.
__device__ __forceinline__ float rotate_low(float v, float partner, float cs, float sn) {
  return __fmaf_rn(v, cs, -(partner * sn));
}
__device__ __forceinline__ float rotate_high(float v, float partner, float cs, float sn) {
  return __fmaf_rn(v, cs, partner * sn);
}

__device__ __forceinline__ void pack_bf16x8(const float r[8], uint32_t w[4]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = (uint32_t)float_to_bf16(r[2 * e]) | ((uint32_t)float_to_bf16(r[2 * e + 1]) << 16);
}
