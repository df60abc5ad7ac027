// Shared device helpers for the gfx950 kernels: element types, wave and block
// reductions.  Everything here assumes 64-wide wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define FE_WAVE 64

// Status codes returned by every extern "C" entry point.
#define FE_OK 0
#define FE_BAD_ARGUMENT 1
#define FE_LAUNCH_FAILED 2

// Element type tags used across the C interface.
#define FE_F32 0
#define FE_BF16 1

typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

__device__ __forceinline__ float load_as_float(const float* p) { return *p; }
__device__ __forceinline__ float load_as_float(const bf16_t* p) { return bf16_to_float(*p); }
__device__ __forceinline__ void store_from_float(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_from_float(bf16_t* p, float v) { *p = float_to_bf16(v); }

// This lane's value combined with that of lane ^ 16 or lane ^ 32 by the lane-swap instructions
// of gfx950 (vector ALU, no trip through the LDS crossbar, which a general shuffle takes with a
// wait behind it).  permlane16_swap(a, b) exchanges the odd rows of 16 lanes of a with the even
// rows of b, permlane32_swap the upper half of a with the lower half of b; with a = b = v the two
// results hold, in every lane, the values of both partners.  The sums have the same bits in both
// partners and the same bits as v + shuffle(v).
__device__ __forceinline__ float sum_xor16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float max_xor16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, FE_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, FE_WAVE));
  return v;
}

// The same over the data-parallel lane permutes and the lane swaps: no trip through the LDS
// crossbar (six of them, each with a wait behind it, in the forms above).  Another order of the
// same additions, so not for code whose bits another kernel has to reproduce.
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // lane ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // 7 - lane within 8
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // 15 - lane within 16
  return sum_xor32(sum_xor16(v));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true)));
  return max_xor32(max_xor16(v));
}

// Sum over a block of up to 1024 threads; `scratch` holds one float per wave
// (at least 16).  Every thread gets the total.  Contains two barriers, or one where nothing
// has used `scratch` before (SCRATCH_IS_FRESH).
template <bool SCRATCH_IS_FRESH = false>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (FE_WAVE - 1);
  const int wave = threadIdx.x / FE_WAVE;
  const int waves = (blockDim.x + FE_WAVE - 1) / FE_WAVE;
  v = wave_sum_dpp(v);
  if (!SCRATCH_IS_FRESH) __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < waves; ++i) total += scratch[i];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (FE_WAVE - 1);
  const int wave = threadIdx.x / FE_WAVE;
  const int waves = (blockDim.x + FE_WAVE - 1) / FE_WAVE;
  v = wave_max_dpp(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int i = 1; i < waves; ++i) total = fmaxf(total, scratch[i]);
  return total;
}

static inline int fe_check_launch() {
  return hipGetLastError() == hipSuccess ? FE_OK : FE_LAUNCH_FAILED;
}
