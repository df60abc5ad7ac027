// Row-wise kernels: embedding gather, (residual add +) RMSNorm, SwiGLU.
// The residual stream is float32 in every mode; activations handed to matrix
// products are float32 or bfloat16.
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[t, :] = float(table[ids[t], :]).  One block per token.
template <typename TW>
__global__ void embed_rows_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                                  float* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* dst = out + (size_t)t * hidden;
  if (id < 0 || id >= vocab) {  // host validates ids; never read outside the table
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = __int_as_float(0x7fc00000);
    return;
  }
  const TW* src = table + (size_t)id * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = load_as_float(src + i);
}

extern "C" int fe_embed_rows(const int* ids, const void* table, int table_dtype, float* out,
                             int tokens, int hidden, int vocab, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (hidden <= 0 || vocab <= 0) return FE_BAD_ARGUMENT;
  const int threads = hidden >= 1024 ? 256 : 64;
  if (table_dtype == FE_F32)
    embed_rows_kernel<float><<<tokens, threads, 0, stream>>>(ids, (const float*)table, out, hidden, vocab);
  else if (table_dtype == FE_BF16)
    embed_rows_kernel<bf16_t><<<tokens, threads, 0, stream>>>(ids, (const bf16_t*)table, out, hidden, vocab);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// ------------------------------------------------------- add + RMSNorm
// For output row r (source row s = rows ? rows[r] : r):
//   sum = h[s] + delta[s]          (float32; written back to h[s] if store_sum)
//   out[r] = sum * rsqrt(mean(sum^2) + eps) * w
// delta may come in `parts` pieces `part_stride` elements apart (the partial sums of a product
// whose K was split over blocks); they are added in order before anything else.
// Statistics, scaling and the weight product are float32; one rounding at the
// store.  One block per row; the row is re-read from h/delta in the second
// pass (it is cache-resident), so any width works.
template <typename TD>
__device__ __forceinline__ float delta_sum(const TD* p, int parts, size_t part_stride) {
  float d = load_as_float(p);
  for (int k = 1; k < parts; ++k) d += load_as_float(p + k * part_stride);
  return d;
}

template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                   const float* __restrict__ w, TO* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps,
                                   int store_sum, int parts, size_t part_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int s = rows ? rows[r] : r;
  float* hrow = h + (size_t)s * hidden;
  const TD* drow = delta ? delta + (size_t)s * hidden : nullptr;
  float sumsq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = hrow[i];
    if (drow) {
      v += delta_sum(drow + i, parts, part_stride);
      if (store_sum) hrow[i] = v;
    }
    sumsq += v * v;
  }
  const float total = block_sum<true>(sumsq, scratch);
  const float inv = rsqrtf(total / (float)hidden + eps);
  TO* orow = out + (size_t)r * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = hrow[i];
    if (drow && !store_sum) v += delta_sum(drow + i, parts, part_stride);
    store_from_float(orow + i, v * inv * w[i]);
  }
}

// The same for rows of up to 256 * 4 * VEC floats with hidden % 4 == 0: the row stays in
// registers between the two passes and memory is touched in 16-byte pieces.
__device__ __forceinline__ float4 load4_as_float(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 load4_as_float(const bf16_t* p) {
  const uint2 v = *(const uint2*)p;
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                     __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}
__device__ __forceinline__ void store4_from_float(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void store4_from_float(bf16_t* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16(v.x) | ((uint32_t)float_to_bf16(v.y) << 16);
  u.y = (uint32_t)float_to_bf16(v.z) | ((uint32_t)float_to_bf16(v.w) << 16);
  *(uint2*)p = u;
}

template <typename TD, typename TO, int VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_regs_kernel(
    float* __restrict__ h, const TD* __restrict__ delta, const float* __restrict__ w,
    TO* __restrict__ out, const int* __restrict__ rows, int hidden, float eps, int store_sum,
    int parts, size_t part_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int s = rows ? rows[r] : r;
  float* hrow = h + (size_t)s * hidden;
  const TD* drow = delta ? delta + (size_t)s * hidden : nullptr;
  float4 v[VEC], ww[VEC];      // the norm's weight is requested with the row, not after the sum
  float sumsq = 0.f;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int i = (threadIdx.x + j * THREADS) * 4;
    v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    ww[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < hidden) {
      v[j] = load4_as_float(hrow + i);
      ww[j] = *(const float4*)(w + i);
      if (drow) {
        float4 d = load4_as_float(drow + i);
        for (int k = 1; k < parts; k += 8) {     // eight parts' loads fly together; added in order
          float4 e[8];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            e[u] = k + u < parts ? load4_as_float(drow + (k + u) * part_stride + i) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (k + u < parts) { d.x += e[u].x; d.y += e[u].y; d.z += e[u].z; d.w += e[u].w; }
        }
        v[j].x += d.x; v[j].y += d.y; v[j].z += d.z; v[j].w += d.w;
        if (store_sum) *(float4*)(hrow + i) = v[j];
      }
      sumsq += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  const float total = block_sum<true>(sumsq, scratch);
  const float inv = rsqrtf(total / (float)hidden + eps);
  TO* orow = out + (size_t)r * hidden;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int i = (threadIdx.x + j * THREADS) * 4;
    if (i < hidden)
      store4_from_float(orow + i, make_float4(v[j].x * inv * ww[j].x, v[j].y * inv * ww[j].y,
                                              v[j].z * inv * ww[j].z, v[j].w * inv * ww[j].w));
  }
}

template <typename TD, typename TO>
static void launch_add_rmsnorm_typed(float* h, const TD* delta, const float* w, TO* out, const int* rows,
                                     int n_rows, int hidden, float eps, int store_sum, int parts,
                                     size_t part_stride, hipStream_t stream) {
  const bool aligned = hidden % 4 == 0 && part_stride % 4 == 0 && (((uintptr_t)h | (uintptr_t)delta | (uintptr_t)w | (uintptr_t)out) & 15) == 0;
  if (aligned && n_rows <= 512 && hidden > 1024 && hidden <= 4096)   // up to a few hundred rows: a whole row in flight at once
    add_rmsnorm_regs_kernel<TD, TO, 1, 1024><<<n_rows, 1024, 0, stream>>>(h, delta, w, out, rows, hidden, eps, store_sum, parts, part_stride);
  else if (aligned && n_rows <= 512 && hidden > 4096 && hidden <= 8192)
    add_rmsnorm_regs_kernel<TD, TO, 2, 1024><<<n_rows, 1024, 0, stream>>>(h, delta, w, out, rows, hidden, eps, store_sum, parts, part_stride);
  else if (aligned && hidden <= 1024)
    add_rmsnorm_regs_kernel<TD, TO, 1, 256><<<n_rows, 256, 0, stream>>>(h, delta, w, out, rows, hidden, eps, store_sum, parts, part_stride);
  else if (aligned && hidden <= 4096)
    add_rmsnorm_regs_kernel<TD, TO, 4, 256><<<n_rows, 256, 0, stream>>>(h, delta, w, out, rows, hidden, eps, store_sum, parts, part_stride);
  else if (aligned && hidden <= 8192)
    add_rmsnorm_regs_kernel<TD, TO, 8, 256><<<n_rows, 256, 0, stream>>>(h, delta, w, out, rows, hidden, eps, store_sum, parts, part_stride);
  else {
    const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
    add_rmsnorm_kernel<TD, TO><<<n_rows, threads, 0, stream>>>(h, delta, w, out, rows, hidden, eps, store_sum, parts, part_stride);
  }
}

template <typename TD>
static int launch_add_rmsnorm(float* h, const TD* delta, const float* w, void* out, int out_dtype,
                              const int* rows, int n_rows, int hidden, float eps, int store_sum,
                              int parts, size_t part_stride, hipStream_t stream) {
  if (out_dtype == FE_F32)
    launch_add_rmsnorm_typed<TD, float>(h, delta, w, (float*)out, rows, n_rows, hidden, eps, store_sum, parts, part_stride, stream);
  else if (out_dtype == FE_BF16)
    launch_add_rmsnorm_typed<TD, bf16_t>(h, delta, w, (bf16_t*)out, rows, n_rows, hidden, eps, store_sum, parts, part_stride, stream);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// delta may be null (plain RMSNorm).  rows may be null (all n_rows rows in order).
// With rows given, store_sum must be 0 unless the rows are distinct.  delta_parts >= 1 pieces of
// delta lie part_stride elements apart.
extern "C" int fe_add_rmsnorm(float* h, const void* delta, int delta_dtype, const float* w,
                              void* out, int out_dtype, const int* rows, int n_rows, int hidden,
                              float eps, int store_sum, int delta_parts, long long part_stride,
                              hipStream_t stream) {
  if (n_rows <= 0) return FE_OK;
  if (hidden <= 0 || !(eps > 0.f) || delta_parts < 1 || delta_parts > 64 || part_stride < 0) return FE_BAD_ARGUMENT;
  if (delta == nullptr || delta_dtype == FE_F32)
    return launch_add_rmsnorm<float>(h, (const float*)delta, w, out, out_dtype, rows, n_rows, hidden, eps, store_sum, delta_parts, (size_t)part_stride, stream);
  if (delta_dtype == FE_BF16)
    return launch_add_rmsnorm<bf16_t>(h, (const bf16_t*)delta, w, out, out_dtype, rows, n_rows, hidden, eps, store_sum, delta_parts, (size_t)part_stride, stream);
  return FE_BAD_ARGUMENT;
}

// h[t] += delta[t] for all rows (flushes a pending update without a norm); delta in `parts`
// pieces `part_stride` elements apart, added in order.
template <typename TD>
__global__ void add_rows_kernel(float* __restrict__ h, const TD* __restrict__ delta, size_t count, int parts,
                                size_t part_stride) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
    h[i] += delta_sum(delta + i, parts, part_stride);
}

extern "C" int fe_add_rows(float* h, const void* delta, int delta_dtype, long long count, int delta_parts,
                           long long part_stride, hipStream_t stream) {
  if (count <= 0) return FE_OK;
  if (delta_parts < 1 || delta_parts > 64 || part_stride < 0) return FE_BAD_ARGUMENT;
  const int threads = 256;
  long long want = (count + threads - 1) / threads;
  const int blocks = (int)(want < 4096 ? want : 4096);
  if (delta_dtype == FE_F32)
    add_rows_kernel<float><<<blocks, threads, 0, stream>>>(h, (const float*)delta, (size_t)count, delta_parts, (size_t)part_stride);
  else if (delta_dtype == FE_BF16)
    add_rows_kernel<bf16_t><<<blocks, threads, 0, stream>>>(h, (const bf16_t*)delta, (size_t)count, delta_parts, (size_t)part_stride);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// ---------------------------------------------------------------- SwiGLU
// gate_up is [T, 2*inter] with gate in the first half of each row:
//   out[t, i] = silu(gate[t, i]) * up[t, i],  silu(z) = z / (1 + exp(-z)),  in float32.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / inter;
    const int c = (int)(i - t * inter);
    const T* row = gate_up + t * 2 * (size_t)inter;
    const float g = load_as_float(row + c);
    const float u = load_as_float(row + inter + c);
    store_from_float(out + i, g / (1.f + expf(-g)) * u);
  }
}

// bfloat16 rows whose width is a multiple of 8: eight elements (16 bytes) of gate and of up per thread.
__global__ __launch_bounds__(256) void swiglu_bf16x8_kernel(const bf16_t* __restrict__ gate_up,
                                                            bf16_t* __restrict__ out, int inter8, size_t total8) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total8; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / inter8;
    const int c = (int)(i - t * inter8);
    const uint4* row = (const uint4*)gate_up + t * 2 * (size_t)inter8;
    const uint4 g = row[c];
    const uint4 u = row[inter8 + c];
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
      ow[k] = (uint32_t)float_to_bf16(g0 / (1.f + expf(-g0)) * u0) |
              ((uint32_t)float_to_bf16(g1 / (1.f + expf(-g1)) * u1) << 16);
    }
    ((uint4*)out)[i] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

extern "C" int fe_swiglu(const void* gate_up, void* out, int dtype, int tokens, int inter, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (inter <= 0) return FE_BAD_ARGUMENT;
  const size_t total = (size_t)tokens * inter;
  const int threads = 256;
  if (dtype == FE_BF16 && inter % 8 == 0 && ((((uintptr_t)gate_up) | ((uintptr_t)out)) & 15) == 0) {
    const size_t total8 = total / 8;
    const size_t want8 = (total8 + threads - 1) / threads;
    swiglu_bf16x8_kernel<<<(int)(want8 < 16384 ? want8 : 16384), threads, 0, stream>>>(
        (const bf16_t*)gate_up, (bf16_t*)out, inter / 8, total8);
    return fe_check_launch();
  }
  size_t want = (total + threads - 1) / threads;
  const int blocks = (int)(want < 8192 ? want : 8192);
  if (dtype == FE_F32)
    swiglu_kernel<float><<<blocks, threads, 0, stream>>>((const float*)gate_up, (float*)out, inter, total);
  else if (dtype == FE_BF16)
    swiglu_kernel<bf16_t><<<blocks, threads, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, inter, total);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// A plain streaming read of `bytes` bytes (a multiple of 16), for measuring what the memory
// delivers to a kernel that does nothing else: every block walks the buffer in 16-byte pieces,
// 2048 blocks of 256 threads.  sink[0] is written only if the data add up to a value they never
// have, so the loads cannot be dropped.
__global__ __launch_bounds__(256) void stream_read_kernel(const float4* __restrict__ data, size_t pieces, float* sink) {
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (size_t)gridDim.x * 256) {
    const float4 v = data[i];
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  if (s.x + s.y + s.z + s.w == 123456.789f) sink[0] = s.x;
}

extern "C" int fe_stream_read(const void* data, long long bytes, float* sink, hipStream_t stream) {
  if (bytes <= 0) return FE_OK;
  if (bytes % 16 || (((uintptr_t)data) & 15) || !sink) return FE_BAD_ARGUMENT;
  stream_read_kernel<<<2048, 256, 0, stream>>>((const float4*)data, (size_t)(bytes / 16), sink);
  return fe_check_launch();
}
