// Sampling over float32 logits rows: argmax, and a draw from
// softmax(logits / temperature) by inverse CDF with a counter-based generator.
// One block of 1024 threads per row; entries equal to -inf have probability 0
// (that is how filters remove tokens).  Each row also gets a status word:
//   bit 0: a NaN was seen, bit 1: +inf was seen, bit 2: no finite entry.
#include "common.h"
#include "sample_api.h"
#include <mutex>

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / FE_WAVE)

__device__ __forceinline__ int row_status(const float* row, int vocab, float* scratch_f, int* scratch_i) {
  int flags = 0;
  int finite = 0;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    if (v != v) flags |= 1;
    else if (v == INFINITY) flags |= 2;
    else if (v != -INFINITY) finite = 1;
  }
  // OR-reduce through LDS
  __syncthreads();
  if (threadIdx.x == 0) { scratch_i[0] = 0; scratch_i[1] = 0; }
  __syncthreads();
  if (flags) atomicOr(&scratch_i[0], flags);
  if (finite) atomicOr(&scratch_i[1], 1);
  __syncthreads();
  int result = scratch_i[0];
  if (!scratch_i[1]) result |= 4;
  (void)scratch_f;
  return result;
}

// tokens[row] = index of the largest entry; the lowest index wins ties.  Two
// stages so that a few long rows still fill the chip: ARGMAX_PARTS blocks per
// row each scan a contiguous part, then one block per row merges them.
#define ARGMAX_PARTS 32

__device__ __forceinline__ void argmax_merge(float& bv, int& bi, float ov, int oi) {
  if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}

__global__ __launch_bounds__(256) void argmax_parts_kernel(
    const float* __restrict__ logits, long long row_stride, int vocab, float* __restrict__ part_v,
    int* __restrict__ part_i, int* __restrict__ part_flags) {
  __shared__ float best_v[4];
  __shared__ int best_i[4];
  __shared__ int flags_s[4];
  const int part = blockIdx.x, row_id = blockIdx.y;
  const float* row = logits + (size_t)row_id * row_stride;
  const int per = ((vocab + ARGMAX_PARTS - 1) / ARGMAX_PARTS + 3) & ~3;     // a multiple of four: parts start aligned
  const int begin = min(vocab, part * per), end = min(vocab, begin + per);
  float bv = -INFINITY;
  int bi = 0x7fffffff, flags = 0;   // bit 0 NaN, bit 1 +inf, bit 3 a finite entry was seen
  auto take = [&](float v, int i) {
    if (v != v) flags |= 1;
    else if (v == INFINITY) flags |= 2;
    else if (v != -INFINITY) flags |= 8;
    argmax_merge(bv, bi, v, i);
  };
  int i = begin + threadIdx.x;
  if ((((uintptr_t)row) & 15) == 0) {          // four at a time, two loads in flight, in index order
    const int whole = begin + ((end - begin) & ~3);
    int at = begin + 4 * threadIdx.x;
    for (; at + 1024 < whole; at += 2048) {
      const float4 a = *(const float4*)(row + at), b = *(const float4*)(row + at + 1024);
      take(a.x, at); take(a.y, at + 1); take(a.z, at + 2); take(a.w, at + 3);
      take(b.x, at + 1024); take(b.y, at + 1025); take(b.z, at + 1026); take(b.w, at + 1027);
    }
    if (at < whole) {
      const float4 a = *(const float4*)(row + at);
      take(a.x, at); take(a.y, at + 1); take(a.z, at + 2); take(a.w, at + 3);
    }
    i = whole + threadIdx.x;                    // what is left: fewer than four entries
  }
  for (; i < end; i += 256) take(row[i], i);
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) {
    argmax_merge(bv, bi, __shfl_xor(bv, offset, FE_WAVE), __shfl_xor(bi, offset, FE_WAVE));
    flags |= __shfl_xor(flags, offset, FE_WAVE);
  }
  const int lane = threadIdx.x & (FE_WAVE - 1), wave = threadIdx.x / FE_WAVE;
  if (lane == 0) { best_v[wave] = bv; best_i[wave] = bi; flags_s[wave] = flags; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) { argmax_merge(bv, bi, best_v[w], best_i[w]); flags |= flags_s[w]; }
    part_v[row_id * ARGMAX_PARTS + part] = bv;
    part_i[row_id * ARGMAX_PARTS + part] = bi;
    part_flags[row_id * ARGMAX_PARTS + part] = flags;
  }
}

__global__ __launch_bounds__(64) void argmax_merge_kernel(
    const float* __restrict__ part_v, const int* __restrict__ part_i, const int* __restrict__ part_flags,
    int* __restrict__ tokens, int* __restrict__ status) {
  const int row_id = blockIdx.x, lane = threadIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff, flags = 0;
  if (lane < ARGMAX_PARTS) {
    bv = part_v[row_id * ARGMAX_PARTS + lane];
    bi = part_i[row_id * ARGMAX_PARTS + lane];
    flags = part_flags[row_id * ARGMAX_PARTS + lane];
  }
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) {
    argmax_merge(bv, bi, __shfl_xor(bv, offset, FE_WAVE), __shfl_xor(bi, offset, FE_WAVE));
    flags |= __shfl_xor(flags, offset, FE_WAVE);
  }
  if (lane == 0) {
    tokens[row_id] = bi == 0x7fffffff ? 0 : bi;
    status[row_id] = (flags & 3) | ((flags & 8) ? 0 : 4);
  }
}

// Philox4x32-10; returns the first output word.
__device__ __forceinline__ uint32_t philox_first_word(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                      uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

// For each row: weights w_i = exp((x_i - max) / temperature); the uniform
// u = (philox(counter = draw index, key = seed) >> 8) * 2^-24 picks the first
// token whose running sum of weights exceeds u * total.  Thread t owns the
// contiguous range [t * chunk, (t + 1) * chunk) so that the running sum follows
// the token order.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    const float* __restrict__ logits, long long row_stride, int vocab,
    const float* __restrict__ temperatures, const unsigned long long* __restrict__ seeds,
    const unsigned long long* __restrict__ draw_index, int* __restrict__ tokens,
    int* __restrict__ status) {
  __shared__ float red[SAMPLE_WAVES];
  __shared__ int flags[2];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ int chosen;
  const int row_id = blockIdx.x;
  const float* row = logits + (size_t)row_id * row_stride;
  const int st = row_status(row, vocab, red, flags);
  if (st) {  // nothing sensible to draw from; the host raises on the status
    if (threadIdx.x == 0) { tokens[row_id] = 0; status[row_id] = st; }
    return;
  }
  const float inv_t = 1.f / temperatures[row_id];
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, red);

  const int chunk = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int begin = threadIdx.x * chunk;
  const int end = min(vocab, begin + chunk);
  float local = 0.f;
  for (int i = begin; i < end; ++i) local += expf((row[i] - mx) * inv_t);
  sums[threadIdx.x] = local;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    // serial scan over 1024 partial sums: a fixed order, negligible time
    float total = 0.f;
    for (int t = 0; t < SAMPLE_THREADS; ++t) total += sums[t];
    const unsigned long long seed = seeds[row_id];
    const unsigned long long index = draw_index[row_id];
    const uint32_t word = philox_first_word((uint32_t)index, (uint32_t)(index >> 32), 0u, 0u,
                                            (uint32_t)seed, (uint32_t)(seed >> 32));
    const float u = (float)(word >> 8) * (1.0f / 16777216.0f);
    const float target = u * total;
    float running = 0.f;
    int owner = -1, last_nonzero = -1;
    for (int t = 0; t < SAMPLE_THREADS; ++t) {
      const float s = sums[t];
      if (s > 0.f) last_nonzero = t;
      if (owner < 0 && running + s > target) { owner = t; break; }
      running += s;
    }
    if (owner < 0) {  // rounding pushed the target past the total: last token with weight
      owner = last_nonzero;
      running = -1.f;  // marks "take the last nonzero entry of the range"
    }
    red[0] = running;
    red[1] = target;
    chosen = owner;
    if (owner < 0) { tokens[row_id] = 0; status[row_id] = 4; }
  }
  __syncthreads();
  if (threadIdx.x == chosen) {
    float running = red[0];
    const float target = red[1];
    int pick = -1, last = -1;
    for (int i = begin; i < end; ++i) {
      const float w = expf((row[i] - mx) * inv_t);
      if (w > 0.f) last = i;
      if (running >= 0.f) {
        running += w;
        if (running > target) { pick = i; break; }
      }
    }
    if (pick < 0) pick = last;
    tokens[row_id] = pick < 0 ? 0 : pick;
    status[row_id] = 0;
  }
}

// scratch: at least rows * 32 * 3 four-byte words (partial maxima, indices, flags).
extern "C" int fe_argmax_rows(const float* logits, long long row_stride, int rows, int vocab,
                              int* tokens, int* status, void* scratch, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (vocab <= 0 || row_stride < vocab || !scratch || rows > 65535) return FE_BAD_ARGUMENT;
  float* part_v = (float*)scratch;
  int* part_i = (int*)scratch + (size_t)rows * ARGMAX_PARTS;
  int* part_flags = part_i + (size_t)rows * ARGMAX_PARTS;
  dim3 grid(ARGMAX_PARTS, rows);
  argmax_parts_kernel<<<grid, 256, 0, stream>>>(logits, row_stride, vocab, part_v, part_i, part_flags);
  argmax_merge_kernel<<<rows, 64, 0, stream>>>(part_v, part_i, part_flags, tokens, status);
  return fe_check_launch();
}

// The scratch of fe_argmax_rows_static.  In host code this name is only a handle for
// hipGetSymbolAddress: each GPU holds its own copy at its own address, kept below per device.
static __device__ __align__(256) int argmax_static_scratch[FE_ARGMAX_STATIC_MAX_ROWS * ARGMAX_PARTS * 3];

#define FE_MAX_DEVICES 64
static std::mutex static_scratch_lock;
static void* static_scratch_of_device[FE_MAX_DEVICES];

// The device address of the array on the current device (looked up at the first call there).
static void* argmax_static_scratch_here() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= FE_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> hold(static_scratch_lock);
  if (!static_scratch_of_device[device]) {
    void* address = nullptr;
    if (hipGetSymbolAddress(&address, HIP_SYMBOL(argmax_static_scratch)) != hipSuccess) return nullptr;
    static_scratch_of_device[device] = address;
  }
  return static_scratch_of_device[device];
}

extern "C" int fe_argmax_rows_static(const float* logits, long long row_stride, int rows, int vocab,
                                     int* tokens, int* status, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (rows > FE_ARGMAX_STATIC_MAX_ROWS) return FE_BAD_ARGUMENT;
  void* scratch = argmax_static_scratch_here();
  if (!scratch) return FE_LAUNCH_FAILED;
  return fe_argmax_rows(logits, row_stride, rows, vocab, tokens, status, scratch, stream);
}

extern "C" int fe_sample_rows(const float* logits, long long row_stride, int rows, int vocab,
                              const float* temperatures, const unsigned long long* seeds,
                              const unsigned long long* draw_index, int* tokens, int* status,
                              hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (vocab <= 0 || row_stride < vocab) return FE_BAD_ARGUMENT;
  sample_rows_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, row_stride, vocab, temperatures, seeds,
                                                          draw_index, tokens, status);
  return fe_check_launch();
}
