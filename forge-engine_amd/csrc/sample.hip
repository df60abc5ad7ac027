// Sampling over float32 logits rows: argmax, and a draw from softmax(logits / temperature)
// after top-k, top-p and min-p by inverse CDF with a counter-based generator, one block of
// 1024 threads per row.  Each row also gets a status word:
//   bit 0: a NaN was seen, bit 1: +inf was seen, bit 2: no finite entry.
#include "common.h"
#include "sample_api.h"
#include <mutex>

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / FE_WAVE)

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

// ---------------------------------------------------------------------------------------------
// One launch for rows that each bring parameters of their own: arg-max (temperature 0), or a draw
// from softmax(logits / temperature) after top-k, top-p and min-p, in that order, each a threshold
// on the logit: with f_i = (x_i - max) / temperature (so the largest is 0) and e_i = exp(f_i),
//   top-k  keeps the k largest f (all of those equal to the k-th),
//   top-p  keeps a token if the e of all larger tokens, over the e of the top-k set, is <= top_p,
//   min-p  keeps a token if e_i >= min_p (its probability over the largest one's),
// and the draw takes the first kept token, in token order, whose running sum of e exceeds u times
// the total, u = (philox(counter = draw index, key = seed) >> 8) * 2^-24.
//
// Sums of e are sums of integers, e_i * 2^40 cut to 64 bits: they do not depend on the order of
// the additions, so histograms by atomic adds and reductions of any shape give the same bits in
// every run, and the place where a running sum crosses its target is exact.  A token whose e is
// below 2^-40 of the largest one's weighs nothing.
//
// Thresholds are found in the space of keys: y_i = -f_i >= 0, key = the bits of y (the order of
// non-negative floats is the order of their bits; -inf logits give y = +inf, the largest key).
// A histogram of 2,048 bins (first linear in y up to 32, then an even split of the chosen bin's
// range of keys, until the range is one key) holds counts for top-k or masses for top-p; a scan
// over the bins finds the bin in which the count reaches k or the mass passes top_p * total.
// One block of 1,024 threads a row; wave w reads the w-th sixteenth of the row, 256 entries a trip.
struct SampleRowParams {
  float temperature;           // 0: arg-max
  int top_k;                   // 0: no limit
  float top_p;                 // >= 1: no limit
  float min_p;                 // 0: no limit
  unsigned long long seed;
  unsigned long long draw_index;
};
static_assert(sizeof(SampleRowParams) == FE_SAMPLE_PARAM_WORDS * 4, "the host packs eight words a row");

#define FILTER_BINS 2048
#define WEIGHT_SCALE 1099511627776.0f      // 2^40
#define KEY_END 0x7f800001u                // one past the key of +inf

struct FilterShared {
  unsigned long long mass[FILTER_BINS];
  unsigned int count[FILTER_BINS];
  unsigned long long wave_sum[SAMPLE_WAVES];
  float wave_best[SAMPLE_WAVES];
  int wave_arg[SAMPLE_WAVES];
  int wave_flags[SAMPLE_WAVES];
  unsigned long long found_before;
  unsigned long long target;
  int found_bin;
  int pick_wave;
};

// f(index, value) for every entry of the row that this thread owns: wave w owns
// [w * segment, (w + 1) * segment), a trip takes 256 entries, a lane four neighbours.
template <class F>
__device__ __forceinline__ void visit_row(const float* __restrict__ row, int vocab, int segment, F f) {
  const int lane = threadIdx.x & (FE_WAVE - 1), wave = threadIdx.x / FE_WAVE;
  const int begin = wave * segment;
  const int end = min(vocab, begin + segment);
  const bool aligned = (((uintptr_t)row) & 15) == 0;
  for (int at = begin + 4 * lane; at < end; at += 256) {
    if (aligned && at + 3 < end) {
      const float4 v = *(const float4*)(row + at);
      f(at, v.x); f(at + 1, v.y); f(at + 2, v.z); f(at + 3, v.w);
    } else {
      for (int c = 0; c < 4 && at + c < end; ++c) f(at + c, row[at + c]);
    }
  }
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, FE_WAVE);
  return v;
}

// Every thread gets the block's total (two barriers).
__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, FilterShared& sh) {
  v = wave_sum_u64(v);
  __syncthreads();
  if ((threadIdx.x & (FE_WAVE - 1)) == 0) sh.wave_sum[threadIdx.x / FE_WAVE] = v;
  __syncthreads();
  unsigned long long total = 0;
  for (int w = 0; w < SAMPLE_WAVES; ++w) total += sh.wave_sum[w];
  return total;
}

__device__ __forceinline__ unsigned long long weight_of(float y) {
  return (unsigned long long)(expf(-y) * WEIGHT_SCALE);
}

__device__ __forceinline__ int first_bin(float y) { return (int)fminf(y * 64.f, (float)(FILTER_BINS - 1)); }

// The bin in which the running total over the bins, in order, reaches the target: by counts the
// bin with before < target <= before + own, by masses the bin with before <= target < before + own.
// Leaves the bin in sh.found_bin (-1 if there is none) and the total before it in sh.found_before.
template <bool BY_MASS>
__device__ __forceinline__ void find_crossing(FilterShared& sh, unsigned long long target) {
  const int t = threadIdx.x, lane = t & (FE_WAVE - 1), wave = t / FE_WAVE;
  const unsigned long long a0 = BY_MASS ? sh.mass[2 * t] : sh.count[2 * t];
  const unsigned long long a1 = BY_MASS ? sh.mass[2 * t + 1] : sh.count[2 * t + 1];
  const unsigned long long own = a0 + a1;
  unsigned long long upto = own;
#pragma unroll
  for (int offset = 1; offset < FE_WAVE; offset <<= 1) {
    const unsigned long long other = __shfl_up(upto, offset, FE_WAVE);
    if (lane >= offset) upto += other;
  }
  __syncthreads();                       // whoever still reads what the call before left has done so
  if (lane == FE_WAVE - 1) sh.wave_sum[wave] = upto;
  if (t == 0) sh.found_bin = -1;
  __syncthreads();
  unsigned long long before = upto - own;
  for (int w = 0; w < wave; ++w) before += sh.wave_sum[w];
  const unsigned long long before1 = before + a0;
  const bool hit0 = BY_MASS ? (before <= target && target < before + a0) : (before < target && target <= before + a0);
  const bool hit1 = BY_MASS ? (before1 <= target && target < before1 + a1) : (before1 < target && target <= before1 + a1);
  if (hit0) { sh.found_bin = 2 * t; sh.found_before = before; }
  else if (hit1) { sh.found_bin = 2 * t + 1; sh.found_before = before1; }
  __syncthreads();
}

// The key at which the running count (top-k) or mass (top-p) over the keys, in order, reaches the
// target, given the first histogram (already in sh) and the target.
template <bool BY_MASS>
__device__ __forceinline__ unsigned int find_key(const float* __restrict__ row, int vocab, int segment, float mx,
                                                 float inv_t, unsigned long long target, FilterShared& sh) {
  find_crossing<BY_MASS>(sh, target);
  int bin = sh.found_bin;
  if (bin < 0) return KEY_END - 1;              // cannot happen (the target lies below the total); keeps everything
  target -= sh.found_before;
  unsigned int lo = __float_as_uint((float)bin * (1.f / 64.f));
  unsigned int hi = bin == FILTER_BINS - 1 ? KEY_END : __float_as_uint((float)(bin + 1) * (1.f / 64.f));
  while (hi - lo > 1) {
    const unsigned int span = hi - lo;
    const int shift = span <= FILTER_BINS ? 0 : 32 - __clz((span - 1) >> 11);    // (span - 1) >> shift < 2048
    __syncthreads();
    for (int i = threadIdx.x; i < FILTER_BINS; i += SAMPLE_THREADS) {
      if (BY_MASS) sh.mass[i] = 0; else sh.count[i] = 0;
    }
    __syncthreads();
    visit_row(row, vocab, segment, [&](int, float v) {
      const float y = (mx - v) * inv_t;
      const unsigned int key = __float_as_uint(y);
      if (key >= lo && key < hi) {
        const unsigned int sub = (key - lo) >> shift;
        if (BY_MASS) atomicAdd(&sh.mass[sub], weight_of(y)); else atomicAdd(&sh.count[sub], 1u);
      }
    });
    __syncthreads();
    find_crossing<BY_MASS>(sh, target);
    bin = sh.found_bin;
    if (bin < 0) return hi - 1;
    target -= sh.found_before;
    lo += (unsigned int)bin << shift;
    hi = min(hi, lo + (1u << shift));
  }
  return lo;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_filtered_rows_kernel(
    const float* __restrict__ logits, long long row_stride, int vocab, const SampleRowParams* __restrict__ params,
    int* __restrict__ tokens, int* __restrict__ status) {
  __shared__ FilterShared sh;
  const int row_id = blockIdx.x;
  const float* row = logits + (size_t)row_id * row_stride;
  const int lane = threadIdx.x & (FE_WAVE - 1), wave = threadIdx.x / FE_WAVE;
  const int segment = (vocab + SAMPLE_WAVES * 256 - 1) / (SAMPLE_WAVES * 256) * 256;
  const SampleRowParams p = params[row_id];

  // the largest entry (lowest index among equals) and what the guards look for
  float bv = -INFINITY;
  int bi = 0x7fffffff, flags = 0;
  visit_row(row, vocab, segment, [&](int i, float v) {
    if (v != v) flags |= 1;
    else if (v == INFINITY) flags |= 2;
    else if (v != -INFINITY) flags |= 8;
    argmax_merge(bv, bi, v, i);
  });
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) {
    argmax_merge(bv, bi, __shfl_xor(bv, offset, FE_WAVE), __shfl_xor(bi, offset, FE_WAVE));
    flags |= __shfl_xor(flags, offset, FE_WAVE);
  }
  if (lane == 0) { sh.wave_best[wave] = bv; sh.wave_arg[wave] = bi; sh.wave_flags[wave] = flags; }
  __syncthreads();
  bv = sh.wave_best[0]; bi = sh.wave_arg[0]; flags = sh.wave_flags[0];
  for (int w = 1; w < SAMPLE_WAVES; ++w) { argmax_merge(bv, bi, sh.wave_best[w], sh.wave_arg[w]); flags |= sh.wave_flags[w]; }
  const int st = (flags & 3) | ((flags & 8) ? 0 : 4);
  if (st || !(p.temperature > 0.f)) {     // nothing sensible to draw from (the host raises on the status), or arg-max
    if (threadIdx.x == 0) { tokens[row_id] = st || bi == 0x7fffffff ? 0 : bi; status[row_id] = st; }
    return;
  }
  const float mx = bv, inv_t = 1.f / p.temperature;

  unsigned int key_limit = KEY_END - 1;       // keys up to this one stay
  if (p.top_k > 0 && p.top_k < vocab) {
    for (int i = threadIdx.x; i < FILTER_BINS; i += SAMPLE_THREADS) sh.count[i] = 0;
    __syncthreads();
    visit_row(row, vocab, segment, [&](int, float v) { atomicAdd(&sh.count[first_bin((mx - v) * inv_t)], 1u); });
    __syncthreads();
    key_limit = find_key<false>(row, vocab, segment, mx, inv_t, (unsigned long long)p.top_k, sh);
  }
  if (p.top_p < 1.f) {
    __syncthreads();
    for (int i = threadIdx.x; i < FILTER_BINS; i += SAMPLE_THREADS) sh.mass[i] = 0;
    __syncthreads();
    unsigned long long within = 0;          // the mass of what top-k left
    visit_row(row, vocab, segment, [&](int, float v) {
      const float y = (mx - v) * inv_t;
      const unsigned long long w = weight_of(y);
      atomicAdd(&sh.mass[first_bin(y)], w);
      if (__float_as_uint(y) <= key_limit) within += w;
    });
    within = block_sum_u64(within, sh);     // its barriers also end the histogram
    const unsigned long long target = (unsigned long long)((double)within * (double)p.top_p);
    // what lies past top-k comes after every key that top-k keeps and cannot move the crossing
    key_limit = min(key_limit, find_key<true>(row, vocab, segment, mx, inv_t, target, sh));
  }

  // the draw: totals of the kept weights per wave, the wave in which the running sum passes the
  // target, then that wave walks its part of the row again
  const float min_e = p.min_p;
  auto kept_weight = [&](float v) -> unsigned long long {
    const float y = (mx - v) * inv_t;
    if (__float_as_uint(y) > key_limit) return 0ull;
    const float e = expf(-y);
    return e >= min_e ? (unsigned long long)(e * WEIGHT_SCALE) : 0ull;
  };
  unsigned long long mine = 0;
  visit_row(row, vocab, segment, [&](int, float v) { mine += kept_weight(v); });
  mine = wave_sum_u64(mine);
  __syncthreads();
  if (lane == 0) sh.wave_sum[wave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long total = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) total += sh.wave_sum[w];
    const uint32_t word = philox_first_word((uint32_t)p.draw_index, (uint32_t)(p.draw_index >> 32), 0u, 0u,
                                            (uint32_t)p.seed, (uint32_t)(p.seed >> 32));
    const unsigned long long u24 = word >> 8;
    // floor(total * u24 / 2^24) from the 128-bit product
    const unsigned long long target = (__umul64hi(total, u24) << 40) | ((total * u24) >> 24);
    unsigned long long before = 0;
    int w = 0;
    while (w < SAMPLE_WAVES - 1 && before + sh.wave_sum[w] <= target) before += sh.wave_sum[w++];
    sh.pick_wave = w;
    sh.found_before = before;
    sh.target = target;
  }
  __syncthreads();
  if (wave != sh.pick_wave) return;
  unsigned long long before = sh.found_before;
  const unsigned long long target = sh.target;
  const int begin = wave * segment, end = min(vocab, begin + segment);
  for (int base = begin; base < end; base += 256) {       // the same order as visit_row's
    const int at = base + 4 * lane;
    unsigned long long w4[4];
    unsigned long long own = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) { w4[c] = at + c < end ? kept_weight(row[at + c]) : 0ull; own += w4[c]; }
    unsigned long long upto = own;
#pragma unroll
    for (int offset = 1; offset < FE_WAVE; offset <<= 1) {
      const unsigned long long other = __shfl_up(upto, offset, FE_WAVE);
      if (lane >= offset) upto += other;
    }
    const unsigned long long trip = __shfl(upto, FE_WAVE - 1, FE_WAVE);
    if (before + trip > target) {
      const unsigned long long hits = __ballot(before + upto > target);
      if (lane == __ffsll((long long)hits) - 1) {
        unsigned long long running = before + upto - own;
        int pick = at;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          running += w4[c];
          if (running > target) { pick = at + c; break; }
        }
        tokens[row_id] = pick;
        status[row_id] = 0;
      }
      return;
    }
    before += trip;
  }
  if (lane == 0) { tokens[row_id] = bi; status[row_id] = 0; }    // cannot happen: the target lies below the total
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

extern "C" int fe_sample_filtered_rows(const float* logits, long long row_stride, int rows, int vocab,
                                       const void* params, int* tokens, int* status, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (vocab <= 0 || row_stride < vocab || !params || (((uintptr_t)params) & 7)) return FE_BAD_ARGUMENT;
  sample_filtered_rows_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, row_stride, vocab,
                                                                   (const SampleRowParams*)params, tokens, status);
  return fe_check_launch();
}
