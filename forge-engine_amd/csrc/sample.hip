// Sampling over float32 logits rows: argmax, and a draw from softmax(logits / temperature)
// after top-k, top-p and min-p by inverse CDF with a counter-based generator; a row is shared
// by several blocks.  Each row also gets a status word:
//   bit 0: a NaN was seen, bit 1: +inf was seen, bit 2: no finite entry.
#include "common.h"
#include "sample_api.h"
#include <mutex>

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
// Rows that each bring parameters of their own: arg-max (temperature 0), or a draw from
// softmax(logits / temperature) after top-k, top-p and min-p, in that order, each a threshold on
// the logit: with f_i = (x_i - max) / temperature (so the largest is 0) and e_i = exp(f_i),
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
// range of keys) holds counts for top-k, masses and counts for top-p; a scan over the bins finds
// the bin in which the count reaches k or the mass passes top_p * total, and the search ends when
// the bin is one key wide or all of it stays (the count reaches k at its end, or it holds one
// entry).
//
// One CU would need 25 us for one pass over a row of 150,000 entries (the exponentials), so a
// row is cut into `split` slices with a block each, and every pass is a launch of its own: what
// a pass leaves (partial maxima and sums, the histogram, a header with the state of the row's
// search) lies in the row's scratch, and every block of the next launch works out the same next
// state from it before it does that state's pass over its slice.  A row goes through
//   the maximum; [top-k: first histogram, refinements]; [top-p: first histogram, refinements];
//   the sums of what stays; the pick
// and rows that are through do nothing in the launches that are left (the host launches what the
// longest search can need: 3 + 4 for top-k + 4 for top-p).
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
#define PHASE_THREADS 256
#define PHASE_WAVES (PHASE_THREADS / FE_WAVE)
#define BINS_PER_THREAD (FILTER_BINS / PHASE_THREADS)

enum : int { PH_MAX = 0, PH_COUNT_FIRST, PH_COUNT_REFINE, PH_MASS_FIRST, PH_MASS_REFINE, PH_DRAW_SUM, PH_DRAW_PICK, PH_DONE };

struct RowHeader {                 // what the launch before did for the row, and where its search stands
  int phase;
  int shift;                       // a refinement's bins are (key - lo) >> shift
  unsigned int lo, hi;             // the keys [lo, hi) that the histogram of that launch splits
  unsigned int key_limit;          // keys up to this one stay (from the searches that are finished)
  int owner;                       // the pick: the slice in which the running sum passes the target (a row that ends at its maximum: its status)
  unsigned long long target;       // the count or mass to reach within [lo, hi); the pick's target
  unsigned long long before;       // the pick: the sum of the slices before the owner
  float mx;
  int arg;
};

struct RowScratch {
  RowHeader header[2];             // written by launch n into [n & 1], read by launch n + 1
  float part_best[FE_SAMPLE_MAX_SPLIT];
  int part_arg[FE_SAMPLE_MAX_SPLIT];
  int part_flags[FE_SAMPLE_MAX_SPLIT];
  unsigned long long part_within[FE_SAMPLE_MAX_SPLIT];  // per slice: the mass of what top-k left
  unsigned long long part_sum[FE_SAMPLE_MAX_SPLIT];     // per slice: the mass of what stays (another array: a launch
                                                        // that writes these may still have blocks reading those)
  unsigned long long mass[3][FILTER_BINS];              // launch n adds into [n % 3], reads [(n - 1) % 3], clears [(n + 1) % 3]
  unsigned int count[3][FILTER_BINS];
};
static_assert(sizeof(RowScratch) <= FE_SAMPLE_SCRATCH_BYTES_PER_ROW, "the header states the scratch a row needs");

struct PhaseShared {
  unsigned long long mass[FILTER_BINS];
  unsigned int count[FILTER_BINS];
  unsigned long long wave_sum[PHASE_WAVES];
  float wave_best[PHASE_WAVES];
  int wave_arg[PHASE_WAVES];
  int wave_flags[PHASE_WAVES];
  unsigned long long found_before, found_own;
  unsigned int found_count;
  int found_bin;
};

// f(index, value) for every entry of the thread's own run [begin, end) of the row, in order; begin is
// a multiple of four.  Eight loads of four entries are in flight before the first is used (none
// of them under a condition: a load past the run reads the row's last whole four again and is
// not used), so a run costs one or two trips to memory, not one per load.
template <class F>
__device__ __forceinline__ void visit(const float* __restrict__ row, int vocab, int begin, int end, F f) {
  if ((((uintptr_t)row) & 15) != 0 || vocab < 4) {       // rows that do not start on 16 bytes: entry by entry
    for (int i = begin; i < end; ++i) f(i, row[i]);
    return;
  }
  const int last_four = (vocab - 4) & ~3;                // the last place a whole four can be read from
  const int whole_end = end & ~3;                        // end is a multiple of four unless it is the row's end
  for (int at = begin; at < whole_end; at += 32) {
    float4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *(const float4*)(row + min(at + 4 * j, last_four));
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = at + 4 * j;
      if (i < whole_end) { f(i, v[j].x); f(i + 1, v[j].y); f(i + 2, v[j].z); f(i + 3, v[j].w); }
    }
  }
  for (int i = max(begin, whole_end); i < end; ++i) f(i, row[i]);
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
  for (int offset = FE_WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, FE_WAVE);
  return v;
}

// Every thread gets the block's total (two barriers).
__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, PhaseShared& sh) {
  v = wave_sum_u64(v);
  __syncthreads();
  if ((threadIdx.x & (FE_WAVE - 1)) == 0) sh.wave_sum[threadIdx.x / FE_WAVE] = v;
  __syncthreads();
  unsigned long long total = 0;
  for (int w = 0; w < PHASE_WAVES; ++w) total += sh.wave_sum[w];
  return total;
}

__device__ __forceinline__ int first_bin(float y) { return (int)fminf(y * 64.f, (float)(FILTER_BINS - 1)); }

// The bin in which the running total over the bins of a histogram in global memory, in order,
// reaches the target: by counts the bin with before < target <= before + own, by masses the bin
// with before <= target < before + own.  Leaves the bin in sh.found_bin (-1 if there is none),
// the total before it, its own total and its count.
template <bool BY_MASS>
__device__ __forceinline__ void find_crossing(const unsigned long long* __restrict__ mass,
                                              const unsigned int* __restrict__ count, unsigned long long target,
                                              PhaseShared& sh) {
  const int t = threadIdx.x, lane = t & (FE_WAVE - 1), wave = t / FE_WAVE;
  unsigned long long a[BINS_PER_THREAD];
  unsigned int c[BINS_PER_THREAD];
  unsigned long long own = 0;
#pragma unroll
  for (int i = 0; i < BINS_PER_THREAD; ++i) {
    c[i] = count[t * BINS_PER_THREAD + i];
    a[i] = BY_MASS ? mass[t * BINS_PER_THREAD + i] : (unsigned long long)c[i];
    own += a[i];
  }
  unsigned long long upto = own;
#pragma unroll
  for (int offset = 1; offset < FE_WAVE; offset <<= 1) {
    const unsigned long long other = __shfl_up(upto, offset, FE_WAVE);
    if (lane >= offset) upto += other;
  }
  __syncthreads();                       // whoever still reads what an earlier use of sh left has done so
  if (lane == FE_WAVE - 1) sh.wave_sum[wave] = upto;
  if (t == 0) sh.found_bin = -1;
  __syncthreads();
  unsigned long long before = upto - own;
  for (int w = 0; w < wave; ++w) before += sh.wave_sum[w];
#pragma unroll
  for (int i = 0; i < BINS_PER_THREAD; ++i) {
    const bool hit = BY_MASS ? (before <= target && target < before + a[i]) : (before < target && target <= before + a[i]);
    if (hit) {
      sh.found_bin = t * BINS_PER_THREAD + i;
      sh.found_before = before;
      sh.found_own = a[i];
      sh.found_count = c[i];
    }
    before += a[i];
  }
  __syncthreads();
}

// After a histogram's crossing bin is known: the keys of that bin become the range to split next,
// or the search ends (its limit is then the bin's last key).  Returns whether it has ended.
__device__ __forceinline__ bool narrow(RowHeader& h, bool first, bool by_mass, const PhaseShared& sh) {
  const int bin = sh.found_bin;
  if (bin < 0) {                  // cannot happen (the target lies below the total); keeps the whole range
    h.lo = h.hi - 1;
    return true;
  }
  if (first) {
    h.lo = __float_as_uint((float)bin * (1.f / 64.f));
    h.hi = bin == FILTER_BINS - 1 ? KEY_END : __float_as_uint((float)(bin + 1) * (1.f / 64.f));
  } else {
    h.lo += (unsigned int)bin << h.shift;
    h.hi = min(h.hi, h.lo + (1u << h.shift));
  }
  h.target -= sh.found_before;
  const unsigned int span = h.hi - h.lo;
  // all of the bin stays: the count reaches k at its end, or a single entry holds the crossing
  const bool whole = by_mass ? sh.found_count == 1 : h.target == sh.found_own;
  if (span <= 1 || whole) return true;
  h.shift = span <= FILTER_BINS ? 0 : 32 - __clz((int)((span - 1) >> 11));      // (span - 1) >> shift < 2048
  return false;
}

__global__ __launch_bounds__(PHASE_THREADS) void sample_phase_kernel(
    const float* __restrict__ logits, long long row_stride, int vocab, const SampleRowParams* __restrict__ params,
    RowScratch* __restrict__ scratch, int split, int launch, int* __restrict__ tokens, int* __restrict__ status) {
  __shared__ PhaseShared sh;
  const int row_id = blockIdx.y, slice_id = blockIdx.x;
  const float* row = logits + (size_t)row_id * row_stride;
  RowScratch& rs = scratch[row_id];
  const int t = threadIdx.x, lane = t & (FE_WAVE - 1), wave = t / FE_WAVE;
  const SampleRowParams p = params[row_id];
  // a slice: a multiple of 1,024 entries, of which every thread owns a run of neighbours (a multiple of four)
  const int slice = (vocab + split * 1024 - 1) / (split * 1024) * 1024;
  const int begin = min(vocab, slice_id * slice + t * (slice / PHASE_THREADS));
  const int end = min(vocab, begin + slice / PHASE_THREADS);
  const int write_to = launch % 3, read_from = (launch + 2) % 3, clear = (launch + 1) % 3;
  for (int i = slice_id * PHASE_THREADS + t; i < FILTER_BINS; i += split * PHASE_THREADS) {
    rs.mass[clear][i] = 0;
    rs.count[clear][i] = 0;
  }

  if (launch == 0) {      // the largest entry (lowest index among equals) and what the guards look for
    float bv = -INFINITY;
    int bi = 0x7fffffff, flags = 0;
    visit(row, vocab, begin, end, [&](int i, float v) {
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
    if (t == 0) {
      for (int w = 1; w < PHASE_WAVES; ++w) { argmax_merge(bv, bi, sh.wave_best[w], sh.wave_arg[w]); flags |= sh.wave_flags[w]; }
      rs.part_best[slice_id] = bv; rs.part_arg[slice_id] = bi; rs.part_flags[slice_id] = flags;
      if (slice_id == 0) {
        RowHeader h = {};
        h.phase = PH_MAX;
        rs.header[0] = h;
        status[row_id] = 8;      // not through yet; the row's last pass writes the status
      }
    }
    return;
  }

  // from what the launch before left, the state of the row now: the same in every block of the row
  RowHeader h = rs.header[(launch - 1) & 1];
  const bool has_k = p.top_k > 0 && p.top_k < vocab, has_p = p.top_p < 1.f;
  bool done_row = false;       // this launch writes the row's token (its slice 0 does)
  switch (h.phase) {
    case PH_MAX: {
      float bv = rs.part_best[0];
      int bi = rs.part_arg[0], flags = rs.part_flags[0];
      for (int s = 1; s < split; ++s) { argmax_merge(bv, bi, rs.part_best[s], rs.part_arg[s]); flags |= rs.part_flags[s]; }
      const int st = (flags & 3) | ((flags & 8) ? 0 : 4);
      h.mx = bv;
      h.arg = st || bi == 0x7fffffff ? 0 : bi;
      h.key_limit = KEY_END - 1;
      if (st || !(p.temperature > 0.f)) {     // nothing sensible to draw from (the host raises on the status), or arg-max
        h.phase = PH_DONE;
        h.owner = st;
        done_row = true;
      } else if (has_k) {
        h.phase = PH_COUNT_FIRST;
        h.target = (unsigned long long)p.top_k;
      } else {
        h.phase = has_p ? PH_MASS_FIRST : PH_DRAW_SUM;
      }
      break;
    }
    case PH_COUNT_FIRST:
    case PH_COUNT_REFINE: {
      find_crossing<false>(rs.mass[read_from], rs.count[read_from], h.target, sh);
      if (narrow(h, h.phase == PH_COUNT_FIRST, false, sh)) {
        h.key_limit = h.hi - 1;
        h.phase = has_p ? PH_MASS_FIRST : PH_DRAW_SUM;
      } else {
        h.phase = PH_COUNT_REFINE;
      }
      break;
    }
    case PH_MASS_FIRST:
    case PH_MASS_REFINE: {
      if (h.phase == PH_MASS_FIRST) {
        unsigned long long within = 0;        // the mass of what top-k left
        for (int s = 0; s < split; ++s) within += rs.part_within[s];
        h.target = (unsigned long long)((double)within * (double)p.top_p);
      }
      // what lies past top-k comes after every key that top-k keeps and cannot move the crossing
      find_crossing<true>(rs.mass[read_from], rs.count[read_from], h.target, sh);
      if (narrow(h, h.phase == PH_MASS_FIRST, true, sh)) {
        h.key_limit = min(h.key_limit, h.hi - 1);
        h.phase = PH_DRAW_SUM;
      } else {
        h.phase = PH_MASS_REFINE;
      }
      break;
    }
    case PH_DRAW_SUM: {
      unsigned long long total = 0;
      for (int s = 0; s < split; ++s) total += rs.part_sum[s];
      const uint32_t word = philox_first_word((uint32_t)p.draw_index, (uint32_t)(p.draw_index >> 32), 0u, 0u,
                                              (uint32_t)p.seed, (uint32_t)(p.seed >> 32));
      const unsigned long long u24 = word >> 8;
      // floor(total * u24 / 2^24) from the 128-bit product
      h.target = (__umul64hi(total, u24) << 40) | ((total * u24) >> 24);
      unsigned long long before = 0;
      int s = 0;
      while (s < split - 1 && before + rs.part_sum[s] <= h.target) before += rs.part_sum[s++];
      h.owner = s;
      h.before = before;
      h.phase = PH_DRAW_PICK;
      break;
    }
    default:
      h.phase = PH_DONE;
      if (slice_id == 0 && t == 0) rs.header[launch & 1] = h;
      return;
  }
  if (slice_id == 0 && t == 0) {
    rs.header[launch & 1] = h;
    if (done_row) { tokens[row_id] = h.arg; status[row_id] = h.owner; }
  }
  if (h.phase == PH_DONE) return;

  const float mx = h.mx, inv_t = 1.f / p.temperature;
  if (h.phase == PH_COUNT_FIRST || h.phase == PH_COUNT_REFINE || h.phase == PH_MASS_FIRST || h.phase == PH_MASS_REFINE) {
    const bool by_mass = h.phase == PH_MASS_FIRST || h.phase == PH_MASS_REFINE;
    const bool first = h.phase == PH_COUNT_FIRST || h.phase == PH_MASS_FIRST;
    for (int i = t; i < FILTER_BINS; i += PHASE_THREADS) { sh.mass[i] = 0; sh.count[i] = 0; }
    __syncthreads();
    unsigned long long within = 0;
    const unsigned int lo = h.lo, hi = h.hi, key_limit = h.key_limit;
    const int shift = h.shift;
    visit(row, vocab, begin, end, [&](int, float v) {
      const float y = (mx - v) * inv_t;
      const unsigned int key = __float_as_uint(y);
      int bin;
      if (first) bin = first_bin(y);
      else if (key >= lo && key < hi) bin = (int)((key - lo) >> shift);
      else return;
      atomicAdd(&sh.count[bin], 1u);
      if (by_mass) {
        const unsigned long long w = (unsigned long long)(expf(-y) * WEIGHT_SCALE);
        atomicAdd(&sh.mass[bin], w);
        if (key <= key_limit) within += w;
      }
    });
    if (h.phase == PH_MASS_FIRST) {
      within = block_sum_u64(within, sh);
      if (t == 0) rs.part_within[slice_id] = within;
    }
    __syncthreads();
    for (int i = t; i < FILTER_BINS; i += PHASE_THREADS) {
      const unsigned int c = sh.count[i];
      if (c) {
        atomicAdd(&rs.count[write_to][i], c);
        if (by_mass) atomicAdd(&rs.mass[write_to][i], sh.mass[i]);
      }
    }
    return;
  }

  // the draw: the sums of the kept weights per slice, then the slice in which the running sum
  // passes the target walks its entries again
  const float min_e = p.min_p;
  const unsigned int key_limit = h.key_limit;
  auto kept_weight = [&](float v) -> unsigned long long {
    const float y = (mx - v) * inv_t;
    if (__float_as_uint(y) > key_limit) return 0ull;
    const float e = expf(-y);
    return e >= min_e ? (unsigned long long)(e * WEIGHT_SCALE) : 0ull;
  };
  if (h.phase == PH_DRAW_SUM) {
    unsigned long long mine = 0;
    visit(row, vocab, begin, end, [&](int, float v) { mine += kept_weight(v); });
    mine = block_sum_u64(mine, sh);
    if (t == 0) rs.part_sum[slice_id] = mine;
    return;
  }
  // PH_DRAW_PICK: the thread in whose run the running sum passes the target walks its run again
  if (slice_id != h.owner) return;
  unsigned long long mine = 0;
  visit(row, vocab, begin, end, [&](int, float v) { mine += kept_weight(v); });
  unsigned long long upto = mine;
#pragma unroll
  for (int offset = 1; offset < FE_WAVE; offset <<= 1) {
    const unsigned long long other = __shfl_up(upto, offset, FE_WAVE);
    if (lane >= offset) upto += other;
  }
  if (lane == FE_WAVE - 1) sh.wave_sum[wave] = upto;
  if (t == 0) sh.found_bin = -1;
  __syncthreads();
  unsigned long long before = h.before + upto - mine;
  for (int w = 0; w < wave; ++w) before += sh.wave_sum[w];
  const unsigned long long target = h.target;
  if (before <= target && target < before + mine) {
    unsigned long long running = before;
    int pick = -1;
    visit(row, vocab, begin, end, [&](int i, float v) {
      running += kept_weight(v);
      if (pick < 0 && running > target) pick = i;
    });
    sh.found_bin = pick;
    tokens[row_id] = pick < 0 ? h.arg : pick;
    status[row_id] = 0;
  }
  __syncthreads();
  if (t == 0 && sh.found_bin < 0) { tokens[row_id] = h.arg; status[row_id] = 0; }    // cannot happen: the target lies below the total
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
                                       const void* params, int* tokens, int* status, void* scratch, int split,
                                       int launches, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (vocab <= 0 || row_stride < vocab || !params || (((uintptr_t)params) & 7) || !scratch || (((uintptr_t)scratch) & 7))
    return FE_BAD_ARGUMENT;
  if (split < 1 || split > FE_SAMPLE_MAX_SPLIT || launches < 3 || launches > 16 || rows > 65535) return FE_BAD_ARGUMENT;
  const dim3 grid(split, rows);
  for (int launch = 0; launch < launches; ++launch)
    sample_phase_kernel<<<grid, PHASE_THREADS, 0, stream>>>(logits, row_stride, vocab, (const SampleRowParams*)params,
                                                            (RowScratch*)scratch, split, launch, tokens, status);
  return fe_check_launch();
}
