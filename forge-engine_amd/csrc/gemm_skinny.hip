// bfloat16 matrix product for few rows (decode): y[M, N] = x[M, K] * W[N, K]^T,
// M <= 64, float32 accumulation on the matrix cores.  The weight is streamed
// from HBM exactly once and never staged: every weight element is used by one
// wave only, so it goes from global memory straight into the MFMA operand
// registers.  x is small and stays in the L2 cache; each wave reads the part
// it needs straight into the other operand.
//
// Work split: one block per 16, 32 or 64 weight rows (for the gated feed-forward:
// gate rows and the up rows that go with them); every wave of the block covers
// all of the block's rows, so one read of x serves them all.  The waves split K among
// themselves in interleaved 128-wide steps, so that a launch has a few thousand
// waves with all their loads in flight at once, which is what a product of a
// few microseconds needs.  The waves' float32 partial sums meet in LDS and are
// added in wave order: no global scratch, no atomics, and a result that does
// not depend on timing or on the rows beside it.
//
// MFMA 16x16x32 bf16 layout used here (A = x, B = W^T, D = A*B):
//   lane l supplies A[m = l % 16][k = 8*(l / 16) .. +8] and B[k = 8*(l / 16) .. +8][n = l % 16]
//   and receives D[m = 4*(l / 16) + i][n = l % 16], i < 4.
//
// Epilogues: store float32, store bfloat16, or silu(gate) * up -> bfloat16.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define KSTEP 128   // k per wave step: 4 lane groups x 32
#define ROWS 16     // weight rows per block and tile

#define EPI_F32 0
#define EPI_BF16 1
#define EPI_SWIGLU 2

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.f + __expf(-g)) * u; }

template <int MT, int NW>
struct StepRegs {
  uintx4 w[NW][4];
  uintx4 x[MT][4];
};

// NT row tiles per wave (for the gated product: NT gate tiles and their NT up
// tiles), WAVES waves per block sharing K.
template <int MT, int NT, int EPI, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out_base, int M, int N,
    int K, long long ldw, long long ldo, int second_offset, int steps_per_split, long long part_stride) {
  constexpr int NW = EPI == EPI_SWIGLU ? 2 * NT : NT;   // weight tiles per wave
  // blockIdx.y: which part of K this block sums (float32 epilogue only); its sums go to a part of their own
  void* out = EPI == EPI_F32 ? (void*)((float*)out_base + (size_t)blockIdx.y * part_stride) : out_base;
  __shared__ __attribute__((aligned(16))) float red[WAVES][64][4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int lr = lane & 15;
  const int lq = lane >> 4;
  const int base = blockIdx.x * (ROWS * NT);

  const bf16_t* wrow[NW];
  bool row_ok[NW];
#pragma unroll
  for (int t = 0; t < NW; ++t) {
    const int local = base + (t % NT) * ROWS + lr;   // row within [0, N)
    row_ok[t] = local < N;
    wrow[t] = w + (size_t)(row_ok[t] ? local + (t / NT) * second_offset : 0) * ldw;
  }
  const bf16_t* xrow[MT];
  bool x_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    x_ok[mt] = mt * 16 + lr < M;
    xrow[mt] = x + (size_t)(x_ok[mt] ? mt * 16 + lr : 0) * K;
  }

  floatx4 acc[MT][NW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NW; ++t) acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // One step = 128 k = four MFMAs; in MFMA c lane group lq holds k = 32*c + 8*lq .. +8 of
  // both operands, so one load instruction reads 64 contiguous bytes of each of 16 rows.
  // Every load is unconditional: rows beyond M or N read row 0 again (their sums are never
  // stored) and k beyond K reads the row's start (x is set to zero there where it is used, in
  // the one step that can reach beyond K).  A load under a per-lane condition becomes a branch,
  // and where branches meet the compiler waits for every load in flight.
  auto load = [&](StepRegs<MT, NW>& r, int step) {
    const int k = step * KSTEP + lq * 8;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int at = k + c * 32 < K ? k + c * 32 : 0;
#pragma unroll
      for (int t = 0; t < NW; ++t) r.w[t][c] = *(const uintx4*)(wrow[t] + at);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) r.x[mt][c] = *(const uintx4*)(xrow[mt] + at);
    }
  };
  auto multiply = [&](const StepRegs<MT, NW>& r, int step) {
    const bool reaches_beyond = (step + 1) * KSTEP > K;      // the same for the whole wave
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        uintx4 xv = r.x[mt][c];
        if (reaches_beyond && step * KSTEP + lq * 8 + c * 32 >= K) xv = uintx4{0u, 0u, 0u, 0u};
        const bf16x8 a = __builtin_bit_cast(bf16x8, xv);
#pragma unroll
        for (int t = 0; t < NW; ++t)
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, r.w[t][c]), acc[mt][t], 0, 0, 0);
      }
  };

  // steps wave, wave + WAVES, ...: two register sets, the next step's loads fly while this one multiplies
  const int all_steps = (K + KSTEP - 1) / KSTEP;
  const int first_step = blockIdx.y * steps_per_split;
  const int steps = min(all_steps, first_step + steps_per_split);
  // The product of a step is written out in both arms of each branch, so that the wait before it
  // is the arm's own: behind a common join it would be a wait for every load in flight.
  StepRegs<MT, NW> ra, rb;
  int step = first_step + wave;
  if (step < steps) {
    load(ra, step);
    while (true) {
      const int next = step + WAVES;
      if (next >= steps) { multiply(ra, step); break; }
      load(rb, next);
      multiply(ra, step);
      const int after = next + WAVES;
      if (after >= steps) { multiply(rb, next); break; }
      load(ra, after);
      multiply(rb, next);
      step = after;
    }
  }

  // the waves' partial sums meet in LDS, one (m tile, n tile) at a time, and are added in wave order
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int p = 0; p < NT; ++p) {
      float gate = 0.f;
#pragma unroll
      for (int half = 0; half < NW / NT; ++half) {
        __syncthreads();
        *(floatx4*)&red[wave][lane][0] = acc[mt][p + half * NT];
        __syncthreads();
        if (tid < 256) {
          const int src_lane = tid >> 2;
          const int i = tid & 3;
          float v = 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) v += red[wv][src_lane][i];
          const int m = mt * 16 + (src_lane >> 4) * 4 + i;
          const int n = base + p * ROWS + (src_lane & 15);
          if (m < M && n < N) {
            if (EPI == EPI_SWIGLU) {
              if (half == 0) gate = v;
              else ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(silu_mul(gate, v));
            } else if (EPI == EPI_F32) {
              ((float*)out)[(size_t)m * ldo + n] = v;
            } else {
              ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(v);
            }
          }
        }
      }
    }
}

struct SkinnyCall {
  const void* x;
  const void* w;
  void* out;
  int M, N, K;
  long long ldw, ldo;
  int second_offset;      // rows between a gate row and its up row
  int splits;             // parts of K, each summed by blocks of its own (float32 epilogue)
  long long part_stride;  // floats between the parts' outputs
  hipStream_t stream;
};

template <int MT, int NT, int EPI, int WAVES>
static int launch_skinny(const SkinnyCall& c) {
  const int blocks = (c.N + ROWS * NT - 1) / (ROWS * NT);
  const int steps = (c.K + KSTEP - 1) / KSTEP;
  const int splits = EPI == EPI_F32 ? c.splits : 1;
  const int per_split = (steps + splits - 1) / splits;
  gemm_skinny_kernel<MT, NT, EPI, WAVES><<<dim3(blocks, splits), WAVES * 64, 0, c.stream>>>(
      (const bf16_t*)c.x, (const bf16_t*)c.w, c.out, c.M, c.N, c.K, c.ldw, c.ldo, c.second_offset, per_split,
      c.part_stride);
  return fe_check_launch();
}

// Resident variant for weights with many row tiles and K up to 6144: a launch has at most
// RESIDENT_BLOCKS blocks, each takes tiles blockIdx.x, blockIdx.x + gridDim.x, ... and reads its
// slices of x ONCE into registers for all of them.  Reading x again for every 16 weight rows
// costs a third of the speed at 8 rows of x although it comes from the L2 cache (measured on
// MI355X: 4.4 against 6.2 TB/s for the 778 MB of a 151936 x 2560 head).  The sums are formed in
// the same order as in the kernel above, so both give the same bits.
// K beyond 4096 (up to 6144) takes blocks of 16 waves instead of 8, so that a wave holds at most
// three steps of x: 256 such blocks, one a CU.
#define RESIDENT_BLOCKS 512
#define RESIDENT_WAVES 8
#define RESIDENT_WAVES_WIDE 16
#define RESIDENT_MAX_STEPS (3 * RESIDENT_WAVES_WIDE)    // three steps a wave: four would spill at 16 waves a block

template <int EPI, int XS, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_resident_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N,
    int K, long long ldw, long long ldo, int second_offset, int tiles) {
  constexpr int HALVES = EPI == EPI_SWIGLU ? 2 : 1;
  __shared__ __attribute__((aligned(16))) float red[HALVES][WAVES][64][4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int lr = lane & 15;
  const int lq = lane >> 4;

  // this wave's k-steps are wave, wave + WAVES, ...; XS of them cover K
  uintx4 xr[XS][4];
  {
    const bf16_t* xrow = x + (size_t)(lr < M ? lr : 0) * K;
#pragma unroll
    for (int s = 0; s < XS; ++s) {
      const int k = (wave + s * WAVES) * KSTEP + lq * 8;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        uintx4 v = uintx4{0u, 0u, 0u, 0u};
        if (lr < M && k + c * 32 < K) v = *(const uintx4*)(xrow + k + c * 32);
        xr[s][c] = v;
      }
    }
  }

  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int row = tile * ROWS + lr;
    const bool row_ok = row < N;
    floatx4 acc[HALVES];
#pragma unroll
    for (int half = 0; half < HALVES; ++half) {
      const bf16_t* wrow = w + (size_t)(row_ok ? row + half * second_offset : 0) * ldw;
      uintx4 wr[XS][4];
#pragma unroll
      for (int s = 0; s < XS; ++s) {
        const int k = (wave + s * WAVES) * KSTEP + lq * 8;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          uintx4 v = uintx4{0u, 0u, 0u, 0u};
          if (row_ok && k + c * 32 < K) v = *(const uintx4*)(wrow + k + c * 32);
          wr[s][c] = v;
        }
      }
      acc[half] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < XS; ++s)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          acc[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xr[s][c]),
                                                              __builtin_bit_cast(bf16x8, wr[s][c]), acc[half], 0, 0, 0);
    }
    __syncthreads();
#pragma unroll
    for (int half = 0; half < HALVES; ++half) *(floatx4*)&red[half][wave][lane][0] = acc[half];
    __syncthreads();
    if (tid < 256) {
      const int src_lane = tid >> 2;
      const int i = tid & 3;
      float v[HALVES];
#pragma unroll
      for (int half = 0; half < HALVES; ++half) {
        v[half] = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) v[half] += red[half][wv][src_lane][i];
      }
      const int m = (src_lane >> 4) * 4 + i;
      const int n = tile * ROWS + (src_lane & 15);
      if (m < M && n < N) {
        if (EPI == EPI_SWIGLU) ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(silu_mul(v[0], v[HALVES - 1]));
        else if (EPI == EPI_F32) ((float*)out)[(size_t)m * ldo + n] = v[0];
        else ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(v[0]);
      }
    }
  }
}

static bool resident_fits(int M, int N, int K) {
  const int steps = (K + KSTEP - 1) / KSTEP;
  return M <= 16 && steps <= RESIDENT_MAX_STEPS && (N + ROWS - 1) / ROWS > RESIDENT_BLOCKS;
}

template <int EPI>
static int launch_resident(const void* x, const void* w, void* out, int M, int N, int K, long long ldw,
                           long long ldo, int second_offset, hipStream_t stream) {
  const int tiles = (N + ROWS - 1) / ROWS;
  const int steps = (K + KSTEP - 1) / KSTEP;
  const bool wide = steps > 4 * RESIDENT_WAVES;
  const int waves = wide ? RESIDENT_WAVES_WIDE : RESIDENT_WAVES;
  const int most = wide ? RESIDENT_BLOCKS / 2 : RESIDENT_BLOCKS;
  const int blocks = tiles < most ? tiles : most;
  const int xs = (steps + waves - 1) / waves;
#define FE_GO(XS, WV)                                                                               \
  gemm_skinny_resident_kernel<EPI, XS, WV><<<blocks, WV * 64, 0, stream>>>(                          \
      (const bf16_t*)x, (const bf16_t*)w, out, M, N, K, ldw, ldo, second_offset, tiles)
  if (wide) FE_GO(3, RESIDENT_WAVES_WIDE);
  else if (xs <= 1) FE_GO(1, RESIDENT_WAVES);
  else if (xs == 2) FE_GO(2, RESIDENT_WAVES);
  else if (xs == 3) FE_GO(3, RESIDENT_WAVES);
  else FE_GO(4, RESIDENT_WAVES);
#undef FE_GO
  return fe_check_launch();
}

// Register budget: a wave holds MT x (weight tiles) accumulators and two sets of
// operand registers; shapes beyond these limits would spill.
static constexpr bool shape_fits(int mt, int weight_tiles, int waves) {
  const int registers = 2 * 16 * (weight_tiles + mt) + 4 * mt * weight_tiles;   // operands twice + sums
  return registers <= 240 && (waves < 16 || (mt == 1 && weight_tiles <= 2));
}

static int clamp_tiles(int mt, int epilogue, int tiles) {
  const int pair = epilogue == EPI_SWIGLU ? 2 : 1;
  while (tiles > 1 && !shape_fits(mt, tiles * pair, 8)) tiles >>= 1;
  return tiles;
}

template <int MT, int NT, int EPI>
static int dispatch_waves(int waves, const SkinnyCall& c) {
  constexpr int WT = NT * (EPI == EPI_SWIGLU ? 2 : 1);
  if constexpr (shape_fits(MT, WT, 16)) {
    if (waves == 16) return launch_skinny<MT, NT, EPI, 16>(c);
  }
  if (waves >= 8) return launch_skinny<MT, NT, EPI, 8>(c);
  return launch_skinny<MT, NT, EPI, 4>(c);
}

template <int MT, int EPI>
static int dispatch_tiles(int nt, int waves, const SkinnyCall& c) {
  constexpr int PAIR = EPI == EPI_SWIGLU ? 2 : 1;
  if constexpr (shape_fits(MT, 4 * PAIR, 8)) {
    if (nt == 4) return dispatch_waves<MT, 4, EPI>(waves, c);
  }
  if constexpr (shape_fits(MT, 2 * PAIR, 8)) {
    if (nt >= 2) return dispatch_waves<MT, 2, EPI>(waves, c);
  }
  return dispatch_waves<MT, 1, EPI>(waves, c);
}

template <int EPI>
static int dispatch(int mt, int nt, int waves, const SkinnyCall& c) {
  if (mt == 1) return dispatch_tiles<1, EPI>(nt, waves, c);
  if (mt == 2) return dispatch_tiles<2, EPI>(nt, waves, c);
  return dispatch_tiles<4, EPI>(nt, waves, c);
}

// x [M, K] bf16 contiguous; w [N, K] (epilogue 0, 1) or [2N, K] with the gate
// rows first (epilogue 2), row stride ldw; out [M, N] with row stride ldo,
// float32 (0) or bf16 (1, 2).  tiles/waves: 0 lets the kernel choose how many
// 16-row tiles a wave takes (1, 2, 4: more tiles share each read of x) and how
// many waves share a block's K (4, 8, 16), aiming at a few thousand waves.  tiles -1 asks for
// the resident variant (refused where it does not apply); 0 uses it wherever it applies.
// splits > 1 (float32 epilogue, at most 16): K is cut into that many parts of whole 128-steps,
// each summed by blocks of its own into out + part * part_stride; the caller adds the parts up
// (in a fixed order, so the result stays deterministic).
extern "C" int fe_gemm_skinny(const void* x, const void* w, void* out, int M, int N, int K,
                              long long ldw, long long ldo, int epilogue, int tiles, int waves,
                              int splits, long long part_stride, hipStream_t stream) {
  if (M < 1) return FE_OK;
  if (splits < 1 || splits > 16 || (splits > 1 && (epilogue != EPI_F32 || part_stride < (long long)M * ldo)))
    return FE_BAD_ARGUMENT;
  if (M > 64 || N < 1 || K < 8 || K % 8 || ldw < K || ldw % 8 || ldo < N) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)x) & 15) || (((uintptr_t)w) & 15)) return FE_BAD_ARGUMENT;
  if (epilogue < 0 || epilogue > 2) return FE_BAD_ARGUMENT;
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int steps = (K + KSTEP - 1) / KSTEP;
  const int weight_rows = epilogue == EPI_SWIGLU ? 2 * N : N;
  if (tiles == -1 || (tiles == 0 && waves == 0 && splits == 1 && resident_fits(M, N, K))) {
    if (M > 16 || steps > RESIDENT_MAX_STEPS || splits != 1) return FE_BAD_ARGUMENT;
    if (epilogue == EPI_SWIGLU) return launch_resident<EPI_SWIGLU>(x, w, out, M, N, K, ldw, ldo, N, stream);
    if (epilogue == EPI_F32) return launch_resident<EPI_F32>(x, w, out, M, N, K, ldw, ldo, 0, stream);
    return launch_resident<EPI_BF16>(x, w, out, M, N, K, ldw, ldo, 0, stream);
  }
  if (tiles == 0) {
    // measured on MI355X: up to 16 rows of x one tile per wave is fastest at every width; with more
    // rows two tiles share each read of x and win once the weight has a few thousand rows
    tiles = (mt > 1 && weight_rows >= 4096) ? 2 : 1;
    if (epilogue == EPI_SWIGLU) tiles = 1;   // a gated tile is already a pair
  }
  if (tiles != 1 && tiles != 2 && tiles != 4) return FE_BAD_ARGUMENT;
  tiles = clamp_tiles(mt, epilogue, tiles);
  if (waves == 0) {
    waves = 8;
    while (waves > 4 && waves > (steps + splits - 1) / splits) waves >>= 1;
  }
  if (waves != 4 && waves != 8 && waves != 16) return FE_BAD_ARGUMENT;
  if (waves == 16 && !shape_fits(mt, tiles * (epilogue == EPI_SWIGLU ? 2 : 1), 16)) waves = 8;
  const SkinnyCall call = {x, w, out, M, N, K, ldw, ldo, epilogue == EPI_SWIGLU ? N : 0, splits, part_stride, stream};
  if (epilogue == EPI_SWIGLU) return dispatch<EPI_SWIGLU>(mt, tiles, waves, call);
  if (epilogue == EPI_F32) return dispatch<EPI_F32>(mt, tiles, waves, call);
  return dispatch<EPI_BF16>(mt, tiles, waves, call);
}
