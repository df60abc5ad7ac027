// bfloat16 matrix products for steps that hold dozens to thousands of rows (portions of prompts,
// whole prompts, large decode batches), with the ending fused:
//   gated:  out[M, I] = silu(x Wg^T) * (x Wu^T)   for a fused gate/up weight [2 I, K], gate rows first
//
// A block keeps a tile of rows of x, 64 elements of K at a time, in LDS, several steps deep; the
// tile goes there by `global_load_lds_dwordx4` (no staging registers, no LDS stores) and is shared
// by the block's waves.  The weight goes from memory straight into MFMA operand registers, several
// steps ahead.  A wave owns 16 * MT rows of the tile and, of the output, 16 * NG columns: their
// gate rows and their up rows, so that 16 * MT x 32 * NG accumulators stay in registers for the
// whole of K and silu(gate) * up is formed from them lane by lane, without a trip through memory
// for the 2 I wide intermediate.  An A fragment read from LDS feeds 2 NG MFMAs, a B fragment from
// memory MT of them.  The block is RW x CW waves: RW take different rows, CW different columns.
//
// With one or two waves a SIMD nothing hides a wave's own latencies, so the order of a step is
// written out: the A fragments are read a fixed number of fragments ahead of the MFMAs that use
// them, across the boundary between two steps, and the block's one barrier a step sits where the
// reads cross that boundary.  The LDS reads and the weight's loads are inline assembly, each with
// the wait for it written out and tied to the registers it is for.  The compiler's own waits would
// empty the pipeline at every step: it orders every LDS read that it sees behind ALL loads into LDS
// in flight, and while loads into LDS and loads into registers are both in flight it turns every
// wait for the latter into a wait for everything.  The counts of the written waits rest on the one
// order in which a wave issues its loads (the weight of a step, then the x of a step, in turn).
//
// MFMA 16x16x32 bf16 with A = W (16 weight rows), B = x^T (16 rows of x):
//   lane l supplies A[m = l % 16][k = 8*(l / 16) .. +8], B[k = 8*(l / 16) .. +8][n = l % 16]
//   and receives D[m = 4*(l / 16) + i][n = l % 16]: four neighbouring output columns of one row
//   of x, which leave as one 8-byte store.
#include "common.h"
#include <algorithm>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define KSTEP 64          // elements of K a step

// wait until at most n of this wave's vector memory operations are outstanding (n < 64)
#define FE_WAIT_VMEM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | ((((n) >> 4) & 0x3) << 14) | (0x7 << 4) | (0xF << 8))

__device__ __forceinline__ void load_to_lds(const void* global, void* lds) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                   (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// 16 bytes from LDS byte address `at` + OFFSET (a constant below 65536); nothing waits for them here
template <int OFFSET>
__device__ __forceinline__ uintx4 lds_read16(unsigned int at) {
  uintx4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(OFFSET) : "memory");
  return v;
}
// wait until at most PENDING of this wave's LDS reads are outstanding; `v` is what the wait is for
template <int PENDING>
__device__ __forceinline__ void lds_arrived(uintx4& v) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(PENDING));
}
// 16 bytes from global memory at `from` + OFFSET bytes (a constant below 4096) into `v`; nothing waits
// for them here.  `v` is an operand that is read and written: the registers of a load in flight must
// not look free to the compiler (it would give them to something else, and the data would land on
// that), so every load into a variable is chained to the one before it and, through the wait that
// follows some time later, to the use.
template <int OFFSET>
__device__ __forceinline__ void global_read16(uintx4& v, const void* from) {
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "+v"(v) : "v"(from), "n"(OFFSET) : "memory");
}
// wait until at most PENDING of this wave's loads from global memory are outstanding; `v` is what the wait is for
template <int PENDING, int COUNT>
__device__ __forceinline__ void global_arrived(uintx4* v) {
  static_assert(COUNT == 4 || COUNT == 8, "a wave's weight operands of a step");
  if constexpr (COUNT == 4)
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : "n"(PENDING));
  else
    asm volatile("s_waitcnt vmcnt(%8)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])
                 : "n"(PENDING));
}

__device__ __forceinline__ float silu_times(float g, float u) { return g / (1.f + __expf(-g)) * u; }

// LDS holds a step of x as [row][8 chunks of 16 bytes], chunk c of row r at position c ^ (r % 8):
// the lanes that a 16-byte read serves in one cycle then hit different bank groups.  A wave's load
// instruction fills 64 consecutive 16-byte units (8 rows); which chunk of memory a lane asks for is
// what places the chunks.
//
// One tile: block `block_id` of a region of `col_blocks` column blocks x `row_tiles` row tiles whose
// first column is `first_col` (a launch is one region, or two with tiles of different widths).
template <int MT, int NG, int RW, int CW, int STAGES, int R, int D>
__device__ __forceinline__ void gated_tile(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, bf16_t* __restrict__ out, int M, int N,
    int K, long long ldw, long long ldo, long long up_offset, int block_id, int col_blocks, int row_tiles,
    int first_col) {
  constexpr int THREADS = 64 * RW * CW;
  constexpr int ROWS = MT * 16 * RW;                 // rows of x a block holds
  constexpr int NF = 2 * NG;                         // weight operands a wave holds: NG gate tiles, then their NG up tiles
  constexpr int XL = ROWS * 8 / THREADS;             // load instructions a thread issues for a step of x
  constexpr int WL = NF * 2;                         // ... and for a step of its weight rows
  constexpr int STAGE_BYTES = ROWS * 128;
  constexpr int P = 2 * MT;                          // A fragments a wave reads a step: position p is k half p / MT of row tile p % MT
  static_assert(ROWS * 8 % THREADS == 0 && STAGES >= 3 && R >= 2, "tile shape");
  static_assert(P % D == 0 && D <= P && D >= 1 && D <= 16, "fragments are read D ahead, in a ring of D");
  static_assert((STAGES - 2) * (XL + WL) < 64 && (R - 1) * (XL + WL) < 64, "the count of loads in flight must fit the wait instruction");
  extern __shared__ __attribute__((aligned(16))) uintx4 xs[];     // [STAGES][ROWS][8]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int lr = lane & 15;
  const int lq = lane >> 4;
  const int wave_row = wave / CW, wave_col = wave % CW;
  // Block id b runs on XCD b % 8.  The row tiles of one column block read the same weight rows:
  // they get neighbouring ids on one XCD, so that the second tile finds the rows in that XCD's L2.
  const int group = block_id / (8 * row_tiles), within = block_id % (8 * row_tiles);
  const int col_block = group * 8 + within % 8;
  const int row_tile = within / 8;
  if (col_block >= col_blocks) return;
  const int col0 = first_col + (col_block * CW + wave_col) * 16 * NG;
  const int m0 = row_tile * ROWS;

  // x: unit u = tid + THREADS * i of a stage is position u % 8 of row u / 8 and holds the row's chunk
  // (u % 8) ^ (row % 8); rows beyond M read the last row again (their results are never stored)
  // (as 32-bit element offsets: both operands are smaller than 2^32 elements, the host checks)
  const int x_chunk = (tid & 7) ^ ((tid >> 3) & 7);
  unsigned int x_from[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int row = min(m0 + (tid >> 3) + (THREADS / 8) * i, M - 1);
    x_from[i] = (unsigned int)row * (unsigned int)K + x_chunk * 8;
  }
  // weight rows of this lane: columns beyond N read the last column's rows again
  unsigned int w_from[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int col = min(col0 + (f % NG) * 16 + lr, N - 1);
    w_from[f] = (unsigned int)((size_t)col * ldw + (f >= NG ? up_offset : 0) + lq * 8);
  }
  const int steps = K / KSTEP;
  // where this lane reads its A fragments: row lr of the wave's rows, chunk lq (k half 0) or 4 + lq (k half 1)
  const unsigned int lds_base = (unsigned int)(size_t)(__attribute__((address_space(3))) char*)xs;
  const unsigned int a_lane[2] = {
      lds_base + (unsigned int)(((wave_row * MT * 16 + lr) * 8 + ((0 + lq) ^ (lr & 7))) * 16),
      lds_base + (unsigned int)(((wave_row * MT * 16 + lr) * 8 + ((4 + lq) ^ (lr & 7))) * 16)};

  floatx4 acc[NF][MT];
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[f][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  uintx4 wr[R][WL];
#pragma unroll
  for (int u = 0; u < R; ++u)
#pragma unroll
    for (int i = 0; i < WL; ++i) wr[u][i] = uintx4{0, 0, 0, 0};
  uintx4 ring[D];
  // Loads.  A wave issues NV = XL + WL of them a step, always in the same order: the XL pieces of the x
  // of step t + AX, then the WL pieces of its weight of step t + AW, spread over the step's positions
  // (issued in one burst, the four waves' loads queue up in front of the CU's one address unit and every
  // wave stands still behind its own).  Every load is unconditional: a step beyond the last reads the
  // last step again, into a stage, or registers, that nobody reads any more, and the steps before the
  // first (the prologue) read step 0.  So "the x (the weight) of step s has arrived" is "at most the
  // loads issued after it are outstanding", and that count is the same at every step.
  constexpr int NV = XL + WL;
  constexpr int AX = STAGES - 2;       // the stage of step t + AX was read last in step t - 2: every wave is past the barrier behind it
  constexpr int AW = R - 1;
  constexpr int PB = P - D;            // the position before which the step's barrier stands: from there on the reads are the next step's
  static_assert(P >= NV, "a position issues at most one load");
  auto issue = [&](int j, int t, int u) {       // load j of the NV that step t issues; u = t modulo R, kept apart so that it is a constant
    if (j < XL) {
      const int target = t + AX;
      const int s = min(max(target, 0), steps - 1);
      uintx4* stage = xs + (size_t)((target + STAGES) % STAGES) * (STAGE_BYTES / 16);
      load_to_lds(x + x_from[j] + s * KSTEP, stage + wave * 64 + THREADS * j);
    } else {
      const int k = j - XL;
      const int s = min(max(t + AW, 0), steps - 1);
      uintx4& to = wr[(u + AW) % R][k];
      if (k % 2 == 0) global_read16<0>(to, w + w_from[k / 2] + s * KSTEP);
      else global_read16<64>(to, w + w_from[k / 2] + s * KSTEP);
    }
  };
  // load j goes out behind position j * P / NV
  auto load_behind = [](int p) { const int j = (p * NV + P - 1) / P; return j < NV && j * P / NV == p ? j : -1; };
  constexpr int before_barrier = (PB * NV + P - 1) / P;     // loads of a step issued before its barrier

  // position q of a step whose stage begins `stage_offset` bytes into LDS (q is a constant wherever
  // this is called: the row tile's offset is an immediate of the instruction)
  auto read_fragment = [&](int q, unsigned int stage_offset) -> uintx4 {
    const unsigned int from = stage_offset + a_lane[q / MT];
    switch (q % MT) {
#define FE_CASE(I) case I: return lds_read16<(I) * 2048>(from);
      FE_CASE(0) FE_CASE(1) FE_CASE(2) FE_CASE(3) FE_CASE(4) FE_CASE(5) FE_CASE(6) FE_CASE(7)
      FE_CASE(8) FE_CASE(9) FE_CASE(10) FE_CASE(11) FE_CASE(12) FE_CASE(13) FE_CASE(14) FE_CASE(15)
#undef FE_CASE
    }
    return uintx4{0, 0, 0, 0};
  };

  // the steps before the first: their loads, in the order of every step
  constexpr int V = AX > AW ? AX : AW;
#pragma unroll
  for (int t = -V; t < 0; ++t) {
#pragma unroll
    for (int j = 0; j < NV; ++j) issue(j, t, ((t % R) + R) % R);
    __builtin_amdgcn_sched_barrier(0);
  }
  FE_WAIT_VMEM(WL + (AX - 1) * NV);      // behind the x of step 0: the weight loads of its step and AX - 1 whole steps
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int p = 0; p < D; ++p) ring[p] = read_fragment(p, 0);
  __builtin_amdgcn_sched_barrier(0);

  for (int step = 0; step < steps; step += R) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int t = step + u;
      if (t < steps) {
        const unsigned int here = (unsigned int)((t % STAGES) * STAGE_BYTES);
        const unsigned int next = (unsigned int)(((t + 1) % STAGES) * STAGE_BYTES);
        // the weight of this step was the last that step t - AW issued: behind it came AW - 1 whole steps
        global_arrived<(AW - 1) * NV, WL>(wr[u]);
#pragma unroll
        for (int p = 0; p < P; ++p) {
          if (p == PB) {
            // From here on the reads are the next step's.  Its x has arrived for this wave (behind it came
            // the weight loads of its step, AX - 2 whole steps and this step's loads so far) and, behind the
            // barrier, for every wave.
            FE_WAIT_VMEM(WL + (AX - 2) * NV + before_barrier);
            __builtin_amdgcn_s_barrier();
          }
          lds_arrived<D - 1>(ring[p % D]);
          const bf16x8 a = __builtin_bit_cast(bf16x8, ring[p % D]);
#pragma unroll
          for (int f = 0; f < NF; ++f)
            acc[f][p % MT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(bf16x8, wr[u][f * 2 + p / MT]), a, acc[f][p % MT], 0, 0, 0);
          if (load_behind(p) >= 0) issue(load_behind(p), t, u);
          // the position read now, D ahead: of this step, or of the next
          ring[p % D] = read_fragment((p + D) % P, p + D < P ? here : next);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
  // The last steps requested fragments and weight of steps that do not exist.  Their registers stay
  // taken until the data has arrived: a register that the compiler believes free while a load into it
  // is in flight would be given to something else and then overwritten.
#pragma unroll
  for (int p = 0; p < D; ++p) lds_arrived<0>(ring[p]);
#pragma unroll
  for (int u = 0; u < R; ++u) global_arrived<0, WL>(wr[u]);

  // D[m = 4 lq + i][n = lr] of row tile mt: columns col .. col + 3 of row lr of the tile, gate and up of
  // the same element in the same lane.  (Where the lane stands is worked out again from its number, behind
  // a statement that the compiler cannot see through: kept from the top, these few values would be the ones
  // that do not fit the registers during the loop.)
  int tid_again = threadIdx.x;
  asm volatile("" : "+v"(tid_again));
  const int lr_out = tid_again & 15, lq_out = (tid_again & 63) >> 4;
  const int wave_row_out = (tid_again >> 6) / CW, wave_col_out = (tid_again >> 6) % CW;
  const int col0_out = first_col + (col_block * CW + wave_col_out) * 16 * NG;
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int col = col0_out + g * 16 + lq_out * 4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = m0 + (wave_row_out * MT + mt) * 16 + lr_out;
      if (m >= M) continue;
      bf16_t y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = float_to_bf16(silu_times(acc[g][mt][i], acc[NG + g][mt][i]));
      bf16_t* to = out + (size_t)m * ldo + col;
      if (col + 3 < N && (ldo & 3) == 0 && ((uintptr_t)out & 7) == 0) {
        uint2 packed;
        packed.x = (unsigned int)y[0] | ((unsigned int)y[1] << 16);
        packed.y = (unsigned int)y[2] | ((unsigned int)y[3] << 16);
        *(uint2*)to = packed;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < N) to[i] = y[i];
      }
    }
  }
}

template <int MT, int NG, int RW, int CW, int STAGES, int R, int D>
__global__ __launch_bounds__(64 * RW * CW, 1) void gemm_gated_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, bf16_t* __restrict__ out, int M, int N,
    int K, long long ldw, long long ldo, long long up_offset, int col_blocks, int row_tiles) {
  gated_tile<MT, NG, RW, CW, STAGES, R, D>(x, w, out, M, N, K, ldw, ldo, up_offset, blockIdx.x, col_blocks, row_tiles, 0);
}

// Tiles of 256 x 128 for as many columns as fill whole rounds of one block a CU, tiles of 256 x 64 for
// the columns that are left: the last, partly filled round then takes two thirds of a round's time
// instead of a whole one (2,048 rows x 9,728 columns: 608 wide tiles are 2.4 rounds of 256 CUs; 512
// wide and 192 narrow ones are 2 + 0.66).  The blocks of the wide tiles come first.
__global__ __launch_bounds__(256, 1) void gemm_gated_mixed_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, bf16_t* __restrict__ out, int M, int N,
    int K, long long ldw, long long ldo, long long up_offset, int wide_blocks, int wide_col_blocks,
    int narrow_col_blocks, int row_tiles) {
  if ((int)blockIdx.x < wide_blocks)
    gated_tile<16, 2, 1, 4, 4, 3, 4>(x, w, out, M, N, K, ldw, ldo, up_offset, blockIdx.x, wide_col_blocks, row_tiles, 0);
  else
    gated_tile<16, 1, 1, 4, 4, 4, 8>(x, w, out, M, N, K, ldw, ldo, up_offset, blockIdx.x - wide_blocks, narrow_col_blocks,
                                     row_tiles, wide_col_blocks * 128);
}

// The kernels' loads are waited for by hand, on registers that the compiler must leave alone
// meanwhile: a build that spills registers to scratch memory would move values that are still in
// flight (and its scratch accesses would be loads that the waits do not count).  Such a build is
// never launched.  Also raises the kernel's LDS limit.  0: not yet asked, 1: fit, -1: refused.
static int fit_to_launch(const void* kernel, size_t lds_bytes, int* checked) {
  if (*checked == 0) {
    hipFuncAttributes attributes;
    if (hipFuncGetAttributes(&attributes, kernel) != hipSuccess) return FE_LAUNCH_FAILED;
    if (attributes.localSizeBytes != 0) { *checked = -1; return FE_BAD_ARGUMENT; }
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
      return FE_LAUNCH_FAILED;
    *checked = 1;                 // (a race here only repeats the calls)
  }
  return *checked < 0 ? FE_BAD_ARGUMENT : FE_OK;
}

template <int MT, int NG, int RW, int CW, int STAGES, int R, int D>
static int launch_gated(const void* x, const void* w, void* out, int M, int N, int K, long long ldw, long long ldo,
                        hipStream_t stream) {
  constexpr int rows = MT * 16 * RW;
  constexpr size_t lds_bytes = (size_t)STAGES * rows * 128;
  static_assert(lds_bytes <= 160 * 1024, "LDS of a CU");
  static int checked = 0;
  auto kernel = gemm_gated_kernel<MT, NG, RW, CW, STAGES, R, D>;
  const int fit = fit_to_launch((const void*)kernel, lds_bytes, &checked);
  if (fit != FE_OK) return fit;
  const int col_blocks = (N + CW * 16 * NG - 1) / (CW * 16 * NG);
  const int row_tiles = (M + rows - 1) / rows;
  const long long blocks = (long long)((col_blocks + 7) / 8) * 8 * row_tiles;
  if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  kernel<<<(unsigned)blocks, 64 * RW * CW, lds_bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)out, M, N, K,
                                                               ldw, ldo, (long long)N * ldw, col_blocks, row_tiles);
  return fe_check_launch();
}

#define FE_CUS 256
// Wide tiles alone, or wide tiles for whole rounds and narrow ones for the rest, whichever takes fewer
// rounds (a round of narrow tiles counted as two thirds of a round of wide ones: measured).
static int launch_gated_rounds(const void* x, const void* w, void* out, int M, int N, int K, long long ldw, long long ldo,
                               hipStream_t stream) {
  const int row_tiles = (M + 255) / 256;
  const int all_wide = (N + 127) / 128;
  const long long tiles = (long long)row_tiles * all_wide;
  const int wide_cols = (int)std::min<long long>(all_wide, (tiles / FE_CUS) * FE_CUS / row_tiles);   // column blocks of the whole rounds
  const int narrow_cols = (N - wide_cols * 128 + 63) / 64;
  const double plain = (double)((tiles + FE_CUS - 1) / FE_CUS);
  const double mixed = (double)(((long long)wide_cols * row_tiles + FE_CUS - 1) / FE_CUS) +
                       0.67 * (double)(((long long)narrow_cols * row_tiles + FE_CUS - 1) / FE_CUS);
  if (wide_cols == 0 || narrow_cols <= 0 || mixed >= plain)
    return launch_gated<16, 2, 1, 4, 4, 3, 4>(x, w, out, M, N, K, ldw, ldo, stream);
  constexpr size_t lds_bytes = (size_t)4 * 256 * 128;
  static int checked = 0;
  const int fit = fit_to_launch((const void*)gemm_gated_mixed_kernel, lds_bytes, &checked);
  if (fit != FE_OK) return fit;
  const long long wide_blocks = (long long)((wide_cols + 7) / 8) * 8 * row_tiles;
  const long long narrow_blocks = (long long)((narrow_cols + 7) / 8) * 8 * row_tiles;
  if (wide_blocks + narrow_blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  gemm_gated_mixed_kernel<<<(unsigned)(wide_blocks + narrow_blocks), 256, lds_bytes, stream>>>(
      (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)out, M, N, K, ldw, ldo, (long long)N * ldw, (int)wide_blocks, wide_cols,
      narrow_cols, row_tiles);
  return fe_check_launch();
}

// x [M, K] bf16 contiguous, K a multiple of 64; w [2 N, K] bf16 with row stride ldw (a multiple of 8),
// gate rows first; out [M, N] bf16 with row stride ldo: out = silu(x gate^T) * (x up^T), float32 sums.
// shape: which tile a block of four waves takes (rows of x x output columns):
//   0: 256 x 64, waves of 256 rows x 16 columns     1: 256 x 128, waves of 256 rows x 32 columns
//   2: 128 x 64, waves of 128 rows x 16 columns
//   3: tiles of 256 x 128 for the columns that fill whole rounds of one block a CU, 256 x 64 for the rest
// The weight is read once per row tile.  Both operands must be smaller than 2^32 elements.
// FE_BAD_ARGUMENT also if the library was built with registers spilled to scratch memory (see
// launch_gated): the kernel then never runs.
extern "C" int fe_gemm_gated(const void* x, const void* w, void* out, int M, int N, int K, long long ldw, long long ldo,
                             int shape, hipStream_t stream) {
  if (M < 1) return FE_OK;
  if (N < 1 || K < KSTEP || K % KSTEP || ldw < K || ldw % 8 || ldo < N) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)x) & 15) || (((uintptr_t)w) & 15)) return FE_BAD_ARGUMENT;
  if ((long long)M * K >= (1LL << 32) || 2LL * N * ldw >= (1LL << 32)) return FE_BAD_ARGUMENT;   // 32-bit element offsets inside
  switch (shape) {
    case 0: return launch_gated<16, 1, 1, 4, 4, 4, 8>(x, w, out, M, N, K, ldw, ldo, stream);
    case 1: return launch_gated<16, 2, 1, 4, 4, 3, 4>(x, w, out, M, N, K, ldw, ldo, stream);
    case 2: return launch_gated<8, 1, 1, 4, 6, 4, 8>(x, w, out, M, N, K, ldw, ldo, stream);
    case 3: return launch_gated_rounds(x, w, out, M, N, K, ldw, ldo, stream);
  }
  return FE_BAD_ARGUMENT;
}
