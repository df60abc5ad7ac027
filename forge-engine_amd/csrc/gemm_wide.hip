// bfloat16 matrix product for a few to a few hundred rows of x (a step of decoding requests, or
// one that holds a portion of a prompt):
//   out[M, N] = x[M, K] * W[N, K]^T
// with one of three endings: float32 partial sums over parts of K ([parts][M, N]; the consumer, the
// next norm, adds them in order), bfloat16, or silu(gate) * up as bfloat16 for a fused gate/up
// weight.  At these row counts the product is bound by the weight's bytes and by how the rows of x
// reach the matrix cores, not by arithmetic: the matrix library, tuned for large products, takes
// three to four times the time the bytes need.
//
// Block = (64 weight rows, a part of K, a tile of MT * 16 rows of x); four waves of 16 weight rows
// (with the gate/up ending: 16 gate rows and the 16 up rows that belong to them).  The weight goes
// from HBM straight into MFMA operand registers, each element used by one wave only; x (shared by
// the four waves) is staged through LDS in 64-wide steps, two stages, one barrier a step; operands
// are fetched four steps ahead (eight gained nothing), every load unconditional.  A wave needs no
// other wave's sums.  What bounds the kernel, measured over tile shapes and row counts: the bytes
// that all blocks together pull into their CUs (the weight once per row tile, x once per 64 weight
// rows, the partial sums), at about 8 TB/s for the whole chip, so only a launch that keeps every CU
// busy streams the weight at the memory's speed: hence the parts of K where a weight has few rows.
// Tiles of x rows beyond the first read the weight again (from L2: the tiles of one weight tile
// run side by side).
//
// MFMA 16x16x32 bf16 with A = x (16 rows), B = W^T (16 weight rows):
//   lane l supplies A[m = l % 16][k = 8*(l / 16) .. +8], B[k = 8*(l / 16) .. +8][n = l % 16]
//   and receives D[m = 4*(l / 16) + i][n = l % 16].
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define WSTEP 64          // elements of K a step

#define EPI_PARTS 0
#define EPI_BF16 1
#define EPI_SWIGLU 2
#define EPI_SWIGLU_HALF 3     // a wave's 16 weight rows are 8 gate rows and the 8 up rows that belong to them

__device__ __forceinline__ float silu_times(float g, float u) { return g / (1.f + __expf(-g)) * u; }

// 16 bytes from LDS byte address `at` + 2048 * STEP (sixteen rows of a stage further); nothing waits for them here
template <int STEP>
__device__ __forceinline__ uintx4 lds_read16(unsigned int at) {
  uintx4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(STEP * 2048) : "memory");
  return v;
}
// ... with a step that is a constant only once the loop around the call is unrolled
__device__ __forceinline__ uintx4 lds_read16_step(unsigned int at, int step) {
  switch (step) {
#define FE_CASE(I) case I: return lds_read16<I>(at);
    FE_CASE(0) FE_CASE(1) FE_CASE(2) FE_CASE(3) FE_CASE(4) FE_CASE(5) FE_CASE(6) FE_CASE(7)
    FE_CASE(8) FE_CASE(9) FE_CASE(10) FE_CASE(11) FE_CASE(12) FE_CASE(13) FE_CASE(14) FE_CASE(15)
#undef FE_CASE
  }
  return uintx4{0u, 0u, 0u, 0u};
}
// wait until at most PENDING of this wave's LDS accesses are outstanding; `v` is what the wait is for.
// (LDS accesses finish in order.  Whatever else the compiler has under way on the same counter, its own
// LDS stores or a scalar load, makes such a wait stricter, never weaker; and its own waits, which do not
// know of the reads above, likewise.)
template <int PENDING>
__device__ __forceinline__ void lds_arrived(uintx4& v) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(PENDING));
}

// LDS holds a step of x as [row][8 chunks of 16 bytes], chunk c of row r at position c ^ (r % 8):
// the eight lanes that a 16-byte read serves in one cycle then hit eight different bank groups.
template <int MT, int EPI, int R, int WPB>
__global__ __launch_bounds__(64 * WPB, 2) void gemm_wide_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N,
    int K, long long ldw, long long ldo, int steps_per_part, long long part_stride, long long up_offset) {
  constexpr int WF = EPI == EPI_SWIGLU ? 2 : 1;     // weight operands a wave holds: a gate tile and an up tile, or one
  constexpr int THREADS = 64 * WPB;
  constexpr int PIECES = MT * 128;                  // 16-byte pieces of a step of x
  constexpr int XL = (PIECES + THREADS - 1) / THREADS;   // ... that a thread fetches (where the threads do not divide them, the last piece more than once)
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16][WSTEP];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int lr = lane & 15;
  const int lq = lane >> 4;
  // the weight row this lane feeds and the output column it receives: the wave's 16 rows, or, with the
  // half-tile gate/up ending, 8 gate rows (lanes with lr < 8) and the 8 up rows of the same columns
  const int n = EPI == EPI_SWIGLU_HALF ? blockIdx.x * (8 * WPB) + wave * 8 + (lr & 7)
                                       : blockIdx.x * (16 * WPB) + wave * 16 + lr;
  const int m0 = blockIdx.z * MT * 16;
  const bf16_t* wrow = w + (size_t)(n < N ? n : 0) * ldw + (EPI == EPI_SWIGLU_HALF && lr >= 8 ? up_offset : 0);
  const int steps = K / WSTEP;
  const int first = blockIdx.y * steps_per_part;
  const int last = min(steps, first + steps_per_part);

  floatx4 acc[WF][MT];
#pragma unroll
  for (int f = 0; f < WF; ++f)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[f][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  if (first < last) {
    static_assert(R % 2 == 0, "a round of the loop is a whole number of LDS stage rotations");
    uintx4 xr[R][XL], wr[R][WF * 2];
    // x loader: piece p = tid + THREADS i is chunk p % 8 of row p / 8.  Rows of x beyond M read row 0
    // again: their sums are never stored.  Nothing is selected on a loaded value, so no load is
    // waited for where it is issued; a step beyond the part's end reads the last step again.
    auto load_x = [&](int step, uintx4* xdst) {
      step = min(step, last - 1);
#pragma unroll
      for (int i = 0; i < XL; ++i) {
        const int p = min(tid + THREADS * i, PIECES - 1);
        const int row = m0 + (p >> 3);
        xdst[i] = *(const uintx4*)(x + (size_t)(row < M ? row : 0) * K + step * WSTEP + (p & 7) * 8);
      }
    };
    auto load_w = [&](int step, uintx4* wdst) {
      step = min(step, last - 1);
#pragma unroll
      for (int f = 0; f < WF; ++f)
#pragma unroll
        for (int c = 0; c < 2; ++c)
          wdst[f * 2 + c] = *(const uintx4*)(wrow + f * up_offset + step * WSTEP + lq * 8 + c * 32);
    };
    auto store_x = [&](int stage, const uintx4* xsrc) {
#pragma unroll
      for (int i = 0; i < XL; ++i) {
        const int p = min(tid + THREADS * i, PIECES - 1);
        const int row = p >> 3;
        *(uintx4*)&xs[stage][row][((p & 7) ^ (row & 7)) * 8] = xsrc[i];
      }
    };
    // Tiles of 128 rows: the fragments of x (k half c, row tile mt) are requested from LDS AHEAD
    // fragments before the MFMAs that use them, with the waits written out.  The compiler, left to
    // itself, reads every fragment into the same registers and waits for it right there; other waves
    // fill most of those waits (a step of 256 tokens 5.69 -> 5.63 ms with the reads ahead, of 128
    // tokens 4.28 -> 4.21 ms), and with tiles of up to 64 rows all of them (64 rows: 4.84 against 4.87
    // ms a decode step), so those keep the compiler's order.  A lane's address is its place in a
    // stage's first sixteen rows (one for each k half: the swizzle mixes it in) plus a multiple of
    // 2,048 bytes (stage and row tile) that is a constant of the instruction.
    constexpr int FRAGMENTS = 2 * MT;
    constexpr int AHEAD = 3, RING = AHEAD + 1;
    const unsigned int xs_at = (unsigned int)(size_t)(const __attribute__((address_space(3))) char*)&xs[0][0][0];
    const unsigned int a_lane[2] = {xs_at + (unsigned int)(lr * 128 + ((0 + lq) ^ (lr & 7)) * 16),
                                    xs_at + (unsigned int)(lr * 128 + ((4 + lq) ^ (lr & 7)) * 16)};
    auto multiply = [&](int stage, const uintx4* wreg) {
      if constexpr (MT < 8) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const int row = mt * 16 + lr;
            const bf16x8 a = *(const bf16x8*)&xs[stage][row][((c * 4 + lq) ^ (lr & 7)) * 8];
#pragma unroll
            for (int t = 0; t < WF; ++t)
              acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, wreg[t * 2 + c]), acc[t][mt], 0, 0, 0);
          }
        }
      } else {
        auto fragment = [&](int f) -> uintx4 { return lds_read16_step(a_lane[f / MT], stage * MT + f % MT); };
        uintx4 ring[RING];
#pragma unroll
        for (int f = 0; f < AHEAD; ++f) ring[f] = fragment(f);
#pragma unroll
        for (int f = 0; f < FRAGMENTS; ++f) {
          if (f + AHEAD < FRAGMENTS) ring[(f + AHEAD) % RING] = fragment(f + AHEAD);
          const int pending = FRAGMENTS - 1 - f < AHEAD ? FRAGMENTS - 1 - f : AHEAD;
          if (pending >= 3) lds_arrived<3>(ring[f % RING]); else if (pending == 2) lds_arrived<2>(ring[f % RING]);
          else if (pending == 1) lds_arrived<1>(ring[f % RING]); else lds_arrived<0>(ring[f % RING]);
          const bf16x8 a = __builtin_bit_cast(bf16x8, ring[f % RING]);
          const int c = f / MT, mt = f % MT;
#pragma unroll
          for (int t = 0; t < WF; ++t)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, wreg[t * 2 + c]), acc[t][mt], 0, 0, 0);
        }
      }
    };

    // Step s (counted from the part's first) has its operands in register sets s % R: the weight's,
    // fetched R - 1 steps ahead, feed the MFMAs directly; those of x, fetched R steps ahead, go to
    // LDS stage s % 2 one step before they are used (a step's arithmetic is far shorter than a trip
    // to memory, what is stored to LDS has to have arrived, and a launch of few blocks keeps the
    // memory busy only through what each block has in flight).  The loop takes R steps a round so
    // that all of these are compile-time constants; one barrier a step.
#pragma unroll
    for (int u = 0; u < R - 1; ++u) load_w(first + u, wr[u]);
#pragma unroll
    for (int u = 0; u < R; ++u) load_x(first + u, xr[u]);
    store_x(0, xr[0]);
    __syncthreads();
    // The rounds are straight-line code: where branches meet, every load in flight would be waited for.
    int step = first;
    for (; step + R <= last; step += R) {
#pragma unroll
      for (int u = 0; u < R; ++u) {
        load_w(step + u + R - 1, wr[(u + R - 1) % R]);
        load_x(step + u + R, xr[u]);
        multiply(u % 2, wr[u]);
        store_x((u + 1) % 2, xr[(u + 1) % R]);
        __syncthreads();
      }
    }
    const int left = last - step;          // 0 .. R - 1 steps, the same for every thread; their operands are on their way
#pragma unroll
    for (int u = 0; u < R - 1; ++u) {
      if (u < left) {
        multiply(u % 2, wr[u]);
        if (u + 1 < left) {
          store_x((u + 1) % 2, xr[(u + 1) % R]);
          __syncthreads();
        }
      }
    }
  }

  // D[m = 4 lq + i][n = lr] of row tile mt: for each i the 16 lanes of a group write 16 neighbouring n
  if (n < N) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + mt * 16 + lq * 4 + i;
        if (EPI != EPI_SWIGLU_HALF && m >= M) continue;      // (the half-tile ending exchanges between lanes first)
        if (EPI == EPI_PARTS) ((float*)out)[(size_t)blockIdx.y * part_stride + (size_t)m * ldo + n] = acc[0][mt][i];
        else if (EPI == EPI_BF16) ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(acc[0][mt][i]);
        else if (EPI == EPI_SWIGLU_HALF) {
          // the lane 8 further in its row of 16 holds the up projection of this lane's column (and the other way round)
          const float other = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc[0][mt][i]), 0x128, 0xF, 0xF, true));
          if (lr < 8 && m < M) ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(silu_times(acc[0][mt][i], other));
        }
        else ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(silu_times(acc[0][mt][i], acc[WF - 1][mt][i]));
      }
  }
}

// x [M, K] bf16 contiguous, K a multiple of 64; w [N, K] bf16 with row stride ldw, rows 16-byte aligned.
// ending 0: out holds `parts` float32 matrices [M, N] (row stride ldo) part_stride floats apart, part s
//   the sum over the s-th run of whole 64-steps of K; every part is written in full (zeros where a part
//   has no steps), so the caller may add all of them up.
// ending 1: out is bfloat16 [M, N] with row stride ldo; parts must be 1.
// ending 2: w is a fused gate/up weight [2 N, K], gate rows first; out is bfloat16 [M, N] =
//   silu(x gate^T) * (x up^T); parts must be 1.  A wave multiplies 16 gate rows and their 16 up rows.
// ending 3: the same result with 8 gate rows and their 8 up rows a wave (one weight operand, the two halves
//   of a result tile meet by a lane exchange), so that a block takes 8 columns a wave: block_rows = 32 to 64
//   in steps of 8 (four to eight waves) is then the block's columns, chosen so that the blocks fill rounds of
//   one a CU.
// Any M: rows are taken in tiles of row_tile = 16, 32, 64 or 128 (smaller tiles: more blocks, and the weight
// read again, from L2, once per tile; a tile's rows beyond M are fetched and multiplied all the same, so
// few rows want a small tile; ending 2 takes tiles of 64 and 128 only).  block_rows = 64 or 32: the weight rows (gate/up ending: output
// columns) a block of four or two waves takes; 32 gives a launch of few blocks twice as many; 128 (eight
// waves, plain endings) halves how often x is read.
extern "C" int fe_gemm_wide(const void* x, const void* w, void* out, int M, int N, int K, long long ldw,
                            long long ldo, int ending, int parts, long long part_stride, int row_tile,
                            int block_rows, hipStream_t stream) {
  if (M < 1) return FE_OK;
  if (N < 1 || K < WSTEP || K % WSTEP || ldw < K || ldw % 8 || ldo < N) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)x) & 15) || (((uintptr_t)w) & 15)) return FE_BAD_ARGUMENT;
  if (ending < EPI_PARTS || ending > EPI_SWIGLU_HALF) return FE_BAD_ARGUMENT;
  if (parts < 1 || parts > 64 || (ending != EPI_PARTS && parts != 1)) return FE_BAD_ARGUMENT;
  if (parts > 1 && part_stride < (long long)M * ldo) return FE_BAD_ARGUMENT;
  const int steps = K / WSTEP;
  const int per_part = (steps + parts - 1) / parts;
  if (row_tile != 16 && row_tile != 32 && row_tile != 64 && row_tile != 128) return FE_BAD_ARGUMENT;
  const int mt = row_tile / 16;
  const long long m_tiles = (M + mt * 16 - 1) / (mt * 16);
  if (m_tiles > 65535) return FE_BAD_ARGUMENT;
  if (ending == EPI_SWIGLU_HALF ? (block_rows < 32 || block_rows > 64 || block_rows % 8) : (block_rows != 128 && block_rows != 64 && block_rows != 32))
    return FE_BAD_ARGUMENT;
  dim3 grid((N + block_rows - 1) / block_rows, parts, (unsigned)m_tiles);
  const long long up_offset = (long long)N * ldw;
#define FE_LAUNCH(MT, EPI, WPB)                                                                                  \
  gemm_wide_kernel<MT, EPI, 4, WPB><<<grid, 64 * WPB, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, \
                                                                    ldw, ldo, per_part, part_stride, up_offset)
#define FE_GO(MT, EPI)                                  \
  do {                                                  \
    if (block_rows == 128) FE_LAUNCH(MT, EPI, 8);       \
    else if (block_rows == 64) FE_LAUNCH(MT, EPI, 4);   \
    else FE_LAUNCH(MT, EPI, 2);                         \
  } while (0)
#define FE_HALF(MT)                                                                                              \
  do {                                                                                                           \
    const int waves = block_rows / 8;                                                                            \
    if (waves == 4) FE_LAUNCH(MT, EPI_SWIGLU_HALF, 4); else if (waves == 5) FE_LAUNCH(MT, EPI_SWIGLU_HALF, 5);  \
    else if (waves == 6) FE_LAUNCH(MT, EPI_SWIGLU_HALF, 6); else if (waves == 7) FE_LAUNCH(MT, EPI_SWIGLU_HALF, 7); \
    else FE_LAUNCH(MT, EPI_SWIGLU_HALF, 8);                                                                      \
  } while (0)
  if (mt == 1) {         // up to 16 rows a tile: the plain endings and the half-tile gate/up ending
    if (ending == EPI_PARTS) FE_GO(1, EPI_PARTS); else if (ending == EPI_BF16) FE_GO(1, EPI_BF16);
    else if (ending == EPI_SWIGLU) return FE_BAD_ARGUMENT; else FE_HALF(1);
  } else if (mt == 2) {
    if (ending == EPI_PARTS) FE_GO(2, EPI_PARTS); else if (ending == EPI_BF16) FE_GO(2, EPI_BF16);
    else if (ending == EPI_SWIGLU) return FE_BAD_ARGUMENT; else FE_HALF(2);
  } else if (mt == 4) {
    if (ending == EPI_PARTS) FE_GO(4, EPI_PARTS); else if (ending == EPI_BF16) FE_GO(4, EPI_BF16);
    else if (ending == EPI_SWIGLU) FE_GO(4, EPI_SWIGLU); else FE_HALF(4);
  } else {
    if (ending == EPI_PARTS) FE_GO(8, EPI_PARTS); else if (ending == EPI_BF16) FE_GO(8, EPI_BF16);
    else if (ending == EPI_SWIGLU) FE_GO(8, EPI_SWIGLU); else FE_HALF(8);
  }
#undef FE_HALF
#undef FE_GO
#undef FE_LAUNCH
  return fe_check_launch();
}
