// bfloat16 matrix product for 17 to 64 rows with float32 partial sums:
//   parts[s][M, N] = x[M, Ks] * W[N, Ks]^T   for the s-th part Ks of K,
// the update of the residual stream that the output and down projections produce
// when a few dozen requests decode together.  At these row counts the product is
// still bound by the weight's bytes, and the weight (N = hidden size) has too few
// rows to fill the chip unless K is split; the consumer (the next norm) adds the
// parts in order, so no atomics and a result that does not depend on timing.
//
// Block = 64 weight rows (four waves of 16) x one part of K.  The weight goes from
// HBM straight into MFMA operand registers, each element used by one wave only;
// x (shared by the four waves) is staged through LDS in 128-wide steps, three
// stages, one barrier a step, operands fetched two steps ahead.  A wave needs no other wave's sums: its 16 weight
// rows are its own, so there is no reduction at the end.
//
// MFMA 16x16x32 bf16 with A = x (16 rows), B = W^T (16 weight rows):
//   lane l supplies A[m = l % 16][k = 8*(l / 16) .. +8], B[k = 8*(l / 16) .. +8][n = l % 16]
//   and receives D[m = 4*(l / 16) + i][n = l % 16].
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;

#define KSTEP 128
#define BLOCK_ROWS 64

// MT row tiles of x (16 rows each).  LDS holds a step of x as [row][16 chunks of 16 bytes], chunk c
// of row r at position c ^ (r % 16): the 16 lanes that read one chunk index of 16 rows then hit
// 16 different bank groups.
//
// A step's operands are fetched two steps before they are used: a step's arithmetic (16 MFMAs
// at 64 rows) is far shorter than a trip to memory, and a part of K is only a few steps long.
// Three register sets rotate through a loop unrolled three times; the one or two steps that
// remain run after it from the sets they were fetched into.  Every load is unconditional (past
// the part's end the last step is read again and not used), so the loop body is straight-line
// code and the loads stay where they are issued.
template <int MT>
__global__ __launch_bounds__(256, 2) void gemm_mid_parts_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, float* __restrict__ out, int M, int N,
    int K, long long ldw, long long ldo, int steps_per_part, long long part_stride) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[3][MT * 16][KSTEP];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int lr = lane & 15;
  const int lq = lane >> 4;
  const int n = blockIdx.x * BLOCK_ROWS + wave * 16 + lr;
  const bf16_t* wrow = w + (size_t)(n < N ? n : 0) * ldw;
  const int steps = (K + KSTEP - 1) / KSTEP;
  const int first = blockIdx.y * steps_per_part;
  const int last = min(steps, first + steps_per_part);

  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  if (first < last) {
    uintx4 xr[3][MT], wr[3][4];
    // x loader: piece p = tid + 256 i is chunk p % 16 of row p / 16 (MT pieces a thread)
    // K is a multiple of the step, and rows of x beyond M read row 0 again: their sums are
    // never stored.  Nothing is selected on a loaded value, so no load is waited for where it
    // is issued.
    auto load = [&](int step, uintx4* xdst, uintx4* wdst) {
      step = min(step, last - 1);
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int p = tid + 256 * i;
        const int row = p >> 4;
        xdst[i] = *(const uintx4*)(x + (size_t)(row < M ? row : 0) * K + step * KSTEP + (p & 15) * 8);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) wdst[c] = *(const uintx4*)(wrow + step * KSTEP + lq * 8 + c * 32);
    };
    auto store_x = [&](int stage, const uintx4* xsrc) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int p = tid + 256 * i;
        const int row = p >> 4;
        *(uintx4*)&xs[stage][row][(((p & 15) ^ (row & 15))) * 8] = xsrc[i];
      }
    };
    auto multiply = [&](int stage, const uintx4* wreg) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bf16x8 b = __builtin_bit_cast(bf16x8, wreg[c]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int row = mt * 16 + lr;
          const bf16x8 a = *(const bf16x8*)&xs[stage][row][((c * 4 + lq) ^ lr) * 8];
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
        }
      }
    };

    // Step s (counted from the part's first) has its operands in register set s % 3 and its x in
    // LDS stage s % 3.  The loop takes three steps a round so that both are compile-time constants.
    load(first, xr[0], wr[0]);
    load(first + 1, xr[1], wr[1]);
    store_x(0, xr[0]);
    __syncthreads();
    int step = first;
    for (; step + 3 <= last; step += 3) {
#pragma unroll
      for (int u = 0; u < 3; ++u) {
        load(step + u + 2, xr[(u + 2) % 3], wr[(u + 2) % 3]);
        multiply(u, wr[u]);
        store_x((u + 1) % 3, xr[(u + 1) % 3]);
        __syncthreads();
      }
    }
    const int left = last - step;          // 0 .. 2 steps, the same for every thread
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (u < left) {
        if (u + 2 < left) load(step + u + 2, xr[(u + 2) % 3], wr[(u + 2) % 3]);
        multiply(u % 3, wr[u % 3]);
        if (u + 1 < left) {
          store_x((u + 1) % 3, xr[(u + 1) % 3]);
          __syncthreads();
        }
      }
    }
  }

  // D[m = 4 lq + i][n = lr] of row tile mt: for each i the 16 lanes of a group write 16 neighbouring n
  if (n < N) {
    float* dst = out + (size_t)blockIdx.y * part_stride + n;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = mt * 16 + lq * 4 + i;
        if (m < M) dst[(size_t)m * ldo] = acc[mt][i];
      }
  }
}

// x [M, K] bf16 contiguous, 16 < M <= 64 (fewer rows work too), K a multiple of 128; w [N, K] bf16 with row stride ldw;
// out: `parts` float32 matrices [M, N] (row stride ldo) part_stride floats apart, part s holding
// the sum over the s-th run of whole 128-steps of K.  Every part is written in full (zeros where a
// part has no steps), so the caller may add all of them up.
extern "C" int fe_gemm_mid_parts(const void* x, const void* w, float* out, int M, int N, int K,
                                 long long ldw, long long ldo, int parts, long long part_stride,
                                 hipStream_t stream) {
  if (M < 1) return FE_OK;
  if (M > 64 || N < 1 || K < KSTEP || K % KSTEP || ldw < K || ldw % 8 || ldo < N) return FE_BAD_ARGUMENT;
  if ((((uintptr_t)x) & 15) || (((uintptr_t)w) & 15)) return FE_BAD_ARGUMENT;
  if (parts < 1 || parts > 64 || (parts > 1 && part_stride < (long long)M * ldo)) return FE_BAD_ARGUMENT;
  const int steps = (K + KSTEP - 1) / KSTEP;
  const int per_part = (steps + parts - 1) / parts;
  dim3 grid((N + BLOCK_ROWS - 1) / BLOCK_ROWS, parts);
  const int mt = (M + 15) / 16;
#define FE_GO(MT)                                                                                      \
  gemm_mid_parts_kernel<MT><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, \
                                                      ldw, ldo, per_part, part_stride)
  if (mt == 1) FE_GO(1);
  else if (mt == 2) FE_GO(2);
  else if (mt == 3) FE_GO(3);
  else FE_GO(4);
#undef FE_GO
  return fe_check_launch();
}
