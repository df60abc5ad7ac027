// True float32 matrix product C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]), both
// operands K-contiguous (activations times a weight in [out, in] layout).
// Plain FMA on the vector ALU, float32 accumulation in a fixed K order that
// does not depend on M: no matrix-core instruction, so no reduced-precision
// mode can slip in.  64x64 output tile per block of 256 threads, K in steps
// of 16 through LDS; any M, N, K.  Up to 16 rows of A with K a multiple of four take a
// weight-streaming variant (below) instead.
#include "common.h"
#include <algorithm>

#define TILE_M 64
#define TILE_N 64
#define TILE_K 16

__global__ __launch_bounds__(256) void gemm_nt_f32_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias,
    float* __restrict__ C, int M, int N, int K, long long lda, long long ldb, long long ldc) {
  // [k][row], padded so that the transposing stores spread over banks
  __shared__ float As[TILE_K][TILE_M + 4];
  __shared__ float Bs[TILE_K][TILE_N + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TILE_M;
  const int n0 = blockIdx.x * TILE_N;
  const int tx = tid % 16;  // 4 columns each
  const int ty = tid / 16;  // 4 rows each
  // loader: thread -> (row = tid / 4, k quad = tid % 4)
  const int lrow = tid / 4;
  const int lk = (tid % 4) * 4;
  const bool vec_ok = (K % 4 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) &&
                      ((((uintptr_t)A) & 15) == 0) && ((((uintptr_t)B) & 15) == 0);

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TILE_K) {
    float a[4] = {0.f, 0.f, 0.f, 0.f};
    float b[4] = {0.f, 0.f, 0.f, 0.f};
    const int am = m0 + lrow;
    const int bn = n0 + lrow;
    const int kk = k0 + lk;
    if (am < M) {
      const float* p = A + (size_t)am * lda + kk;
      if (vec_ok && kk + 3 < K) {
        const float4 v = *(const float4*)p;
        a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) if (kk + i < K) a[i] = p[i];
      }
    }
    if (bn < N) {
      const float* p = B + (size_t)bn * ldb + kk;
      if (vec_ok && kk + 3 < K) {
        const float4 v = *(const float4*)p;
        b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) if (kk + i < K) b[i] = p[i];
      }
    }
    __syncthreads();  // previous tile fully consumed
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[lk + i][lrow] = a[i];
      Bs[lk + i][lrow] = b[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) {
      const float4 av = *(const float4*)&As[k][ty * 4];
      const float4 bv = *(const float4*)&Bs[k][tx * 4];
      const float ar[4] = {av.x, av.y, av.z, av.w};
      const float br[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], br[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * ldc + n] = acc[i][j] + (bias ? bias[n] : 0.f);
    }
  }
}

// The same product for up to 16 rows of A (a decode step), where the work is reading B once:
// a block takes R rows of B and MR rows of A; its four waves split K in interleaved steps of
// 256 (a lane reads 16 contiguous bytes of every row, a wave 1 KB), each lane keeps R x MR
// sums over its own k, the sums meet by a butterfly over the lanes and then over the waves in
// LDS, in a fixed order.  The order of a row's sum depends on K alone: not on M, not on the
// rows beside it, not on R or MR.  Needs K % 4 == 0 and 16-byte aligned rows.
template <int MR, int R>
__global__ __launch_bounds__(256) void gemm_rows_f32_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias,
    float* __restrict__ C, int M, int N, int K, long long lda, long long ldb, long long ldc) {
  __shared__ float red[4][R * MR];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * R, m0 = blockIdx.y * MR;
  const float* arow[MR];
  const float* brow[R];
#pragma unroll
  for (int m = 0; m < MR; ++m) arow[m] = A + (size_t)min(m0 + m, M - 1) * lda;     // rows beyond M: the last again, never stored
#pragma unroll
  for (int r = 0; r < R; ++r) brow[r] = B + (size_t)min(n0 + r, N - 1) * ldb;
  float acc[R][MR];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;

  // Loads are unconditional (a load under a per-lane condition becomes a branch, and where
  // branches meet every load in flight is waited for): a step beyond K reads the row's last
  // four elements again and is never used, because the loop ends first.
  int k = (wave * 64 + lane) * 4;
  float4 bnext[R];
#pragma unroll
  for (int r = 0; r < R; ++r) bnext[r] = *(const float4*)(brow[r] + min(k, K - 4));
  for (; k < K; k += 1024) {
    float4 bv[R], av[MR];
#pragma unroll
    for (int r = 0; r < R; ++r) bv[r] = bnext[r];
#pragma unroll
    for (int m = 0; m < MR; ++m) av[m] = *(const float4*)(arow[m] + k);
    const int kn = min(k + 1024, K - 4);           // the next step's rows of B fly during this step's sums
#pragma unroll
    for (int r = 0; r < R; ++r) bnext[r] = *(const float4*)(brow[r] + kn);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        float s = acc[r][m];
        s = fmaf(av[m].x, bv[r].x, s);
        s = fmaf(av[m].y, bv[r].y, s);
        s = fmaf(av[m].z, bv[r].z, s);
        s = fmaf(av[m].w, bv[r].w, s);
        acc[r][m] = s;
      }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float total = wave_sum(acc[r][m]);
      if (lane == 0) red[wave][r * MR + m] = total;
    }
  __syncthreads();
  if (tid < R * MR) {
    const int r = tid / MR, m = tid - r * MR;
    const int n = n0 + r, row = m0 + m;
    if (n < N && row < M) {
      const float total = ((red[0][tid] + red[1][tid]) + red[2][tid]) + red[3][tid];
      C[(size_t)row * ldc + n] = total + (bias ? bias[n] : 0.f);
    }
  }
}

// The same product for up to 8 rows of A with the rows of A held in registers: a lane's places in K
// are its own for the whole launch (k = 4 (64 wave + lane) + 256 WAVES step), so a block fetches its
// slices of A once and then walks tiles of two rows of B (blocks are persistent: tile b, b + blocks,
// ...), reading nothing but B: the streaming kernel above pulls every row of A through L1 again for
// every four rows of B, twice the bytes of B itself.  The next tile's rows of B fly while this tile
// is multiplied.  The 16 sums of a tile (2 rows of B x 8 of A) meet across the 64 lanes by a
// butterfly that halves the values a lane holds at every exchange (one exchange a value instead of
// six), then across the waves in LDS, in wave order.  K beyond 768 WAVES elements takes further
// passes over the tiles, each adding to what the pass before stored (the same thread wrote it).
// The order of a row's sum depends on K alone.
template <int XS, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_rows_resident_f32_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias,
    float* __restrict__ C, int M, int N, int K, long long lda, long long ldb, long long ldc) {
  constexpr int MR = 8, R = 2, SPAN = 256 * WAVES * XS;     // SPAN: elements of K a pass covers
  __shared__ float red[2][WAVES][R * MR];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k_lane = (wave * 64 + lane) * 4;
  const int tiles = (N + R - 1) / R;
  for (int k0 = 0; k0 < K; k0 += SPAN) {
    // this pass's slices of A: zero beyond K, rows beyond M the last row again (never stored)
    float4 xr[XS][MR];
    int kk[XS];
#pragma unroll
    for (int s = 0; s < XS; ++s) {
      const int k = k0 + k_lane + 256 * WAVES * s;
      kk[s] = min(k, K - 4);
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const float4 v = *(const float4*)(A + (size_t)min(m, M - 1) * lda + kk[s]);
        xr[s][m] = k < K ? v : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
    const bool last_pass = k0 + SPAN >= K;
    float4 bnext[R][XS];
    auto fetch = [&](int tile) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float* brow = B + (size_t)min(tile * R + r, N - 1) * ldb;
#pragma unroll
        for (int s = 0; s < XS; ++s) bnext[r][s] = *(const float4*)(brow + kk[s]);
      }
    };
    fetch(min((int)blockIdx.x, tiles - 1));
    int round = 0;
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x, round ^= 1) {
      float4 bv[R][XS];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int s = 0; s < XS; ++s) bv[r][s] = bnext[r][s];
      fetch(min(tile + (int)gridDim.x, tiles - 1));       // unconditional: past the end the last tile again, never used
      float acc[R * MR];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          float sum = 0.f;
#pragma unroll
          for (int s = 0; s < XS; ++s) {
            sum = fmaf(xr[s][m].x, bv[r][s].x, sum);
            sum = fmaf(xr[s][m].y, bv[r][s].y, sum);
            sum = fmaf(xr[s][m].z, bv[r][s].z, sum);
            sum = fmaf(xr[s][m].w, bv[r][s].w, sum);
          }
          acc[r * MR + m] = sum;
        }
      // 16 values over 64 lanes: lanes 32 apart exchange halves (each keeps eight sums of two lanes), lanes
      // 16 apart quarters, then 8 and 4 apart, and the last two exchanges add what the four lanes of a
      // quad hold: lane l ends with value 8 b5 + 4 b4 + 2 b3 + b2 of its bits, summed over all lanes.
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[i]), __float_as_uint(acc[i + 8]), false, false);
        acc[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(acc[i]), __float_as_uint(acc[i + 4]), false, false);
        acc[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
      }
      const bool up8 = lane & 8, up4 = lane & 4;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float keep = up8 ? acc[i + 2] : acc[i], send = up8 ? acc[i] : acc[i + 2];
        acc[i] = keep + __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(send), 0x128, 0xF, 0xF, true));   // lane ^ 8: a row rotated by 8
      }
      {
        const float keep = up4 ? acc[1] : acc[0], send = up4 ? acc[0] : acc[1];
        acc[0] = keep + __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(send), 0x141, 0xF, 0xF, true));   // 7 - lane within 8
      }
      acc[0] += __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(acc[0]), 0x4E, 0xF, 0xF, true));   // lane ^ 2
      acc[0] += __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(acc[0]), 0xB1, 0xF, 0xF, true));   // lane ^ 1
      if ((lane & 3) == 0) red[round][wave][((lane >> 5) & 1) * 8 + ((lane >> 4) & 1) * 4 + ((lane >> 3) & 1) * 2 + ((lane >> 2) & 1)] = acc[0];
      __syncthreads();
      if (tid < R * MR) {
        const int r = tid / MR, m = tid - r * MR;
        const int n = tile * R + r;
        if (n < N && m < M) {
          float total = red[round][0][tid];
#pragma unroll
          for (int w = 1; w < WAVES; ++w) total += red[round][w][tid];
          float* dst = C + (size_t)m * ldc + n;
          if (k0 > 0) total += *dst;
          *dst = total + (last_pass && bias ? bias[n] : 0.f);
        }
      }
    }
    __syncthreads();    // the last tile's sums are read before the next pass writes over them
  }
}

#define FE_ROWS_F32_MAX 16     // most rows of A that the weight-streaming variant takes
#define FE_ROWS_F32_RESIDENT_MAX 64   // most rows of A that go through the variant with A in registers, eight at a time

extern "C" int fe_gemm_nt_f32(const float* A, const float* B, const float* bias, float* C,
                              int M, int N, int K, long long lda, long long ldb, long long ldc,
                              hipStream_t stream) {
  if (M <= 0 || N <= 0) return FE_OK;
  if (K <= 0 || lda < K || ldb < K || ldc < N) return FE_BAD_ARGUMENT;
  const bool rows_ok = M <= FE_ROWS_F32_MAX && K % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0 &&
                       ((((uintptr_t)A) | ((uintptr_t)B)) & 15) == 0;
  const bool aligned = K % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0 && ((((uintptr_t)A) | ((uintptr_t)B)) & 15) == 0;
  if (aligned && M <= FE_ROWS_F32_RESIDENT_MAX && K >= 1024) {
    // persistent blocks, two a CU with four waves (K up to 3,072 a pass), one with eight; more than
    // eight rows in groups of eight, a launch each: the weight is streamed once a group, which up to
    // 64 rows still beats the tiles below (measured at the 4B sizes, a decode step: 9 rows 11.7 ->
    // 8.2 ms, 17 rows 50.4 -> 11.8 ms, 32 rows 51.5 -> 16.2 ms; 64 rows 31.2 ms), and a row's sums
    // are those of the row alone
    const int tiles = (N + 1) / 2;
    for (int m0 = 0; m0 < M; m0 += 8) {
      const float* a = A + (size_t)m0 * lda;
      float* c = C + (size_t)m0 * ldc;
      const int rows = std::min(8, M - m0);
      if (K <= 2048) gemm_rows_resident_f32_kernel<2, 4><<<std::min(tiles, 512), 256, 0, stream>>>(a, B, bias, c, rows, N, K, lda, ldb, ldc);
      else if (K <= 3072) gemm_rows_resident_f32_kernel<3, 4><<<std::min(tiles, 512), 256, 0, stream>>>(a, B, bias, c, rows, N, K, lda, ldb, ldc);
      else if (K <= 4096) gemm_rows_resident_f32_kernel<2, 8><<<std::min(tiles, 256), 512, 0, stream>>>(a, B, bias, c, rows, N, K, lda, ldb, ldc);
      else gemm_rows_resident_f32_kernel<3, 8><<<std::min(tiles, 256), 512, 0, stream>>>(a, B, bias, c, rows, N, K, lda, ldb, ldc);
    }
    return fe_check_launch();
  }
  if (rows_ok) {
    if (M <= 4) gemm_rows_f32_kernel<4, 8><<<dim3((N + 7) / 8, 1), 256, 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);
    else if (M <= 8) gemm_rows_f32_kernel<8, 4><<<dim3((N + 3) / 4, 1), 256, 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);   // measured: four rows of B a block beat eight (more waves in flight)
    else gemm_rows_f32_kernel<16, 4><<<dim3((N + 3) / 4, 1), 256, 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);
    return fe_check_launch();
  }
  const long long grid_y = (M + TILE_M - 1) / TILE_M;
  if (grid_y > 65535) return FE_BAD_ARGUMENT;
  dim3 grid((N + TILE_N - 1) / TILE_N, (unsigned)grid_y);
  gemm_nt_f32_kernel<<<grid, 256, 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);
  return fe_check_launch();
}
