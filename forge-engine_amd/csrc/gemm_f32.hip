// True float32 matrix product C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]), both
// operands K-contiguous (activations times a weight in [out, in] layout).
// Plain FMA on the vector ALU, float32 accumulation in a fixed K order that
// does not depend on M: no matrix-core instruction, so no reduced-precision
// mode can slip in.  64x64 output tile per block of 256 threads, K in steps
// of 16 through LDS; any M, N, K.
#include "common.h"

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

extern "C" int fe_gemm_nt_f32(const float* A, const float* B, const float* bias, float* C,
                              int M, int N, int K, long long lda, long long ldb, long long ldc,
                              hipStream_t stream) {
  if (M <= 0 || N <= 0) return FE_OK;
  if (K <= 0 || lda < K || ldb < K || ldc < N) return FE_BAD_ARGUMENT;
  const long long grid_y = (M + TILE_M - 1) / TILE_M;
  if (grid_y > 65535) return FE_BAD_ARGUMENT;
  dim3 grid((N + TILE_N - 1) / TILE_N, (unsigned)grid_y);
  gemm_nt_f32_kernel<<<grid, 256, 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);
  return fe_check_launch();
}
