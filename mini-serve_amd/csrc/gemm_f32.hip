// True float32 matrix product C[M, N] = A[M, K] * W[N, K]^T on the vector ALUs (no matrix-core
// reduced-precision mode). Every output element is one chain of fused multiply-adds over
// k = 0 .. K-1 in ascending order, whatever M is and whichever tile holds it: results do not
// depend on how rows are batched.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16

// mode 0: C = acc (float)   mode 1: C += acc (float)   mode 2: C = bf16(acc)
template <int MODE>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                       void* __restrict__ Cv, int M, int N, int K, int lda, int ldc) {
  __shared__ float As[TK][TM + 4];
  __shared__ float Ws[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tx = tid % 16, ty = tid / 16;  // 16 x 16 threads, 4 x 4 outputs each
  const int lr = tid / 4, lk = (tid % 4) * 4;  // loader: row within tile, k offset
  const bool vec = (K % 4 == 0) && (lda % 4 == 0);
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    float a[4], w[4];
    {
      const int m = m0 + lr, k = k0 + lk;
      if (m < M && vec && k + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(A + (size_t)m * lda + k);
        a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = (m < M && k + i < K) ? A[(size_t)m * lda + k + i] : 0.f;
      }
      const int n = n0 + lr;
      if (n < N && (K % 4 == 0) && k + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(W + (size_t)n * K + k);
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = (n < N && k + i < K) ? W[(size_t)n * K + k + i] : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[lk + i][lr] = a[i];
      Ws[lk + i][lr] = w[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      const size_t at = (size_t)m * ldc + n;
      if (MODE == 0) ((float*)Cv)[at] = acc[i][j];
      else if (MODE == 1) ((float*)Cv)[at] += acc[i][j];
      else ((bf16*)Cv)[at] = static_cast<bf16>(acc[i][j]);
    }
  }
}

extern "C" int ms_gemm_f32(const float* A, const float* W, void* C, int mode, int M, int N, int K, int lda, int ldc,
                           hipStream_t st) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (K <= 0 || lda < K || ldc < N) return MS_BAD_ARG;
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  if (grid.y > 65535) return MS_BAD_ARG;
  if (mode == 0) gemm_f32_kernel<0><<<grid, 256, 0, st>>>(A, W, C, M, N, K, lda, ldc);
  else if (mode == 1) gemm_f32_kernel<1><<<grid, 256, 0, st>>>(A, W, C, M, N, K, lda, ldc);
  else if (mode == 2) gemm_f32_kernel<2><<<grid, 256, 0, st>>>(A, W, C, M, N, K, lda, ldc);
  else return MS_BAD_ARG;
  return launch_status();
}
