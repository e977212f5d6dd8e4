// Matrix products y = x * W^T (+ bias) for gfx950, W stored [N, K] row-major as checkpoints
// hold it.
//  * cw_gemm_f32: true float32 (VALU FMA, float32 operands and accumulation, no reduced-precision
//    matrix mode). The K loop of one output element runs in the same order whatever M is, so a
//    row's result does not depend on what else is in the batch.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

// C[M, N] = A[M, K] * W[N, K]^T + bias[N]. 256 threads, each a 4x4 tile of a 64x64 block.
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, int64_t lda,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ bias,
                                                       float* __restrict__ C, int64_t ldc, int M,
                                                       int N, int K) {
  __shared__ float As[GT_BK][GT_BM + 4];
  __shared__ float Ws[GT_BK][GT_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

  // each thread loads 4 elements of A and 4 of W per K step: row = tid / 4, k = (tid % 4) * 4 .. +3
  const int lr = tid >> 2, lk = (tid & 3) * 4;
  const bool k_vec_ok = (K % 4 == 0) && (lda % 4 == 0);
  for (int k0 = 0; k0 < K; k0 += GT_BK) {
    {
      const int m = m0 + lr, k = k0 + lk;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (m < M) {
        const float* p = A + (int64_t)m * lda + k;
        if (k_vec_ok && k + 3 < K) {
          const float4 q = *reinterpret_cast<const float4*>(p);
          v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (k + j < K) v[j] = p[j];
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) As[lk + j][lr] = v[j];
    }
    {
      const int n = n0 + lr, k = k0 + lk;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (n < N) {
        const float* p = W + (int64_t)n * K + k;
        if (K % 4 == 0 && k + 3 < K) {
          const float4 q = *reinterpret_cast<const float4*>(p);
          v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (k + j < K) v[j] = p[j];
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) Ws[lk + j][lr] = v[j];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GT_BK; ++kk) {
      const float4 a = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);
      const float4 w = *reinterpret_cast<const float4*>(&Ws[kk][tx * 4]);
      const float av[4] = {a.x, a.y, a.z, a.w};
      const float wv[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(int64_t)m * ldc + n] = acc[i][j] + (bias ? bias[n] : 0.0f);
    }
  }
}

CW_EXPORT int cw_gemm_f32(const float* A, int64_t lda, const float* W, const float* bias, float* C,
                          int64_t ldc, int M, int N, int K, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldc < N) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return CW_ERR_ARG;
  dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM), block(256);
  if (grid.y > 65535) return CW_ERR_SIZE;
  hipLaunchKernelGGL(gemm_f32_kernel, grid, block, 0, stream, A, lda, W, bias, C, ldc, M, N, K);
  return cw_launch_status();
}
