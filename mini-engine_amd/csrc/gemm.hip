// The float32 matrix product y = x . W^T with W stored [N, K] row-major (the layout of a bias-free
// linear layer's weight): float32 inputs, float32 accumulation on the vector ALUs in ascending k
// order. The order of additions for one output element does not depend on M, on the tile it falls
// in or on anything else in the batch, so the 32-bit path gives the same value for a token however
// the work is cut.
#include "common.h"

// ------------------------------------------------------------------------------- float32 GEMM
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const TIn* __restrict__ A, const TIn* __restrict__ W,
                                                         TOut* __restrict__ C, int M, int N, int K) {
  __shared__ float As[F32_BK][F32_BM + 4];
  __shared__ float Ws[F32_BK][F32_BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
  const int tx = tid % 16, ty = tid / 16;  // thread computes rows ty*4.., cols tx*4..
  float acc[4][4] = {};
  // loader mapping: 256 threads fetch 64 rows x 16 k; thread -> (row = tid / 4, k4 = (tid % 4) * 4)
  const int lrow = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += F32_BK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + j][lrow] = (am < M && k < K) ? to_float(A[(size_t)am * K + k]) : 0.f;
      Ws[lk + j][lrow] = (wn < N && k < K) ? to_float(W[(size_t)wn * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F32_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
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
      if (n < N) C[(size_t)m * N + n] = from_float<TOut>(acc[i][j]);
    }
  }
}

extern "C" int me_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return me_fail("me_gemm_f32: K=%d", K);
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
  if (grid.y > 65535) return me_fail("me_gemm_f32: M=%d needs more than 65535 row tiles", M);
  gemm_plain_kernel<float, float><<<grid, 256, 0, stream>>>(A, W, C, M, N, K);
  return me_check_launch("me_gemm_f32");
}

// The same kernel for any storage type: bfloat16 operands are widened as they are loaded, the sum stays
// float32 on the vector units, the result is stored as float32 or bfloat16. It takes every size, at a
// fraction of the matrix cores' speed; bfloat16 products that neither the matrix-core kernels nor the GEMM
// library take (widths that are no multiple of 8) go here.
extern "C" int me_gemm_plain(const void* A, const void* W, void* C, int M, int N, int K, int in_dtype, int out_dtype,
                             hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return me_fail("me_gemm_plain: K=%d", K);
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
  if (grid.y > 65535) return me_fail("me_gemm_plain: M=%d needs more than 65535 row tiles", M);
  if (in_dtype == ME_F32 && out_dtype == ME_F32)
    gemm_plain_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (float*)C, M, N, K);
  else if (in_dtype == ME_BF16 && out_dtype == ME_F32)
    gemm_plain_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (float*)C, M, N, K);
  else if (in_dtype == ME_BF16 && out_dtype == ME_BF16)
    gemm_plain_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (bf16_t*)C, M, N, K);
  else
    return me_fail("me_gemm_plain: float32 operands give float32 results");
  return me_check_launch("me_gemm_plain");
}
