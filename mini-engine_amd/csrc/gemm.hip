// Matrix products y = x . W^T with W stored [N, K] row-major (the layout of a bias-free linear
// layer's weight), for two cases:
//
//  * me_gemm_f32: float32 inputs, float32 accumulation on the vector ALUs in ascending k order.
//    The order of additions for one output element does not depend on M, on the tile it falls in
//    or on anything else in the batch, so the 32-bit path gives the same value for a token however
//    the work is cut.
//  * me_gemm_bf16_skinny: bfloat16 inputs with M <= 64 rows (decode steps, logits rows) on the
//    matrix cores. W streams from HBM once; the four waves of a block split k and reduce through
//    LDS. Output is bfloat16 or float32.
#include "common.h"

// ------------------------------------------------------------------------------- float32 GEMM
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                       float* __restrict__ C, int M, int N, int K) {
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
      As[lk + j][lrow] = (am < M && k < K) ? A[(size_t)am * K + k] : 0.f;
      Ws[lk + j][lrow] = (wn < N && k < K) ? W[(size_t)wn * K + k] : 0.f;
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
      if (n < N) C[(size_t)m * N + n] = acc[i][j];
    }
  }
}

extern "C" int me_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return me_fail("me_gemm_f32: K=%d", K);
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
  if (grid.y > 65535) return me_fail("me_gemm_f32: M=%d needs more than 65535 row tiles", M);
  gemm_f32_kernel<<<grid, 256, 0, stream>>>(A, W, C, M, N, K);
  return me_check_launch("me_gemm_f32");
}

// ------------------------------------------------------------------- bfloat16 skinny-M GEMM
// Block = 4 waves, 16 output columns, all M rows (MT tiles of 16). The product is computed
// transposed, C^T[n, m] = sum_k W[n, k] X[m, k], so that both matrix-core operands are read along k,
// the contiguous direction of both W and X, straight from global memory:
//   A operand (16 x 16): lane l holds W[n0 + l%16][kc + (l/16)*4 .. +4]
//   B operand (16 x 16): lane l holds X[m0 + l%16][kc + (l/16)*4 .. +4]
//   result: lane l holds C^T[(l/16)*4 .. +4][l%16], i.e. four consecutive n for row m = l%16.
// A lane fetches 8 consecutive k (16 bytes) at a time and feeds two matrix-core steps from it; the
// same permutation of k is applied to both operands, so the sum is unchanged. Waves interleave
// 32-wide k chunks (wave w takes chunks w, w+4, ...), then add their partial sums through LDS in
// wave order.
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

union Frag16 {
  uint4 u;
  short4_t h[2];
};

template <int MT, int U, typename OutT>
__global__ __launch_bounds__(256) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ X,
                                                               const bf16_t* __restrict__ W,
                                                               OutT* __restrict__ C, int M, int N, int K) {
  __shared__ float red[4][MT][64][4];
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int n0 = blockIdx.x * 16;
  const int r = lane % 16, g = lane / 16;
  const int n = n0 + r;
  const bool n_ok = n < N;
  const bf16_t* wrow = W + (size_t)(n_ok ? n : 0) * K;
  float4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (float4_t){0.f, 0.f, 0.f, 0.f};

  // U chunks of 32 k per round: all loads of a round are issued before the first product, so a
  // wave keeps U weight loads in flight instead of one
  const int chunks = (K + 31) / 32;
  for (int c0 = wave; c0 < chunks; c0 += 4 * U) {
    Frag16 a[U], b[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (c0 + 4 * u) * 32 + g * 8;
      a[u].u = make_uint4(0, 0, 0, 0);
      if (n_ok && k < K) a[u].u = *reinterpret_cast<const uint4*>(wrow + k);  // K % 8 == 0 is checked on the host
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (c0 + 4 * u) * 32 + g * 8;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r;
        b[u][t].u = make_uint4(0, 0, 0, 0);
        if (m < M && k < K) b[u][t].u = *reinterpret_cast<const uint4*>(X + (size_t)m * K + k);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a[u].h[0], b[u][t].h[0], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a[u].h[1], b[u][t].h[1], acc[t], 0, 0, 0);
      }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) red[wave][t][lane][j] = acc[t][j];
  __syncthreads();
  // 256 threads finish MT*64 lanes' worth of results: thread -> (tile t, lane l)
  for (int idx = threadIdx.x; idx < MT * 64; idx += 256) {
    const int t = idx / 64, l = idx % 64;
    const int m = t * 16 + l % 16;
    const int nb = n0 + (l / 16) * 4;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float s = ((red[0][t][l][j] + red[1][t][l][j]) + red[2][t][l][j]) + red[3][t][l][j];
      if (nb + j < N) C[(size_t)m * N + nb + j] = from_float<OutT>(s);
    }
  }
}

template <typename OutT>
static int launch_skinny(const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, hipStream_t stream) {
  const unsigned blocks = (N + 15) / 16;
  const int mt = (M + 15) / 16;
  switch (mt) {
    case 1: gemm_bf16_skinny_kernel<1, 8, OutT><<<blocks, 256, 0, stream>>>(X, W, C, M, N, K); break;
    case 2: gemm_bf16_skinny_kernel<2, 4, OutT><<<blocks, 256, 0, stream>>>(X, W, C, M, N, K); break;
    case 3: gemm_bf16_skinny_kernel<3, 4, OutT><<<blocks, 256, 0, stream>>>(X, W, C, M, N, K); break;
    default: gemm_bf16_skinny_kernel<4, 4, OutT><<<blocks, 256, 0, stream>>>(X, W, C, M, N, K); break;
  }
  return me_check_launch("me_gemm_bf16_skinny");
}

// out_dtype: ME_BF16 or ME_F32. M may be at most 64; K must be a multiple of 8 (16-byte loads).
extern "C" int me_gemm_bf16_skinny(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64) return me_fail("me_gemm_bf16_skinny: M=%d exceeds 64 rows", M);
  if (K <= 0 || K % 8) return me_fail("me_gemm_bf16_skinny: K=%d must be a positive multiple of 8", K);
  if (((uintptr_t)X | (uintptr_t)W) & 15) return me_fail("me_gemm_bf16_skinny: operands must be 16-byte aligned");
  if (out_dtype == ME_F32)
    return launch_skinny<float>((const bf16_t*)X, (const bf16_t*)W, (float*)C, M, N, K, stream);
  return launch_skinny<bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, N, K, stream);
}
