// The float32 matrix product y = x . W^T with W stored [N, K] row-major (the layout of a bias-free
// linear layer's weight): float32 inputs, float32 products and sums. The order of additions for one
// output element does not depend on M, on the tile it falls in or on anything else in the batch, so the
// 32-bit path gives the same value for a token however the work is cut.
//
// me_gemm_f32 runs on the matrix cores' float32 instruction (v_mfma_f32_32x32x2_f32: float32 operands,
// float32 accumulation, no reduced-precision mode), which adds the products of an output element two k at
// a time in ascending k; me_gemm_plain is the same product on the vector ALUs for any storage type.
#include "common.h"

typedef float float16v_t __attribute__((ext_vector_type(16)));

// A block of WM x WN waves owns BM rows of x and BN rows of W and walks k in tiles of 16 through a
// double-buffered LDS stage, k-major ([k][row]: the 64 lanes of a product's operand, 32 rows at each of two k, read
// consecutive words). Wave tiles are multiples of 32 x 32; a lane of a 32 x 32 result holds column lane % 32 and the
// rows 8 (v / 4) + 4 (lane / 32) + v % 4 of its sixteen registers v. Rows beyond M or N and k beyond K are zeros.
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64) void gemm_f32_mfma_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                            float* __restrict__ C, int M, int N, int K, int vector_loads) {
  constexpr int THREADS = WM * WN * 64;
  constexpr int KT = 16, WMR = BM / WM, WNR = BN / WN, FM = WMR / 32, FN = WNR / 32;
  constexpr int GA = BM * (KT / 4), GB = BN * (KT / 4);                          // groups of four k per tile
  constexpr int NA = (GA + THREADS - 1) / THREADS, NB = (GB + THREADS - 1) / THREADS;  // per thread (the last threads may have none)
  static_assert(WMR % 32 == 0 && WNR % 32 == 0, "wave tiles are multiples of 32 x 32");
  __shared__ float As[2][KT][BM + 4];
  __shared__ float Ws[2][KT][BN + 4];
  const int tid = threadIdx.x, wave = tid / ME_WAVE, lane = tid & (ME_WAVE - 1);
  const int wm = wave % WM, wn = wave / WM;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

  float16v_t acc[FM][FN];
#pragma unroll
  for (int a = 0; a < FM; ++a)
#pragma unroll
    for (int b = 0; b < FN; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  // four k of one row per thread and group: four lanes cover 64 contiguous bytes of a row
  auto fetch = [&](const float* __restrict__ src, int rows, int row, int k, float (&v)[4]) {
    v[0] = v[1] = v[2] = v[3] = 0.f;
    if (row >= rows) return;
    const float* p = src + (size_t)row * K + k;
    if (vector_loads && k + 3 < K) {
      const float4 q = *reinterpret_cast<const float4*>(p);
      v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (k + j < K) v[j] = p[j];
    }
  };
  // While a tile is multiplied out of one LDS buffer the next waits in registers, requested at the head of the iteration
  // and written to the other buffer at its end. (Tiles requested further ahead made neither the one-wave blocks of
  // decode-sized steps nor the large tiles faster: the former's time is their chain of dependent matrix instructions
  // and the LDS traffic around it.)
  float ra[NA][4], rb[NB][4];
  auto fetch_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int idx = tid + i * THREADS;
      if (GA % THREADS == 0 || idx < GA) fetch(A, M, m0 + idx / 4, k0 + (idx % 4) * 4, ra[i]);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = tid + i * THREADS;
      if (GB % THREADS == 0 || idx < GB) fetch(W, N, n0 + idx / 4, k0 + (idx % 4) * 4, rb[i]);
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int idx = tid + i * THREADS;
      if (GA % THREADS != 0 && idx >= GA) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) As[buf][(idx % 4) * 4 + j][idx / 4] = ra[i][j];
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = tid + i * THREADS;
      if (GB % THREADS != 0 && idx >= GB) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) Ws[buf][(idx % 4) * 4 + j][idx / 4] = rb[i][j];
    }
  };

  fetch_tile(0);
  store_tile(0);
  __syncthreads();
  const int tiles = (K + KT - 1) / KT;
  const int half = lane / 32, col = lane % 32;
  for (int t = 0; t < tiles; ++t) {
    const int buf = t & 1;
    if (t + 1 < tiles) fetch_tile((t + 1) * KT);
#pragma unroll
    for (int kk = 0; kk < KT; kk += 2) {
      float a[FM], b[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) a[i] = As[buf][kk + half][wm * WMR + i * 32 + col];
#pragma unroll
      for (int j = 0; j < FN; ++j) b[j] = Ws[buf][kk + half][wn * WNR + j * 32 + col];
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (t + 1 < tiles) store_tile(buf ^ 1);  // last read before the barrier that ended tile t - 1
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int n = n0 + wn * WNR + j * 32 + col;
      if (n >= N) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WMR + i * 32 + 8 * (v / 4) + 4 * half + v % 4;
        if (m < M) C[(size_t)m * N + n] = acc[i][j][v];
      }
    }
}

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

// Every tile shape adds an output element's products in the same order, so a row's values do not depend on the
// shape its step happens to get: many rows take 128 x 128 tiles; up to 64 rows take blocks of one wave and 32
// columns (an output element's chain of K / 2 dependent instructions of 64 cycles is such a step's time, whatever
// the rows: as many chains side by side as the columns give).
extern "C" int me_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return me_fail("me_gemm_f32: K=%d", K);
  if (!A || !W || !C) return me_fail("me_gemm_f32: null operand");
  const int vector_loads = K % 4 == 0 && (((uintptr_t)A | (uintptr_t)W) & 15) == 0;
  if (M <= 64) {
    dim3 grid((N + 31) / 32, (M + 31) / 32);
    gemm_f32_mfma_kernel<32, 32, 1, 1><<<grid, 64, 0, stream>>>(A, W, C, M, N, K, vector_loads);
    return me_check_launch("me_gemm_f32");
  }
  dim3 grid((N + 127) / 128, (M + 127) / 128);
  if (grid.y > 65535) return me_fail("me_gemm_f32: M=%d needs more than 65535 row tiles", M);
  gemm_f32_mfma_kernel<128, 128, 2, 2><<<grid, 256, 0, stream>>>(A, W, C, M, N, K, vector_loads);
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
