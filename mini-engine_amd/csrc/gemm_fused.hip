// Skinny bfloat16 product y = x . W^T for decode-sized batches (M <= 64 rows) with what surrounds
// it in a layer fused in, so that a decode step needs fewer, fatter kernels:
//
//   prologue NORM:   the input is the float32 residual stream. Every block forms
//                    s = x_in + delta (float32), uses bf16(s * w_norm) as its operand, sums s^2 on the
//                    way and multiplies its results by rsqrt(mean(s^2) + eps) at the end (the scale of
//                    a row is a common factor of the whole row of the product). Block 0 also writes s
//                    to x_out, the new residual stream; x_out must not alias x_in, since the other
//                    blocks still read x_in.
//   epilogue SWIGLU: W holds gate rows [0, N) and up rows [N, 2N); a block computes 16 gate columns and
//                    the 16 matching up columns and writes silu(gate) * up.
//   rows scaled:     the plain form can multiply its rows by rsqrt(sum of squares / dim + eps), the sums read from
//                    partial sums that the product before left (the second half of a norm carried over, common.h).
//
// A block owns 16 output columns (64 for products with very many columns, whose blocks then share the
// loads of x among four tiles of columns) and all M rows; its WAVES waves split k in interleaved chunks of 32
// and add their partial sums through LDS in wave order. Products use v_mfma_f32_16x16x32_bf16 with
// the transposed arrangement (C^T[n, m] = sum_k W[n, k] X[m, k]): lane l feeds W[n0 + l%16][8 k] and
// X[m0 + l%16][8 k] (k = 32 c + 8 (l/16) ..), both contiguous in memory, and receives
// C^T[4 (l/16) .. +4][l%16]. All loads of a round of U chunks are issued before its products.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

template <int MT, int WAVES, int U, bool NORM, bool SWIGLU, typename OutT, int NT = 1, bool SCALED = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_small_kernel(
    const bf16_t* __restrict__ X, const float* __restrict__ x_in, const bf16_t* __restrict__ delta,
    const float* __restrict__ w_norm, float eps, float* __restrict__ x_out, const bf16_t* __restrict__ W,
    OutT* __restrict__ C, int M, int N, int K, int chunks_per_split, int gate, RowScale rs) {
  // ACCS tiles of 16 weight rows per block: gate and up rows of the same 16 columns (SWIGLU), or NT
  // neighbouring tiles of 16 columns, which share the loads of x (products with very many columns)
  static_assert(!SWIGLU || NT == 1, "the gated form computes one tile of columns per block");
  constexpr int ACCS = SWIGLU ? 2 : NT;
  __shared__ float red[WAVES][MT * ACCS][64][4];
  __shared__ float ssq[WAVES][MT][64];
  __shared__ float row_scale[SCALED ? MT * 16 : 1];  // with rs.ss: what the rows are multiplied by at the end (read behind the barrier below)
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  constexpr int SCALE_ROWS = (MT * 16 + WAVES - 1) / WAVES;  // rows whose scale a wave works out
  float ss_part[SCALE_ROWS];
  if (SCALED && rs.ss) row_ss_fetch<SCALE_ROWS>(rs, M, ss_part, wave, lane, WAVES);
  const int n0 = blockIdx.x * 16 * NT;
  const int r = lane & 15, g = lane >> 4;
  const bf16_t* wrow[ACCS];
  bool n_ok[ACCS];
#pragma unroll
  for (int a = 0; a < ACCS; ++a) {
    const int n = SWIGLU ? n0 + r : n0 + a * 16 + r;
    n_ok[a] = n < N;
    wrow[a] = W + ((SWIGLU && a ? (size_t)N : 0) + (size_t)(n_ok[a] ? n : 0)) * K;
  }
  float4_t acc[MT][ACCS];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] = 0.f;
#pragma unroll
    for (int a = 0; a < ACCS; ++a) acc[t][a] = (float4_t){0.f, 0.f, 0.f, 0.f};
  }
  const bool writes_x = NORM && delta != nullptr && blockIdx.x == 0;

  // blockIdx.y > 0 only with k cut into splits: this block sums chunks [first, last) of 32 k and writes
  // its partial result behind those of the splits before it
  const int first = blockIdx.y * chunks_per_split;
  const int last = min((K + 31) / 32, first + chunks_per_split);
  C += (size_t)blockIdx.y * M * N;
  for (int c0 = first + wave; c0 < last; c0 += WAVES * U) {
    bf16x8_t a[U][ACCS], b[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (c0 + WAVES * u) * 32 + g * 8;
      const bool k_ok = k < K && c0 + WAVES * u < last;  // K % 8 == 0 is checked on the host
#pragma unroll
      for (int aa = 0; aa < ACCS; ++aa) {
        a[u][aa] = bf16x8_t{};
        if (n_ok[aa] && k_ok) a[u][aa] = *reinterpret_cast<const bf16x8_t*>(wrow[aa] + k);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (c0 + WAVES * u) * 32 + g * 8;
      const bool k_ok = k < K && c0 + WAVES * u < last;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r;
        b[u][t] = bf16x8_t{};
        if (m < M && k_ok) {
          if (NORM) {
            const float4 x0 = *reinterpret_cast<const float4*>(x_in + (size_t)m * K + k);
            const float4 x1 = *reinterpret_cast<const float4*>(x_in + (size_t)m * K + k + 4);
            float s[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            if (delta) {
              const uint4 dv = *reinterpret_cast<const uint4*>(delta + (size_t)m * K + k);
              const uint32_t dw[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                s[2 * j] += __uint_as_float(dw[j] << 16);
                s[2 * j + 1] += __uint_as_float(dw[j] & 0xffff0000u);
              }
              if (writes_x) {
                *reinterpret_cast<float4*>(x_out + (size_t)m * K + k) = make_float4(s[0], s[1], s[2], s[3]);
                *reinterpret_cast<float4*>(x_out + (size_t)m * K + k + 4) = make_float4(s[4], s[5], s[6], s[7]);
              }
            }
            const float4 w0 = *reinterpret_cast<const float4*>(w_norm + k);
            const float4 w1 = *reinterpret_cast<const float4*>(w_norm + k + 4);
            const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              ss[t] = fmaf(s[j], s[j], ss[t]);
              b[u][t][j] = (__bf16)(s[j] * wv[j]);
            }
          } else {
            b[u][t] = *reinterpret_cast<const bf16x8_t*>(X + (size_t)m * K + k);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int aa = 0; aa < ACCS; ++aa)
          acc[t][aa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][aa], b[u][t], acc[t][aa], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int aa = 0; aa < ACCS; ++aa)
#pragma unroll
      for (int j = 0; j < 4; ++j) red[wave][t * ACCS + aa][lane][j] = acc[t][aa][j];
    if (NORM) ssq[wave][t][lane] = ss[t];
  }
  if (SCALED && rs.ss) row_scales_finish<SCALE_ROWS>(rs, M, ss_part, row_scale, wave, lane, WAVES);
  __syncthreads();
  if constexpr (!NORM) {
    // Every thread of the block adds up one output element over the waves (thread -> tile t, lane l, element j: row
    // m = 16 t + l % 16, column n0 + 4 (l / 16) + j): eight or sixteen reads of LDS in a row instead of the 32 or 64
    // that a thread had with one wave doing the whole tail.
    for (int e = threadIdx.x; e < MT * 256; e += WAVES * 64) {
      const int t = e >> 8, l = (e >> 2) & 63, j = e & 3;
      const int m = t * 16 + (l & 15);
      if (m >= M) continue;
      const float scale = SCALED && rs.ss ? row_scale[m] : 1.f;
#pragma unroll
      for (int tile = 0; tile < (SWIGLU ? 1 : NT); ++tile) {
        float v0 = 0.f, v1 = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
          v0 += red[w][t * ACCS + tile][l][j];
          if (SWIGLU) v1 += red[w][t * ACCS + 1][l][j];
        }
        v0 *= scale;
        float y = v0;
        if (SWIGLU) y = gate_act_bf16(v0, gate) * (v1 * scale);
        const int col = n0 + (l >> 4) * 4 + tile * 16 + j;
        if (col < N) C[(size_t)m * N + col] = from_float<OutT>(y);
      }
    }
    return;
  }
  // thread -> (tile t, lane l): row m = 16 t + l % 16, columns n0 + 4 (l / 16) .. +4
  for (int idx = threadIdx.x; idx < MT * 64; idx += WAVES * 64) {
    const int t = idx / 64, l = idx % 64;
    const int m = t * 16 + (l & 15);
    const int nb = n0 + (l >> 4) * 4;
    if (m >= M) continue;
    float scale = 1.f;
    if (NORM) {
      // the row's sum of squares: every wave's lanes (l % 16) + 16 g hold a part of it
      float total = 0.f;
      for (int w = 0; w < WAVES; ++w)
        total += (ssq[w][t][l & 15] + ssq[w][t][(l & 15) + 16]) + (ssq[w][t][(l & 15) + 32] + ssq[w][t][(l & 15) + 48]);
      scale = rsqrtf(total / (float)K + eps);
    } else if (SCALED && rs.ss) {
      scale = row_scale[m];
    }
#pragma unroll
    for (int tile = 0; tile < (SWIGLU ? 1 : NT); ++tile) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v0 = 0.f, v1 = 0.f;
        for (int w = 0; w < WAVES; ++w) {
          v0 += red[w][t * ACCS + tile][l][j];
          if (SWIGLU) v1 += red[w][t * ACCS + 1][l][j];
        }
        v0 *= scale;
        float y = v0;
        if (SWIGLU) y = gate_act_bf16(v0, gate) * (v1 * scale);
        const int col = nb + tile * 16 + j;
        if (col < N) C[(size_t)m * N + col] = from_float<OutT>(y);
      }
    }
  }
}

template <int MT, int WAVES, int U, typename OutT>
static void launch_variant(bool norm, int swiglu, const bf16_t* X, const float* x_in, const bf16_t* delta,
                           const float* w_norm, float eps, float* x_out, const bf16_t* W, OutT* C, int M, int N, int K,
                           int splits, RowScale rs, hipStream_t stream) {
  const dim3 blocks((N + 15) / 16, splits);
  const int cps = ((K + 31) / 32 + splits - 1) / splits;
#define ME_LAUNCH(NORM, SWI, SCALED)                                                                                      \
  gemm_small_kernel<MT, WAVES, U, NORM, SWI, OutT, 1, SCALED><<<blocks, WAVES * 64, 0, stream>>>(X, x_in, delta, w_norm, eps, \
                                                                                                 x_out, W, C, M, N, K, cps,   \
                                                                                                 swiglu, rs)
  if (rs.ss && !norm) {  // the forms that scale their rows: instances of their own
    if (swiglu)
      ME_LAUNCH(false, true, true);
    else
      ME_LAUNCH(false, false, true);
    return;
  }
  if (norm && swiglu)
    ME_LAUNCH(true, true, false);
  else if (norm)
    ME_LAUNCH(true, false, false);
  else if (swiglu)
    ME_LAUNCH(false, true, false);
  else
    ME_LAUNCH(false, false, false);
#undef ME_LAUNCH
}

#define WIDE_MIN_COLUMNS 32768

template <typename OutT>
static void launch_small(bool norm, int swiglu, const bf16_t* X, const float* x_in, const bf16_t* delta,
                         const float* w_norm, float eps, float* x_out, const bf16_t* W, OutT* C, int M, int N, int K,
                         int splits, RowScale rs, hipStream_t stream) {
  const int mt = (M + 15) / 16;
  // up to 16 rows: as many chunks of 32 k per wave and round as it takes to have all of k in flight at
  // once (a second round of loads costs a memory round trip, which is most of such a kernel's time)
  const int chunks = ((K + 31) / 32 + splits - 1) / splits;  // per block
  if (mt == 1 && M > 2 && !norm && !swiglu && splits == 1 && N >= WIDE_MIN_COLUMNS && !rs.ss) {
    // very many columns (the output head) and more than a row or two: a block computes 64 columns from
    // one set of loads of x (at 8 rows and 151,936 columns 63 us against 69; at one row it is slower)
    gemm_small_kernel<1, 8, 4, false, false, OutT, 4><<<dim3((N + 63) / 64), 8 * 64, 0, stream>>>(
        X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, chunks, 0, rs);
    return;
  }
  if (mt == 1 && chunks > 8 * 8)
    launch_variant<1, 8, 12, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else if (mt == 1 && chunks > 8 * 4)
    launch_variant<1, 8, 8, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else if (mt == 1)
    launch_variant<1, 8, 4, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else if (mt == 2 && chunks > 8 * 2)
    launch_variant<2, 8, 4, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else if (mt == 2)
    launch_variant<2, 8, 2, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else if (mt == 3)
    launch_variant<3, 8, 4, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else if (swiglu)  // two accumulators per tile: eight waves' partial sums would not fit into 64 KB of LDS
    launch_variant<4, 4, 4, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
  else
    launch_variant<4, 8, 4, OutT>(norm, swiglu, X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, splits, rs, stream);
}

// What both entry points below do; `rs` scales the rows of a plain product (rs.ss == nullptr: not).
static int small_product(const void* X, const float* x_in, const void* delta, const float* w_norm, float eps, float* x_out,
                         const void* W, void* C, int M, int N, int K, int norm, int swiglu, int out_dtype, int k_splits,
                         RowScale rs, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (k_splits < 1 || k_splits > 64) return me_fail("me_gemm_bf16_small: %d splits of k", k_splits);
  if (k_splits > 1 && (norm || swiglu || out_dtype != ME_F32))
    return me_fail("me_gemm_bf16_small: partial sums over splits of k are plain float32 products");
  if (swiglu < ME_GATE_NONE || swiglu > ME_GATE_GELU_TANH) return me_fail("me_gemm_bf16_small: unknown gate activation %d", swiglu);
  if (M > 64) return me_fail("me_gemm_bf16_small: M=%d exceeds 64 rows", M);
  if (K <= 0 || K % 8) return me_fail("me_gemm_bf16_small: K=%d must be a positive multiple of 8", K);
  if (norm) {
    if (!x_in || !w_norm) return me_fail("me_gemm_bf16_small: the norm prologue needs x_in and w_norm");
    if (delta && (!x_out || x_out == x_in)) return me_fail("me_gemm_bf16_small: x_out must be given and must not alias x_in");
    if (((uintptr_t)x_in | (uintptr_t)delta | (uintptr_t)w_norm | (uintptr_t)x_out) & 15)
      return me_fail("me_gemm_bf16_small: residual operands must be 16-byte aligned");
  } else if (!X) {
    return me_fail("me_gemm_bf16_small: X is null");
  }
  if (((uintptr_t)X | (uintptr_t)W) & 15) return me_fail("me_gemm_bf16_small: operands must be 16-byte aligned");
  const bf16_t *x = (const bf16_t*)X, *d = (const bf16_t*)delta, *w = (const bf16_t*)W;
  if (out_dtype == ME_F32)
    launch_small<float>(norm, swiglu, x, x_in, d, w_norm, eps, x_out, w, (float*)C, M, N, K, k_splits, rs, stream);
  else
    launch_small<bf16_t>(norm, swiglu, x, x_in, d, w_norm, eps, x_out, w, (bf16_t*)C, M, N, K, 1, rs, stream);
  return me_check_launch("me_gemm_bf16_small");
}

// C[M, N] = epilogue(prologue(input) . W^T).
//   norm == 0: input is X (bfloat16 [M, K]).  norm == 1: input is rmsnorm(x_in + delta) * w_norm, from the
//   float32 residual stream x_in [M, K], delta (bfloat16 [M, K] or null), w_norm float32 [K]; when delta
//   is given, x_in + delta is written to x_out (float32 [M, K], not aliasing x_in).
//   swiglu == 0: W is [N, K].  swiglu == 1 or 2 (MeGate): W is [2 N, K] (gate rows, then up rows), C = act(gate) * up
//   with act silu or tanh-gelu.
//   out_dtype: ME_BF16 or ME_F32. M <= 64, K % 8 == 0, pointers 16-byte aligned.
//   k_splits > 1 (plain float32 products only): k is cut into that many runs of whole chunks of 32, each
//   summed by blocks of its own, and C is [k_splits, M, N]: partial sums for the caller to add up (more
//   blocks for products with few output columns, and each reads only its run of x).
extern "C" int me_gemm_bf16_small(const void* X, const float* x_in, const void* delta, const float* w_norm, float eps,
                                  float* x_out, const void* W, void* C, int M, int N, int K, int norm, int swiglu,
                                  int out_dtype, int k_splits, hipStream_t stream) {
  return small_product(X, x_in, delta, w_norm, eps, x_out, W, C, M, N, K, norm, swiglu, out_dtype, k_splits, RowScale{}, stream);
}

// The plain form (norm == 0, one run of k) with its rows multiplied by rsqrt(sum_b row_ss[m, b] / ss_dim + eps) before
// the gate: the product behind an RMS norm whose division was left to it (row_ss float32 [M, ss_blocks], as
// me_gemm_bf16_stream_carry writes it).
extern "C" int me_gemm_bf16_small_scaled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                                         const float* row_ss, int ss_blocks, int ss_dim, float eps, hipStream_t stream) {
  if (!row_ss || ss_blocks < 1 || ss_dim < 1) return me_fail("me_gemm_bf16_small_scaled: no sums of squares");
  return small_product(X, nullptr, nullptr, nullptr, 0.f, nullptr, W, C, M, N, K, 0, swiglu, out_dtype, 1,
                       RowScale{row_ss, ss_blocks, 1.f / (float)ss_dim, eps}, stream);
}
