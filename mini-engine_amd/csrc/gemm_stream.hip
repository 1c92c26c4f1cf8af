// Skinny bfloat16 product y = x . W^T (M <= 64 rows) for weights so large that the kernel's time is the
// time to stream W from memory once: the projections of models with wide layers, at any decode batch.
//
// A block of four waves owns 16 * WN output columns and all M rows and walks k in steps of 128. The rows of
// x that a step needs are staged once per block in LDS (double-buffered, one barrier per step) and shared
// by the waves, so x is fetched from the L2 once per block of columns instead of once per 16 columns; W goes
// from global memory straight into the registers that feed the matrix cores, STAGES steps ahead of its use
// (what keeps enough loads in flight to stream at the memory's rate). The
// waves are arranged WN x WK: WN groups of 16 columns, WK runs of 128 / WK k within a step, whose partial sums
// are added through LDS at the end. With k_splits > 1 the grid's second dimension cuts k into runs of whole
// steps, each block writing float32 partial sums behind those of the splits before it, for the caller to add
// up (the next residual add does): products with few columns then still fill the chip.
//
// Products use v_mfma_f32_16x16x32_bf16 in the transposed arrangement (C^T[n, m] = sum_k W[n, k] X[m, k]):
// lane l feeds W[n0 + l % 16][8 k] and X[m0 + l % 16][8 k] (k = 32 c + 8 (l / 16) ..) and receives
// C^T[4 (l / 16) .. +4][l % 16]. The SWIGLU form computes 16 gate columns and the 16 matching up columns per
// wave (W = [gate rows; up rows]) and writes silu(gate) * up.
#include "common.h"

typedef __bf16 sbf16x8_t __attribute__((ext_vector_type(8)));
typedef float sfloat4_t __attribute__((ext_vector_type(4)));
typedef uint32_t suint4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int kStepK = 128;          // k per block and step
constexpr int kBufferFlags = 0x00020000;  // a raw buffer of 32-bit words (gfx9 family)
constexpr int kRow = kStepK + 16;    // LDS row stride in elements: 288 bytes, 32 off a multiple of 64 (conflict-free 16-byte reads)

template <int MT, int WN, int WK, bool SWIGLU, typename OutT, int STAGES>
__global__ __launch_bounds__(256) void gemm_stream_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                          OutT* __restrict__ C, int M, int N, int K, int steps_per_split, int gate) {
  static_assert(WN * WK == 4, "four waves per block");
  constexpr int KC = kStepK / WK;  // k per wave and step
  constexpr int CH = KC / 32;      // products per wave, step and tile of rows
  constexpr int ACCS = SWIGLU ? 2 : 1;
  constexpr int XV = MT * 16 * (kStepK / 8) / 256;  // 16-byte vectors of x per thread and step
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][MT * 16][kRow];
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int wn = wave % WN, wk = wave / WN;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = (blockIdx.x * WN + wn) * 16;
  const int n = n0 + r;

  const int total_steps = (K + kStepK - 1) / kStepK;
  const int first = blockIdx.y * steps_per_split;
  const int steps = min(total_steps, first + steps_per_split) - first;
  const int k_end = min(K, (first + steps) * kStepK);  // this block's run of k ends here
  C += (size_t)blockIdx.y * M * N;

  // Loads go through buffer descriptors: an offset at or beyond the buffer's size gives zeros without a
  // branch, which is how rows beyond M or N, k beyond the run and steps beyond the last are handled.
  const uint32_t w_bytes = (uint32_t)((size_t)(SWIGLU ? 2 : 1) * N * K * 2), x_bytes = (uint32_t)((size_t)M * K * 2);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(W), 0, w_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(X), 0, x_bytes, kBufferFlags);
  uint32_t w_base[ACCS];
#pragma unroll
  for (int a = 0; a < ACCS; ++a) w_base[a] = n < N ? (uint32_t)(((SWIGLU && a ? N : 0) + n) * K + wk * KC + g * 8) * 2 : w_bytes;
  uint32_t x_base[XV];  // row m of thread's i-th vector (rows beyond M lie beyond the buffer)
  int x_k[XV];
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    const int v = threadIdx.x + i * 256;
    x_k[i] = (v % (kStepK / 8)) * 8;
    x_base[i] = (uint32_t)((v / (kStepK / 8)) * K + x_k[i]) * 2;
  }

  sfloat4_t acc[MT][ACCS];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int a = 0; a < ACCS; ++a) acc[t][a] = (sfloat4_t){0.f, 0.f, 0.f, 0.f};

  // The weights and the rows of x of the next STAGES steps, in flight or arrived. Both are fetched the same
  // number of steps ahead: loads complete in the order of their issue, so a step that waited for rows of x
  // fetched later than its weights would wait for every weight in flight.
  suint4_t w[STAGES][ACCS][CH], xreg[STAGES][XV];
  auto load_step = [&](int step, suint4_t (&wd)[ACCS][CH], suint4_t (&xd)[XV]) {
    const int k0 = (first + step) * kStepK;
#pragma unroll
    for (int i = 0; i < XV; ++i)
      xd[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, k0 + x_k[i] < k_end ? (int)(x_base[i] + k0 * 2) : (int)x_bytes, 0, 0);
#pragma unroll
    for (int a = 0; a < ACCS; ++a)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int k = k0 + wk * KC + g * 8 + 32 * c;
        wd[a][c] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, k < k_end ? (int)(w_base[a] + (k0 + 32 * c) * 2) : (int)w_bytes, 0, 0);
      }
  };

  // (the scheduling barriers keep the stages' loads in the order of their use: the waits count loads in flight)
#pragma unroll
  for (int p = 0; p < STAGES; ++p) {
    load_step(p, w[p], xreg[p]);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int s0 = 0; s0 < steps; s0 += STAGES) {  // the last round may run up to STAGES - 1 steps of zeros
#pragma unroll
    for (int u = 0; u < STAGES; ++u) {
      const int s = s0 + u, buf = s & 1;
#pragma unroll
      for (int i = 0; i < XV; ++i) {
        const int v = threadIdx.x + i * 256;
        *reinterpret_cast<suint4_t*>(&xs[buf][v / (kStepK / 8)][(v % (kStepK / 8)) * 8]) = xreg[u][i];
      }
      __syncthreads();  // tile s is in LDS; every wave has left tile s - 1, whose buffer step s + 1 writes
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const sbf16x8_t b = *reinterpret_cast<const sbf16x8_t*>(&xs[buf][t * 16 + r][wk * KC + 32 * c + g * 8]);
#pragma unroll
          for (int a = 0; a < ACCS; ++a)
            acc[t][a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sbf16x8_t, w[u][a][c]), b, acc[t][a], 0, 0, 0);
        }
      __builtin_amdgcn_sched_barrier(0);
      load_step(s + STAGES, w[u], xreg[u]);  // the stage is free again: fetch what it holds next
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  if (WK > 1) {  // the runs of k within a step: waves wk > 0 hand their sums to wave wk == 0 of their columns
    __syncthreads();
    float* red = reinterpret_cast<float*>(&xs[0][0][0]);  // [wk - 1][wn][t][a][j][lane]
    constexpr int PER_WAVE = MT * ACCS * 4 * 64;
    static_assert((WK - 1) * WN * PER_WAVE * 4 <= (int)sizeof(xs), "the partial sums fit the x tiles' memory");
    if (wk > 0) {
      float* mine = red + ((wk - 1) * WN + wn) * PER_WAVE;
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int a = 0; a < ACCS; ++a)
#pragma unroll
          for (int j = 0; j < 4; ++j) mine[((t * ACCS + a) * 4 + j) * 64 + lane] = acc[t][a][j];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int o = 1; o < WK; ++o) {
      const float* theirs = red + ((o - 1) * WN + wn) * PER_WAVE;
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int a = 0; a < ACCS; ++a)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[t][a][j] += theirs[((t * ACCS + a) * 4 + j) * 64 + lane];
    }
  }
  // lane (r, g) holds rows m = 16 t + r, columns n0 + 4 g .. +4
  const int nb = n0 + 4 * g;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    if (m >= M) continue;
    float y[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      y[j] = acc[t][0][j];
      if (SWIGLU) y[j] = gate_act(y[j], gate) * acc[t][1][j];
    }
    OutT* dst = C + (size_t)m * N + nb;
    if (nb + 3 < N && (N & 3) == 0) {
      if (sizeof(OutT) == 4) {
        *reinterpret_cast<float4*>(dst) = make_float4(y[0], y[1], y[2], y[3]);
      } else {
        uint2 packed;
        packed.x = (uint32_t)f32_to_bf16_bits(y[0]) | ((uint32_t)f32_to_bf16_bits(y[1]) << 16);
        packed.y = (uint32_t)f32_to_bf16_bits(y[2]) | ((uint32_t)f32_to_bf16_bits(y[3]) << 16);
        *reinterpret_cast<uint2*>(dst) = packed;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (nb + j < N) dst[j] = from_float<OutT>(y[j]);
    }
  }
}

template <int MT, bool SWIGLU, typename OutT>
void launch_arranged(int wn, const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int splits, int steps_per_split,
                     int gate, hipStream_t stream) {
  const dim3 grid(((N + 15) / 16 + wn - 1) / wn, splits);
  if (wn == 4)
    gemm_stream_kernel<MT, 4, 1, SWIGLU, OutT, (SWIGLU ? 2 : 3)><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate);
  else if (wn == 2)
    gemm_stream_kernel<MT, 2, 2, SWIGLU, OutT, (SWIGLU ? 3 : 4)><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate);
  else
    gemm_stream_kernel<MT, 1, 4, SWIGLU, OutT, (SWIGLU ? 4 : 6)><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate);
}

template <bool SWIGLU, typename OutT>
void launch_rows(int wn, const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int splits, int steps_per_split,
                 int gate, hipStream_t stream) {
  switch ((M + 15) / 16) {
    case 1: launch_arranged<1, SWIGLU, OutT>(wn, X, W, C, M, N, K, splits, steps_per_split, gate, stream); break;
    case 2: launch_arranged<2, SWIGLU, OutT>(wn, X, W, C, M, N, K, splits, steps_per_split, gate, stream); break;
    case 3: launch_arranged<3, SWIGLU, OutT>(wn, X, W, C, M, N, K, splits, steps_per_split, gate, stream); break;
    default: launch_arranged<4, SWIGLU, OutT>(wn, X, W, C, M, N, K, splits, steps_per_split, gate, stream); break;
  }
}

}  // namespace

// How many columns' worth of waves a block gets (4, 2 or 1 groups of 16 columns; the other waves cut k): the
// widest arrangement that still gives the chip enough blocks, since wider blocks fetch x less often. Up to 16
// rows x is small and two blocks per compute unit stream best; with more rows the fetches of x weigh more and
// half a block per compute unit is enough (measured at 32 and 64 rows, 6,144 to 25,600 columns: 16-53 us with
// this rule against 21-63 with the other).
extern "C" int me_gemm_bf16_stream_arrangement(int M, int N, int k_splits, int compute_units) {
  const int tiles = (N + 15) / 16;
  const long long want = M <= 16 ? 2ll * compute_units : compute_units / 2;
  for (int wn = 4; wn > 1; wn >>= 1)
    if ((long long)((tiles + wn - 1) / wn) * k_splits >= want) return wn;
  return 1;
}

// Into how many runs of k a product whose result may stay partial sums is cut: blocks of 64 columns, as many runs
// as give every compute unit about two blocks, each of at least four steps of 128.
extern "C" int me_gemm_bf16_stream_splits(int N, int K, int compute_units) {
  const int blocks = ((N + 15) / 16 + 3) / 4;
  const int steps = (K + kStepK - 1) / kStepK;
  const int want = max(1, min(min((2 * compute_units + blocks - 1) / blocks, steps / 4), 16));
  const int steps_per_split = (steps + want - 1) / want;
  return (steps + steps_per_split - 1) / steps_per_split;  // no empty run
}

// C[M, N] = x . W^T (swiglu 1 or 2, a MeGate code: W is [2 N, K], gate rows then up rows, and C = act(gate) * up), X bfloat16 [M, K],
// M <= 64, K % 8 == 0, pointers 16-byte aligned. out_dtype ME_BF16 or ME_F32. k_splits > 1 (plain float32
// products only): C is [k_splits, M, N], partial sums over runs of k for the caller to add up.
extern "C" int me_gemm_bf16_stream(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                                   int k_splits, int compute_units, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (swiglu < ME_GATE_NONE || swiglu > ME_GATE_GELU_TANH) return me_fail("me_gemm_bf16_stream: unknown gate activation %d", swiglu);
  if (M > 64) return me_fail("me_gemm_bf16_stream: M=%d exceeds 64 rows", M);
  if (K <= 0 || K % 8) return me_fail("me_gemm_bf16_stream: K=%d must be a positive multiple of 8", K);
  if (!X || !W || !C) return me_fail("me_gemm_bf16_stream: null operand");
  if (((uintptr_t)X | (uintptr_t)W | (uintptr_t)C) & 15) return me_fail("me_gemm_bf16_stream: operands must be 16-byte aligned");
  if (out_dtype != ME_BF16 && out_dtype != ME_F32) return me_fail("me_gemm_bf16_stream: output type %d", out_dtype);
  if (k_splits < 1 || k_splits > 64) return me_fail("me_gemm_bf16_stream: %d splits of k", k_splits);
  if (k_splits > 1 && (swiglu || out_dtype != ME_F32))
    return me_fail("me_gemm_bf16_stream: partial sums over splits of k are plain float32 products");
  if (swiglu && out_dtype != ME_BF16) return me_fail("me_gemm_bf16_stream: the gated form writes bfloat16");
  if ((size_t)(swiglu ? 2 : 1) * N * K * 2 >= (1ull << 31) || (size_t)M * K * 2 >= (1ull << 31))
    return me_fail("me_gemm_bf16_stream: operands of 2 GiB and more are not addressed by this kernel");
  if (compute_units < 1) compute_units = 256;
  const int steps = (K + kStepK - 1) / kStepK;
  const int steps_per_split = (steps + k_splits - 1) / k_splits;
  const int splits = (steps + steps_per_split - 1) / steps_per_split;  // no empty run
  if (splits != k_splits) return me_fail("me_gemm_bf16_stream: K=%d cannot be cut into %d runs of whole steps", K, k_splits);
  const int wn = me_gemm_bf16_stream_arrangement(M, N, splits, compute_units);
  const bf16_t *x = (const bf16_t*)X, *w = (const bf16_t*)W;
  if (swiglu)
    launch_rows<true, bf16_t>(wn, x, w, (bf16_t*)C, M, N, K, splits, steps_per_split, swiglu, stream);
  else if (out_dtype == ME_F32)
    launch_rows<false, float>(wn, x, w, (float*)C, M, N, K, splits, steps_per_split, 0, stream);
  else
    launch_rows<false, bf16_t>(wn, x, w, (bf16_t*)C, M, N, K, splits, steps_per_split, 0, stream);
  return me_check_launch("me_gemm_bf16_stream");
}
