// Skinny bfloat16 product y = x . W^T (M <= 64 rows a block; up to 256 rows in groups of 64, the grid's third
// dimension) for weights so large that the kernel's time is the time to stream W from memory once: the projections
// of models with wide layers, at any decode batch.
//
// A block of four waves owns 16 * WN output columns and all M rows and walks k in steps of 128. The rows of
// x that a step needs are staged once per block in LDS (double-buffered, one barrier per step) and shared
// by the waves, so x is fetched from the L2 once per block of columns instead of once per 16 columns; W goes
// from global memory straight into the registers that feed the matrix cores, STAGES steps ahead of its use
// (what keeps enough loads in flight to stream at the memory's rate). The
// waves are arranged WN x WK: WN groups of 16 columns, WK runs of 128 / WK k within a step, whose partial sums
// are added through LDS at the end. With k_splits > 1 the grid's second dimension cuts k into runs of whole
// steps, each block writing float32 partial sums behind those of the splits before it, for the caller to add
// up (the next residual add does): products with few columns then still fill the chip. The grid's first dimension
// deals the columns out in fours, as evenly as they go: the host picks arrangement, runs and blocks so that the launch
// is whole rounds of the compute units where it can (plan_for_runs, plan_with_runs below).
//
// Two forms for a norm carried from a product to the next (common.h), instances of their own (AUX): a plain product of one
// run of k that is a delta of the residual stream adds its columns to the stream in its epilogue and leaves bf16(x * w_norm)
// and its part of the rows' sums of squares (me_gemm_bf16_stream_carry); a product multiplies its rows by
// rsqrt(sum / dim + eps), with the sums read at its head and added up behind its loop (me_gemm_bf16_stream_scaled).
//
// Products use v_mfma_f32_16x16x32_bf16 in the transposed arrangement (C^T[n, m] = sum_k W[n, k] X[m, k]):
// lane l feeds W[n0 + l % 16][8 k] and X[m0 + l % 16][8 k] (k = 32 c + 8 (l / 16) ..) and receives
// C^T[4 (l / 16) .. +4][l % 16]. The SWIGLU form computes 16 gate columns and the 16 matching up columns per
// wave (W = [gate rows; up rows]) and writes silu(gate) * up.
#include "common.h"

#include <algorithm>

typedef __bf16 sbf16x8_t __attribute__((ext_vector_type(8)));
typedef float sfloat4_t __attribute__((ext_vector_type(4)));
typedef uint32_t suint4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int kStepK = 128;          // k per block and step
constexpr int kGroupRows = 64;       // rows per block; more rows are dealt to groups of blocks (the grid's third dimension)
constexpr int kMaxRows = 256;
constexpr int kBufferFlags = 0x00020000;  // a raw buffer of 32-bit words (gfx9 family)
// How the grid's first dimension deals the columns out, in fours, as evenly as they go: block b takes `q` fours, the first
// `r` blocks one more. Worked out on the host: the same from blockIdx and gridDim by division cost every block some four
// hundred scalar instructions before it could ask for its first weights. `rotate`: whether a block walks k from a step of
// its own.
struct ColumnDeal {
  int q, r, rotate;
};
__device__ __forceinline__ int deal_first(const ColumnDeal& d, int b) { return (b * d.q + min(b, d.r)) * 4; }
inline ColumnDeal deal_of(int N, int grid, bool rotate) {
  const int fours = (N + 3) / 4;
  return {fours / grid, fours % grid, rotate ? 1 : 0};
}
// (no division either: a multiplicative hash of the block's number, scaled to [0, steps))
__device__ __forceinline__ int deal_turn(unsigned b, int steps) {
  return (int)((((b * 0x9E3779B1u) >> 16) * (unsigned)steps) >> 16);
}

constexpr int kRow = kStepK + 16;    // LDS row stride in elements: 288 bytes, 32 off a multiple of 64 (conflict-free 16-byte reads)

template <int MT, int WN, int WK, bool SWIGLU, typename OutT, int STAGES, int NT = 1, bool AUX = false>
__global__ __launch_bounds__(256) void gemm_stream_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                          OutT* __restrict__ C, int rows, int N, int K, int steps_per_split, int gate,
                                                          ColumnDeal deal, RowScale rs, CarryOut carry) {
  static_assert(WN * WK == 4, "four waves per block");
  static_assert(NT == 1 || WK == 1, "waves with several tiles of columns do not cut k");
  // The grid's third dimension deals the rows out in groups of 16 MT; a block sees its group's rows only.
  C += (size_t)blockIdx.y * rows * N + (size_t)blockIdx.z * (16 * MT) * N;
  X += (size_t)blockIdx.z * (16 * MT) * K;
  const int M = min(16 * MT, rows - (int)blockIdx.z * 16 * MT);
  constexpr int KC = kStepK / WK;  // k per wave and step
  constexpr int CH = KC / 32;      // products per wave, step, tile of rows and tile of columns
  constexpr int ACCS = (SWIGLU ? 2 : 1) * NT;  // tiles of 16 columns per wave: NT of them, gate and up of each in the gated form
  constexpr int XV = MT * 16 * (kStepK / 8) / 256;  // 16-byte vectors of x per thread and step
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][MT * 16][kRow];
  __shared__ float row_scale[AUX ? MT * 16 : 1];  // with rs.ss: what the rows are multiplied by at the end
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int wn = wave % WN, wk = wave / WN;
  const int r = lane & 15, g = lane >> 4;
  float ss_part[MT * 4];  // the rows whose scale this wave works out: loads here, the sums behind the loop over k
  if (AUX && rs.ss) {
    rs.ss += (size_t)blockIdx.z * (16 * MT) * rs.blocks;
    row_ss_fetch<MT * 4>(rs, M, ss_part, wave, lane, 4);
  }
  // The block's columns: the grid deals N out in fours, as evenly as they go (a grid of N / (16 WN NT) blocks gives every
  // block 16 WN NT columns; a larger one gives each fewer, and the rest of its last tile of 16 is neither fetched nor stored).
  const int c0 = deal_first(deal, blockIdx.x);
  const int c1 = min(N, deal_first(deal, blockIdx.x + 1));
  const int n0 = c0 + wn * NT * 16;  // the wave's first tile; tile i begins 16 i columns on

  const int total_steps = (K + kStepK - 1) / kStepK;
  const int first = blockIdx.y * steps_per_split;
  const int steps = min(total_steps, first + steps_per_split) - first;
  const int k_end = min(K, (first + steps) * kStepK);  // this block's run of k ends here

  // Loads go through buffer descriptors: an offset at or beyond the buffer's size gives zeros without a
  // branch, which is how rows beyond M or N, k beyond the run and steps beyond the last are handled.
  const uint32_t w_bytes = (uint32_t)((size_t)(SWIGLU ? 2 : 1) * N * K * 2), x_bytes = (uint32_t)((size_t)M * K * 2);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(W), 0, w_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(X), 0, x_bytes, kBufferFlags);
  uint32_t w_base[ACCS];  // accumulator a: tile a % NT of the wave, its up rows if a >= NT
#pragma unroll
  for (int a = 0; a < ACCS; ++a) {
    const int n = n0 + (a % NT) * 16 + r;
    w_base[a] = n < c1 ? (uint32_t)(((a >= NT ? N : 0) + n) * K + wk * KC + g * 8) * 2 : w_bytes;
  }
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
  // With `rotate` a block walks its steps of k from a step of its own on, around the end of its run: the blocks that start
  // together then read different memory channels (rows of W that lie a multiple of 4 KiB apart begin in the same one).
  const int rot = deal.rotate ? deal_turn(blockIdx.x * 5u + blockIdx.z, steps) : 0;
  auto load_step = [&](int step, suint4_t (&wd)[ACCS][CH], suint4_t (&xd)[XV]) {
    int turned = step + rot;
    if (turned >= steps) turned -= steps;
    const int k0 = (first + (step < steps ? turned : steps)) * kStepK;  // (steps past the run: beyond its end, nothing is fetched)
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

  // A delta that adds itself to the stream (carry.x): the elements of the stream and of the norm's weight that this lane
  // will add to and multiply with at the end are requested here, ahead of everything, so that the kernel's tail does not
  // wait for memory once more. (Whole groups of four columns only; a ragged edge is read at the end.)
  // With as many tiles of rows as runs of k within a step (or a multiple), every wave finishes the tiles t with
  // t % WK == wk: it hands the sums of the other tiles to their waves and adds up what they hand to it, so that the
  // sums, the gate and the stores of a block of 64 rows are four waves' work and not one's.
  constexpr bool SHARE_TAIL = WK > 1 && MT > 1 && MT % WK == 0;
  float4 x_early[AUX ? MT : 1][AUX ? NT : 1], wn_early[AUX ? NT : 1];
  if constexpr (AUX && !SWIGLU && sizeof(OutT) == 4) {
    if (carry.x && (SHARE_TAIL || wk == 0) && (N & 3) == 0) {
      const size_t row0 = (size_t)blockIdx.z * (16 * MT);
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int nb = n0 + 16 * i + 4 * g;
        if (nb < c1 && nb + 3 < N) {
          wn_early[i] = *reinterpret_cast<const float4*>(carry.w_norm + nb);
#pragma unroll
          for (int t = 0; t < MT; ++t)
            if ((!SHARE_TAIL || t % WK == wk) && t * 16 + r < M)
              x_early[t][i] = *reinterpret_cast<const float4*>(carry.x + (row0 + t * 16 + r) * N + nb);
        }
      }
    }
  }
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

  if (AUX && rs.ss) {
    row_scales_finish<MT * 4>(rs, M, ss_part, row_scale, wave, lane, 4);
    __syncthreads();
  }
  if constexpr (SHARE_TAIL) {
    __syncthreads();
    float* red = reinterpret_cast<float*>(&xs[0][0][0]);  // [wk][wn][t][a][j][lane]
    constexpr int PER_WAVE = MT * ACCS * 4 * 64;
    static_assert(WK * WN * PER_WAVE * 4 <= (int)sizeof(xs), "the partial sums fit the x tiles' memory");
    float* mine = red + (wk * WN + wn) * PER_WAVE;
#pragma unroll
    for (int t = 0; t < MT; ++t)
      if (t % WK != wk)
#pragma unroll
        for (int a = 0; a < ACCS; ++a)
#pragma unroll
          for (int j = 0; j < 4; ++j) mine[((t * ACCS + a) * 4 + j) * 64 + lane] = acc[t][a][j];
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t)
      if (t % WK == wk)
#pragma unroll
        for (int o = 0; o < WK; ++o)
          if (o != wk) {
            const float* theirs = red + (o * WN + wn) * PER_WAVE;
#pragma unroll
            for (int a = 0; a < ACCS; ++a)
#pragma unroll
              for (int j = 0; j < 4; ++j) acc[t][a][j] += theirs[((t * ACCS + a) * 4 + j) * 64 + lane];
          }
  } else if (WK > 1) {  // the runs of k within a step: waves wk > 0 hand their sums to wave wk == 0 of their columns
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
  // lane (r, g) holds rows m = 16 t + r, columns 4 g .. +4 of each of its tiles
  if constexpr (AUX && !SWIGLU && sizeof(OutT) == 4) {
    if (carry.x) {
      // The product is a delta of the residual stream and this block has all of k: x += delta, h = bf16(x * w_norm)
      // and the sums of squares of the rows over the wave's columns, for the product behind the norm.
      const size_t row0 = (size_t)blockIdx.z * (16 * MT);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (SHARE_TAIL && t % WK != wk) continue;
        const int m = t * 16 + r;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          const int nb = n0 + 16 * i + 4 * g;
          if (m < M && nb < c1) {
            float* xp = carry.x + (row0 + m) * N + nb;
            bf16_t* hp = carry.h + (row0 + m) * N + nb;
            if (nb + 3 < N && (N & 3) == 0) {
              float4 v = x_early[t][i];
              const float4 wv = wn_early[i];
              v.x += acc[t][i][0], v.y += acc[t][i][1], v.z += acc[t][i][2], v.w += acc[t][i][3];
              *reinterpret_cast<float4*>(xp) = v;
              uint2 packed;
              packed.x = (uint32_t)f32_to_bf16_bits(v.x * wv.x) | ((uint32_t)f32_to_bf16_bits(v.y * wv.y) << 16);
              packed.y = (uint32_t)f32_to_bf16_bits(v.z * wv.z) | ((uint32_t)f32_to_bf16_bits(v.w * wv.w) << 16);
              *reinterpret_cast<uint2*>(hp) = packed;
              sq = fmaf(v.x, v.x, sq), sq = fmaf(v.y, v.y, sq), sq = fmaf(v.z, v.z, sq), sq = fmaf(v.w, v.w, sq);
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (nb + j < N) {
                  const float v = xp[j] + acc[t][i][j];
                  xp[j] = v;
                  hp[j] = from_float<bf16_t>(v * carry.w_norm[nb + j]);
                  sq = fmaf(v, v, sq);
                }
            }
          }
        }
        sq += __shfl_xor(sq, 16, ME_WAVE);  // the four lanes of a row
        sq += __shfl_xor(sq, 32, ME_WAVE);
        if (g == 0 && m < M) carry.ss[(row0 + m) * carry.blocks + blockIdx.x * WN + wn] = sq;
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int nb = n0 + 16 * i + 4 * g;
    if (nb >= c1) continue;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      if (SHARE_TAIL && t % WK != wk) continue;
      const int m = t * 16 + r;
      if (m >= M) continue;
      const float scale = AUX && rs.ss ? row_scale[m] : 1.f;
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        y[j] = acc[t][i][j] * scale;
        if (SWIGLU) y[j] = gate_act_bf16(y[j], gate) * (acc[t][NT + i][j] * scale);
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
}

// The prologue of the kernel below works on ROWS rows at a time and on four consecutive elements of each per thread:
// s = x_in + delta or + the partial sums, in the order of their runs. What it reads of the first PB runs is requested in
// one go (norm_fetch), and for the thread's first elements before the kernel's first weights: loads complete in the order
// of their issue, so a prologue that asked for its rows behind the weights waited for all of those, and one that asked
// for four runs at a time and for one row after the other took a trip to memory for each (a second row cost the kernel
// 2.3 us, sixteen runs instead of four 0.8). A run beyond the last reads the last one again and counts for nothing; so
// does a row beyond the last.
template <int ROWS, int PB>
struct NormLoads {
  float4 sv[ROWS], wv, pv[PB][ROWS];
  uint2 dv[ROWS];
};

template <int ROWS, int PB>
__device__ __forceinline__ void norm_fetch(NormLoads<ROWS, PB>& ld, const float* __restrict__ x_in, const bf16_t* __restrict__ delta,
                                           const float* __restrict__ parts, int num_parts, size_t part_stride,
                                           const float* __restrict__ w_norm, int m0, int M, int K, int v) {
#pragma unroll
  for (int j = 0; j < ROWS; ++j) {
    const size_t at = (size_t)min(m0 + j, M - 1) * K + 4 * v;
    ld.sv[j] = *reinterpret_cast<const float4*>(x_in + at);
    ld.dv[j] = make_uint2(0, 0);
    if (delta) ld.dv[j] = *reinterpret_cast<const uint2*>(delta + at);
  }
  ld.wv = *reinterpret_cast<const float4*>(w_norm + 4 * v);
  if (parts) {
#pragma unroll
    for (int i = 0; i < PB; ++i)
#pragma unroll
      for (int j = 0; j < ROWS; ++j)
        ld.pv[i][j] = *reinterpret_cast<const float4*>(parts + (size_t)min(i, num_parts - 1) * part_stride +
                                                       (size_t)min(m0 + j, M - 1) * K + 4 * v);
  }
}

// The rows' sums from what norm_fetch brought (and from the runs beyond the first PB), their squares into ss, the sums
// themselves to x_out if given, bf16(s * w_norm) into xn.
template <int ROWS, int PB>
__device__ __forceinline__ void norm_finish(const NormLoads<ROWS, PB>& ld, const bf16_t* __restrict__ delta,
                                            const float* __restrict__ parts, int num_parts, size_t part_stride,
                                            float* __restrict__ x_out, uint16_t* xn, float (&ss)[ROWS], int m0, int M, int K, int krow,
                                            int v) {
#pragma unroll
  for (int j = 0; j < ROWS; ++j) {
    if (m0 + j >= M) break;
    const size_t at = (size_t)(m0 + j) * K + 4 * v;
    float4 t = ld.sv[j];
    if (delta) {
      t.x += __uint_as_float(ld.dv[j].x << 16), t.y += __uint_as_float(ld.dv[j].x & 0xffff0000u);
      t.z += __uint_as_float(ld.dv[j].y << 16), t.w += __uint_as_float(ld.dv[j].y & 0xffff0000u);
    }
    if (parts) {
      float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int i = 0; i < PB; ++i) {
        const float on = i < num_parts ? 1.f : 0.f;
        d.x += on * ld.pv[i][j].x, d.y += on * ld.pv[i][j].y, d.z += on * ld.pv[i][j].z, d.w += on * ld.pv[i][j].w;
      }
      for (int q = PB; q < num_parts; ++q) {
        const float4 a = *reinterpret_cast<const float4*>(parts + (size_t)q * part_stride + at);
        d.x += a.x, d.y += a.y, d.z += a.z, d.w += a.w;
      }
      t.x += d.x, t.y += d.y, t.z += d.z, t.w += d.w;
    }
    if (x_out) *reinterpret_cast<float4*>(x_out + at) = t;
    ss[j] = fmaf(t.x, t.x, ss[j]), ss[j] = fmaf(t.y, t.y, ss[j]), ss[j] = fmaf(t.z, t.z, ss[j]), ss[j] = fmaf(t.w, t.w, ss[j]);
    uint2 packed;
    packed.x = (uint32_t)f32_to_bf16_bits(t.x * ld.wv.x) | ((uint32_t)f32_to_bf16_bits(t.y * ld.wv.y) << 16);
    packed.y = (uint32_t)f32_to_bf16_bits(t.z * ld.wv.z) | ((uint32_t)f32_to_bf16_bits(t.w * ld.wv.w) << 16);
    *reinterpret_cast<uint2*>(xn + (size_t)(m0 + j) * krow + 4 * v) = packed;
  }
}

// The same product for a row or a few with the residual add and the RMSNorm in front of it as its prologue:
// the input is the float32 residual stream x_in [M, K] plus a delta (a bfloat16 tensor, or float32 partial sums
// of the product before, added in the order of their runs, or nothing). While the weights of the first steps
// are on their way, the block forms s = x_in + delta, keeps bf16(s * w_norm) of every row in LDS for the whole
// of k (no rows of x are fetched in the loop) and sums s^2; the results are multiplied by
// rsqrt(mean(s^2) + eps) at the end (a row's scale is a common factor of its products). Block 0 writes s to
// x_out, which must not alias x_in: the other blocks still read it. Every block reads all of x_in and the partial
// sums, so this is for a row or two; no runs of k across blocks.
template <int WN, int WK, bool SWIGLU, typename OutT, int STAGES, int ROWS, int PB>
__device__ __forceinline__ void gemm_stream_norm_body(const float* __restrict__ x_in, const bf16_t* __restrict__ delta,
                                                      const float* __restrict__ parts, int num_parts, size_t part_stride,
                                                      const float* __restrict__ w_norm, float eps, float* __restrict__ x_out,
                                                      const bf16_t* __restrict__ W, OutT* __restrict__ C, int M, int N, int K,
                                                      int gate, ColumnDeal deal) {
  static_assert(WN * WK == 4, "four waves per block");
  constexpr int KC = kStepK / WK, CH = KC / 32, ACCS = SWIGLU ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char norm_lds[];
  const int krow = K + 8;  // elements per row of normed x: rows start 16 bytes apart modulo the banks
  uint16_t* xn = reinterpret_cast<uint16_t*>(norm_lds);                                  // [M][krow]
  float* sums = reinterpret_cast<float*>(norm_lds + (((size_t)M * krow * 2 + 15) & ~(size_t)15));  // [M][4 waves], then [M]
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int wn = wave % WN, wk = wave / WN;
  const int r = lane & 15, g = lane >> 4;
  // The block's columns: the grid deals N out in fours, as evenly as they go (a grid of N / (16 WN) blocks gives every
  // block 16 WN columns; a larger one gives each fewer, and the rest of its last tile of 16 is neither fetched nor stored).
  const int c0 = deal_first(deal, blockIdx.x);
  const int c1 = min(N, deal_first(deal, blockIdx.x + 1));
  const int n0 = c0 + wn * 16;
  const int n = n0 + r;
  const int steps = (K + kStepK - 1) / kStepK;

  const uint32_t w_bytes = (uint32_t)((size_t)(SWIGLU ? 2 : 1) * N * K * 2);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(W), 0, w_bytes, kBufferFlags);
  uint32_t w_base[ACCS];
#pragma unroll
  for (int a = 0; a < ACCS; ++a) w_base[a] = n < c1 ? (uint32_t)(((SWIGLU && a ? N : 0) + n) * K + wk * KC + g * 8) * 2 : w_bytes;
  suint4_t w[STAGES][ACCS][CH];
  // (with `rotate` the block's walk over k starts at a step of its own and goes around the end, as in the kernel above)
  const int rot = deal.rotate ? deal_turn(blockIdx.x * 5u, steps) : 0;
  auto turned = [&](int step) { return step + rot < steps ? step + rot : step + rot - steps; };
  auto load_step = [&](int step, suint4_t (&wd)[ACCS][CH]) {
    const int k0 = (step < steps ? turned(step) : steps) * kStepK;  // (steps past the end: beyond K, nothing is fetched)
#pragma unroll
    for (int a = 0; a < ACCS; ++a)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int k = k0 + wk * KC + g * 8 + 32 * c;
        wd[a][c] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, k < K ? (int)(w_base[a] + (k0 + 32 * c) * 2) : (int)w_bytes, 0, 0);
      }
  };
  // ---- the prologue: every row's sum, its squares, and bf16(s * w_norm) into LDS. What the thread's first elements need
  // is asked for before the weights.
  float* const x_to = blockIdx.x == 0 && (delta != nullptr || parts != nullptr) ? x_out : nullptr;
  NormLoads<ROWS, PB> ld;
  norm_fetch<ROWS, PB>(ld, x_in, delta, parts, num_parts, part_stride, w_norm, 0, M, K, min((int)threadIdx.x, K / 4 - 1));
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int p = 0; p < STAGES; ++p) {
    load_step(p, w[p]);
    __builtin_amdgcn_sched_barrier(0);
  }
  bool fetched = true;
  for (int m0 = 0; m0 < M; m0 += ROWS) {
    float ss[ROWS];
#pragma unroll
    for (int j = 0; j < ROWS; ++j) ss[j] = 0.f;
    for (int v = threadIdx.x; v < K / 4; v += 256) {
      if (!fetched) norm_fetch<ROWS, PB>(ld, x_in, delta, parts, num_parts, part_stride, w_norm, m0, M, K, v);
      fetched = false;
      norm_finish<ROWS, PB>(ld, delta, parts, num_parts, part_stride, x_to, xn, ss, m0, M, K, krow, v);
    }
#pragma unroll
    for (int j = 0; j < ROWS; ++j) {
      if (m0 + j >= M) break;
      const float total = wave_sum(ss[j]);
      if (lane == 0) sums[(m0 + j) * 4 + wave] = total;
    }
  }
  __syncthreads();
  // rows beyond M read row M - 1 and count for nothing: their results are never stored
  const uint16_t* xrow = xn + (size_t)min(r, M - 1) * krow + wk * KC + g * 8;

  sfloat4_t acc[ACCS];
#pragma unroll
  for (int a = 0; a < ACCS; ++a) acc[a] = (sfloat4_t){0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < steps; s0 += STAGES) {  // the last round may run up to STAGES - 1 steps of zero weights
#pragma unroll
    for (int u = 0; u < STAGES; ++u) {
      const int k0 = turned(min(s0 + u, steps - 1)) * kStepK;  // (steps past the end multiply zero weights with some step's rows)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        sbf16x8_t b = sbf16x8_t{};
        if (k0 + wk * KC + 32 * c + g * 8 < K) b = *reinterpret_cast<const sbf16x8_t*>(xrow + k0 + 32 * c);
#pragma unroll
        for (int a = 0; a < ACCS; ++a)
          acc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sbf16x8_t, w[u][a][c]), b, acc[a], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      load_step(s0 + u + STAGES, w[u]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  if (WK > 1) {  // the runs of k within a step: waves wk > 0 hand their sums to wave wk == 0 of their columns
    __syncthreads();  // every wave has left the rows of x, whose memory the sums take
    float* red = reinterpret_cast<float*>(norm_lds) + 64;  // [wk - 1][wn][a][j][lane], behind the rows' sums of squares
    float* keep = reinterpret_cast<float*>(norm_lds);      // [M][4]
    if (threadIdx.x < M * 4) keep[threadIdx.x] = sums[threadIdx.x];  // (M <= 16; read before, written after a barrier)
    constexpr int PER_WAVE = ACCS * 4 * 64;
    __syncthreads();
    sums = keep;
    if (wk > 0) {
      float* mine = red + ((wk - 1) * WN + wn) * PER_WAVE;
#pragma unroll
      for (int a = 0; a < ACCS; ++a)
#pragma unroll
        for (int j = 0; j < 4; ++j) mine[(a * 4 + j) * 64 + lane] = acc[a][j];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int o = 1; o < WK; ++o) {
      const float* theirs = red + ((o - 1) * WN + wn) * PER_WAVE;
#pragma unroll
      for (int a = 0; a < ACCS; ++a)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[a][j] += theirs[(a * 4 + j) * 64 + lane];
    }
  }
  const int m = r, nb = n0 + 4 * g;
  if (m >= M) return;
  const float scale = rsqrtf(((sums[m * 4] + sums[m * 4 + 1]) + (sums[m * 4 + 2] + sums[m * 4 + 3])) / (float)K + eps);
  float y[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    y[j] = acc[0][j] * scale;
    if (SWIGLU) y[j] = gate_act_bf16(y[j], gate) * (acc[1][j] * scale);
  }
  OutT* dst = C + (size_t)m * N + nb;
  if (nb >= c1) return;
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

// One row: up to sixteen runs of partial sums in the prologue's first request; more rows: two at a time, eight runs.
template <int WN, int WK, bool SWIGLU, typename OutT, int STAGES>
__global__ __launch_bounds__(256) void gemm_stream_norm_kernel(const float* __restrict__ x_in, const bf16_t* __restrict__ delta,
                                                               const float* __restrict__ parts, int num_parts, size_t part_stride,
                                                               const float* __restrict__ w_norm, float eps, float* __restrict__ x_out,
                                                               const bf16_t* __restrict__ W, OutT* __restrict__ C, int M, int N,
                                                               int K, int gate, ColumnDeal deal) {
#define ME_NORM_BODY(ROWS, PB)                                                                                                  \
  gemm_stream_norm_body<WN, WK, SWIGLU, OutT, STAGES, ROWS, PB>(x_in, delta, parts, num_parts, part_stride, w_norm, eps, x_out, W, C, \
                                                                M, N, K, gate, deal)
  if (M == 1) {
    if (num_parts <= 4)
      ME_NORM_BODY(1, 4);
    else if (num_parts <= 8)
      ME_NORM_BODY(1, 8);
    else
      ME_NORM_BODY(1, 16);
  } else {
    ME_NORM_BODY(2, 8);
  }
#undef ME_NORM_BODY
}

// How a product is laid over the chip: the waves' arrangement (wn groups of 16 columns, 4 / wn runs of k within a
// step), the runs of k across blocks, and the blocks along the columns.
struct StreamPlan {
  int wn, splits, grid, nt;  // nt: tiles of 16 columns per wave
};

// A compute unit streams at a fixed rate, so a product takes as long as the unit with the most blocks: the blocks
// along the columns are as many as there are runs of 16 wn columns, or up to a third more if the launch then is whole
// rounds of the compute units, or just short of them (every block then has fewer columns, all about as many).
int whole_rounds(int base, int splits, int compute_units) {
  const long long rounds = ((long long)base * splits + compute_units - 1) / compute_units;
  const long long grid = rounds * compute_units / splits;
  return grid >= base && 3 * grid <= 4ll * base ? (int)grid : base;
}

int runs_of(int steps, int want) {  // `want` runs of whole steps, none empty
  const int per = (steps + want - 1) / want;
  return (steps + per - 1) / per;
}

// A product with a given number of runs of k (one, for a result that is no partial sum). Up to 16 rows, where x is
// small: the widest arrangement whose blocks fill whole rounds of the compute units, two rounds for the gated form, which
// keeps half as many steps in flight per wave (measured, weights of 8 to 524 MB; 6,144 x 4,096 at one row: 12.0 us
// with 256 blocks of two tiles against 15.4 with 384 of one; the gated 2 x 25,600 x 5,120: 96 us with 512 blocks of 50
// columns, 109 with 400 of 64), else the widest one with two blocks per unit. With more rows the fetches of x weigh
// more than an uneven round (10,240 x 5,120 at 64 rows: 41 us with 160 blocks of 64 columns, 54 with 768 of 16): the
// widest arrangement with half a block per unit.
StreamPlan plan_for_runs(int M, int N, bool gated, int splits, int compute_units) {
  const int tiles = (N + 15) / 16;
  const int least_rounds = gated ? 2 : 1;
  const int groups = (M + kGroupRows - 1) / kGroupRows;  // the same blocks once per group of 64 rows
  const int across = splits * groups;
  for (int wn = 4; wn >= 1 && M <= 16; wn >>= 1) {
    const int base = (tiles + wn - 1) / wn, grid = whole_rounds(base, splits, compute_units);
    const long long total = (long long)grid * splits, rounds = (total + compute_units - 1) / compute_units;
    if (rounds >= least_rounds && total * 16 >= rounds * compute_units * 15) return {wn, splits, grid, 1};
  }
  const long long want = M <= 16 ? 2ll * compute_units : compute_units / 2;
  int wn = 4;
  while (wn > 1 && (long long)((tiles + wn - 1) / wn) * across < want) wn >>= 1;
  return {wn, splits, whole_rounds((tiles + wn - 1) / wn, across, compute_units), 1};
}

// A product whose result may stay partial sums over runs of k: the widest arrangement that, with k cut into runs of
// at least four steps (16 runs at most), gives about one block per compute unit, at least half as many (measured: 4,096 x
// 12,288 at one row: 19.8 us with 4 runs of 64 blocks of 64 columns against 21.3 with 8 runs of 256 blocks of 16;
// 5,120 x 25,600: 46 against 51; at 64 rows 65 against 71; 1,024 x 3,072: 4.5-5.0 against 5.2). With more than 32 rows
// a block of 64 columns fetches as many bytes of x as of weights; blocks of 128 columns, two tiles a wave, fetch half as
// many, but need twice the runs of k to fill the chip, so they are taken where the partial sums of those runs stay small
// beside the weights (32 x runs x rows <= k: the add-and-norm behind the product reads them too; at 64 rows 5,120 x
// 25,600: 60 us against 70 and a decode step of that shape 2.4% shorter; 4,096 x 12,288: 27.4 against 30.3 and no gain
// in the step; 4,096 x 4,096, whose 8 runs write half as many bytes as the weights have: 11.8 against 11.3).
StreamPlan plan_with_runs(int M, int N, int K, int compute_units) {
  const int tiles = (N + 15) / 16, steps = (K + kStepK - 1) / kStepK;
  const int most = std::max(1, std::min(steps / 4, 16));
  const int groups = (M + kGroupRows - 1) / kGroupRows;  // the same blocks once per group of 64 rows
  for (int width = (M > 32 ? 8 : 4); width >= 1; width >>= 1) {  // tiles of 16 columns per block
    const int base = (tiles + width - 1) / width * groups;
    const int splits = runs_of(steps, std::max(1, std::min(most, (compute_units + base / 2) / base)));
    if (width == 8 && 32ll * splits * std::min(M, kGroupRows) > K) continue;
    if (2ll * base * splits >= compute_units || width == 1)
      return {std::min(width, 4), splits, whole_rounds(base / groups, splits * groups, compute_units), width / std::min(width, 4)};
  }
  return {1, 1, tiles, 1};  // (not reached)
}

// A delta that adds itself to the residual stream: every block walks all of k for a tile of 16 columns, four waves sharing k
// within a step. (Narrower blocks, so that the launch goes round more compute units, are no faster: every block fetches all rows
// of x whatever its width. 1,024 columns at 8 rows: 128 blocks of 8 columns as fast as 64 of 16, 256 of 4 slower.)
StreamPlan plan_for_carry(int N, int compute_units) {
  (void)compute_units;
  return {1, 1, (N + 15) / 16, 1};
}

StreamPlan plan_of(int M, int N, int K, bool gated, int k_splits, int compute_units) {
  if (k_splits > 1) {
    const StreamPlan p = plan_with_runs(M, N, K, compute_units);
    if (p.splits == k_splits) return p;
  }
  return plan_for_runs(M, N, gated, k_splits, compute_units);
}

template <int MT, bool SWIGLU, typename OutT>
void launch_arranged(StreamPlan plan, const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int steps_per_split,
                     int gate, RowScale rs, CarryOut carry, hipStream_t stream) {
  const dim3 grid(plan.grid, plan.splits, (M + kGroupRows - 1) / kGroupRows);
  const int wn = plan.wn;
  // Rows of W that lie a multiple of 4 KiB apart begin in the same memory channel: blocks that all start at k = 0 then
  // queue for a few channels (2 x 12,288 x 4,096 with SwiGLU at 32 rows: 46.7 us; with k = 4,224 38.8). Each block starts its
  // walk over k at a step of its own instead (39.4 us; at 1 and 8 rows 42.7 -> 40.5 and 43.1 -> 41.0; 6,144 x 4,096 at 32
  // rows 15.5 -> 14.3). Runs of k across blocks start at different k already, and other strides spread by themselves
  // (k = 5,120: no change either way), so those keep the plain walk.
  const ColumnDeal rotate = deal_of(N, plan.grid, plan.splits == 1 && K % 2048 == 0);
  if constexpr (MT >= 3 && !SWIGLU && sizeof(OutT) == 4) {
    if (plan.nt == 2) {  // (two steps in flight: 3-15% ahead of three)
      gemm_stream_kernel<MT, 4, 1, false, OutT, 2, 2><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
      return;
    }
  }
  if (rs.ss || carry.x) {  // the forms that scale their rows or add into the residual stream: instances of their own
    if (wn == 4)
      gemm_stream_kernel<MT, 4, 1, SWIGLU, OutT, (SWIGLU ? 2 : 3), 1, true><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
    else if (wn == 2)
      gemm_stream_kernel<MT, 2, 2, SWIGLU, OutT, (SWIGLU ? 3 : 4), 1, true><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
    else
      // (more steps in flight gain nothing for a block that walks all of k: 8 and 12 stages measured slower than 6)
      gemm_stream_kernel<MT, 1, 4, SWIGLU, OutT, (SWIGLU ? 4 : 6), 1, true><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
    return;
  }
  // (64 rows, blocks of 64 columns: a step more in flight, 3 gated and 4 plain, is 0.6% of a decode step of the 8B shape at
  // batch 64 slower and 1.3% of the 32B shape's)
  if (wn == 4)
    gemm_stream_kernel<MT, 4, 1, SWIGLU, OutT, (SWIGLU ? 2 : 3)><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
  else if (wn == 2)
    gemm_stream_kernel<MT, 2, 2, SWIGLU, OutT, (SWIGLU ? 3 : 4)><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
  else
    gemm_stream_kernel<MT, 1, 4, SWIGLU, OutT, (SWIGLU ? 4 : 6)><<<grid, 256, 0, stream>>>(X, W, C, M, N, K, steps_per_split, gate, rotate, rs, carry);
}

template <bool SWIGLU, typename OutT>
void launch_rows(StreamPlan plan, const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int steps_per_split, int gate,
                 RowScale rs, CarryOut carry, hipStream_t stream) {
  switch ((std::min(M, kGroupRows) + 15) / 16) {
    case 1: launch_arranged<1, SWIGLU, OutT>(plan, X, W, C, M, N, K, steps_per_split, gate, rs, carry, stream); break;
    case 2: launch_arranged<2, SWIGLU, OutT>(plan, X, W, C, M, N, K, steps_per_split, gate, rs, carry, stream); break;
    case 3: launch_arranged<3, SWIGLU, OutT>(plan, X, W, C, M, N, K, steps_per_split, gate, rs, carry, stream); break;
    default: launch_arranged<4, SWIGLU, OutT>(plan, X, W, C, M, N, K, steps_per_split, gate, rs, carry, stream); break;
  }
}

}  // namespace

// Into how many runs of k a product of M rows whose result may stay partial sums is cut (see plan_with_runs).
extern "C" int me_gemm_bf16_stream_splits(int M, int N, int K, int compute_units) {
  return plan_with_runs(M, N, K, compute_units < 1 ? 256 : compute_units).splits;
}

// What me_gemm_bf16_stream launches for a product: out[0] the groups of 16 columns per block (the other waves cut k
// within a step), out[1] the runs of k, out[2] the blocks along the columns.
extern "C" void me_gemm_bf16_stream_plan(int M, int N, int K, int gated, int k_splits, int compute_units, int* out) {
  const StreamPlan p = plan_of(M, N, K, gated != 0, k_splits, compute_units < 1 ? 256 : compute_units);
  out[0] = p.wn * p.nt, out[1] = p.splits, out[2] = p.grid;
}

static int stream_product(const char* who, const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                          int k_splits, int compute_units, RowScale rs, CarryOut carry, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (swiglu < ME_GATE_NONE || swiglu > ME_GATE_GELU_TANH) return me_fail("%s: unknown gate activation %d", who, swiglu);
  if (M > kMaxRows) return me_fail("%s: M=%d exceeds %d rows", who, M, kMaxRows);
  if (K <= 0 || K % 8) return me_fail("%s: K=%d must be a positive multiple of 8", who, K);
  if (!X || !W || (!C && !carry.x)) return me_fail("%s: null operand", who);
  if (((uintptr_t)X | (uintptr_t)W | (uintptr_t)C) & 15) return me_fail("%s: operands must be 16-byte aligned", who);
  if (out_dtype != ME_BF16 && out_dtype != ME_F32) return me_fail("%s: output type %d", who, out_dtype);
  if (k_splits < 1 || k_splits > 64) return me_fail("%s: %d splits of k", who, k_splits);
  if (k_splits > 1 && (swiglu || out_dtype != ME_F32))
    return me_fail("%s: partial sums over splits of k are plain float32 products", who);
  if (swiglu && out_dtype != ME_BF16) return me_fail("%s: the gated form writes bfloat16", who);
  if ((size_t)(swiglu ? 2 : 1) * N * K * 2 >= (1ull << 31) || (size_t)M * K * 2 >= (1ull << 31))
    return me_fail("%s: operands of 2 GiB and more are not addressed by this kernel", who);
  if (compute_units < 1) compute_units = 256;
  const int steps = (K + kStepK - 1) / kStepK;
  const int steps_per_split = (steps + k_splits - 1) / k_splits;
  const int splits = (steps + steps_per_split - 1) / steps_per_split;  // no empty run
  if (splits != k_splits) return me_fail("%s: K=%d cannot be cut into %d runs of whole steps", who, K, k_splits);
  const StreamPlan plan = carry.x ? plan_for_carry(N, compute_units) : plan_of(M, N, K, swiglu != 0, splits, compute_units);
  if (carry.x && carry.blocks != plan.grid * plan.wn * plan.nt)
    return me_fail("%s: %d partial sums of squares a row, the launch writes %d", who, carry.blocks, plan.grid * plan.wn * plan.nt);
  const bf16_t *x = (const bf16_t*)X, *w = (const bf16_t*)W;
  if (swiglu)
    launch_rows<true, bf16_t>(plan, x, w, (bf16_t*)C, M, N, K, steps_per_split, swiglu, rs, carry, stream);
  else if (out_dtype == ME_F32)
    launch_rows<false, float>(plan, x, w, (float*)C, M, N, K, steps_per_split, 0, rs, carry, stream);
  else
    launch_rows<false, bf16_t>(plan, x, w, (bf16_t*)C, M, N, K, steps_per_split, 0, rs, carry, stream);
  return me_check_launch(who);
}

// C[M, N] = x . W^T (swiglu 1 or 2, a MeGate code: W is [2 N, K], gate rows then up rows, and C = act(gate) * up), X bfloat16 [M, K],
// M <= 256, K % 8 == 0, pointers 16-byte aligned. out_dtype ME_BF16 or ME_F32. k_splits > 1 (plain float32
// products only): C is [k_splits, M, N], partial sums over runs of k for the caller to add up.
extern "C" int me_gemm_bf16_stream(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                                   int k_splits, int compute_units, hipStream_t stream) {
  return stream_product("me_gemm_bf16_stream", X, W, C, M, N, K, swiglu, out_dtype, k_splits, compute_units, RowScale{}, CarryOut{},
                        stream);
}

// The same product with its rows multiplied by rsqrt(sum_b row_ss[m, b] / ss_dim + eps) before the gate: the product
// behind an RMS norm whose division was left to it (me_gemm_bf16_stream_carry wrote row_ss, float32 [M, ss_blocks]).
extern "C" int me_gemm_bf16_stream_scaled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                                          int compute_units, const float* row_ss, int ss_blocks, int ss_dim, float eps,
                                          hipStream_t stream) {
  if (!row_ss || ss_blocks < 1 || ss_dim < 1) return me_fail("me_gemm_bf16_stream_scaled: no sums of squares");
  return stream_product("me_gemm_bf16_stream_scaled", X, W, C, M, N, K, swiglu, out_dtype, 1, compute_units,
                        RowScale{row_ss, ss_blocks, 1.f / (float)ss_dim, eps}, CarryOut{}, stream);
}

// Partial sums of squares a row that me_gemm_bf16_stream_carry writes for a product of these sizes.
extern "C" int me_gemm_bf16_stream_carry_blocks(int M, int N, int K, int compute_units) {
  (void)M, (void)K;
  const StreamPlan p = plan_for_carry(N, compute_units < 1 ? 256 : compute_units);
  return p.grid * p.wn * p.nt;
}

// x[M, N] += X . W^T in float32 (x the residual stream, X bfloat16 [M, K]), h[M, N] = bf16(x * w_norm) and
// ss[M, blocks] = partial sums of squares of the new rows of x, blocks = me_gemm_bf16_stream_carry_blocks(M, N, K, units):
// every block sums all of k for its columns, so nothing stays to be added up behind it.
extern "C" int me_gemm_bf16_stream_carry(const void* X, const void* W, float* x, void* h, float* ss, const float* w_norm, int M,
                                         int N, int K, int compute_units, hipStream_t stream) {
  if (!x || !h || !ss || !w_norm) return me_fail("me_gemm_bf16_stream_carry: null operand");
  if (((uintptr_t)x | (uintptr_t)w_norm) & 15 || (uintptr_t)h & 7) return me_fail("me_gemm_bf16_stream_carry: operands must be 16-byte aligned");
  const int blocks = me_gemm_bf16_stream_carry_blocks(M, N, K, compute_units);
  return stream_product("me_gemm_bf16_stream_carry", X, W, nullptr, M, N, K, 0, ME_F32, 1, compute_units, RowScale{},
                        CarryOut{x, (bf16_t*)h, ss, w_norm, blocks}, stream);
}

namespace {

template <bool SWIGLU, typename OutT>
int launch_norm(StreamPlan plan, const float* x_in, const bf16_t* delta, const float* parts, int num_parts, size_t part_stride,
                const float* w_norm, float eps, float* x_out, const bf16_t* W, OutT* C, int M, int N, int K, int gate,
                hipStream_t stream) {
  const dim3 grid(plan.grid);
  const int wn = plan.wn, wk = 4 / wn;
  const size_t rows_bytes = (((size_t)M * (K + 8) * 2 + 15) & ~(size_t)15) + (size_t)M * 4 * sizeof(float);
  const size_t sums_bytes = (64 + (size_t)(wk - 1) * wn * (SWIGLU ? 2 : 1) * 4 * 64) * sizeof(float);
  const size_t lds = std::max(rows_bytes, sums_bytes);
  if (lds > 48 * 1024) return me_fail("me_gemm_bf16_stream_norm: %d rows of %d do not fit the block's memory", M, K);
#define ME_NORM_LAUNCH(WN, WK, STAGES)                                                                                   \
  gemm_stream_norm_kernel<WN, WK, SWIGLU, OutT, STAGES><<<grid, 256, lds, stream>>>(x_in, delta, parts, num_parts, part_stride, \
                                                                                    w_norm, eps, x_out, W, C, M, N, K, gate, \
                                                                                    deal_of(N, plan.grid, K % 2048 == 0))
  if (wn == 4)
    ME_NORM_LAUNCH(4, 1, (SWIGLU ? 2 : 3));
  else if (wn == 2)
    ME_NORM_LAUNCH(2, 2, (SWIGLU ? 3 : 4));
  else
    ME_NORM_LAUNCH(1, 4, (SWIGLU ? 4 : 6));
#undef ME_NORM_LAUNCH
  return me_check_launch("me_gemm_bf16_stream_norm");
}

}  // namespace

// Whether me_gemm_bf16_stream_norm takes M rows of K: all rows of the normed input stay in the block's memory.
extern "C" int me_gemm_bf16_stream_norm_fits(int M, int K) {
  return M >= 1 && M <= 16 && K > 0 && K % 8 == 0 && (size_t)M * (K + 8) * 2 + 16 + (size_t)M * 16 <= 48 * 1024;
}

// C[M, N] = rmsnorm(x_in + delta) * w_norm . W^T for a row or a few (M <= 16; every block reads all of x_in and of the
// delta), with the gate as in me_gemm_bf16_stream. x_in float32 [M, K]; the delta is `delta` (bfloat16 [M, K]) or `parts`
// (float32 [num_parts] of [M, K], part_stride elements apart, added in their order) or neither; with a delta the sum
// is written to x_out (float32 [M, K], not aliasing x_in). w_norm float32 [K].
extern "C" int me_gemm_bf16_stream_norm(const float* x_in, const void* delta, const float* parts, int num_parts,
                                        long long part_stride, const float* w_norm, float eps, float* x_out, const void* W,
                                        void* C, int M, int N, int K, int swiglu, int out_dtype, int compute_units,
                                        hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (swiglu < ME_GATE_NONE || swiglu > ME_GATE_GELU_TANH) return me_fail("me_gemm_bf16_stream_norm: unknown gate activation %d", swiglu);
  if (!me_gemm_bf16_stream_norm_fits(M, K)) return me_fail("me_gemm_bf16_stream_norm: M=%d rows of K=%d are not taken", M, K);
  if (!x_in || !w_norm || !W || !C) return me_fail("me_gemm_bf16_stream_norm: null operand");
  if (delta && parts) return me_fail("me_gemm_bf16_stream_norm: a delta or partial sums, not both");
  if ((delta || parts) && (!x_out || x_out == x_in))
    return me_fail("me_gemm_bf16_stream_norm: x_out must be given and must not alias x_in");
  if (parts && (num_parts < 1 || part_stride < (long long)M * K || part_stride % 4))
    return me_fail("me_gemm_bf16_stream_norm: %d partial sums %lld elements apart for %d rows of %d", num_parts, part_stride, M, K);
  if (((uintptr_t)x_in | (uintptr_t)parts | (uintptr_t)w_norm | (uintptr_t)x_out | (uintptr_t)W | (uintptr_t)C) & 15 || (uintptr_t)delta & 7)
    return me_fail("me_gemm_bf16_stream_norm: operands must be 16-byte aligned");
  if (out_dtype != ME_BF16 && out_dtype != ME_F32) return me_fail("me_gemm_bf16_stream_norm: output type %d", out_dtype);
  if (swiglu && out_dtype != ME_BF16) return me_fail("me_gemm_bf16_stream_norm: the gated form writes bfloat16");
  if ((size_t)(swiglu ? 2 : 1) * N * K * 2 >= (1ull << 31))
    return me_fail("me_gemm_bf16_stream_norm: weights of 2 GiB and more are not addressed by this kernel");
  if (compute_units < 1) compute_units = 256;
  const StreamPlan plan = plan_of(M, N, K, swiglu != 0, 1, compute_units);
  const bf16_t *d = (const bf16_t*)delta, *w = (const bf16_t*)W;
  const size_t stride = parts ? (size_t)part_stride : 0;
  if (swiglu)
    return launch_norm<true, bf16_t>(plan, x_in, d, parts, num_parts, stride, w_norm, eps, x_out, w, (bf16_t*)C, M, N, K, swiglu, stream);
  if (out_dtype == ME_F32)
    return launch_norm<false, float>(plan, x_in, d, parts, num_parts, stride, w_norm, eps, x_out, w, (float*)C, M, N, K, 0, stream);
  return launch_norm<false, bf16_t>(plan, x_in, d, parts, num_parts, stride, w_norm, eps, x_out, w, (bf16_t*)C, M, N, K, 0, stream);
}
