// Shared device helpers for the gfx950 kernels: bfloat16 storage type, wave-wide reductions for
// 64-lane wavefronts, and the error-reporting convention of the extern "C" entry points.
//
// Every entry point returns 0 on success. On a refused size or a failed launch it returns a
// non-zero code and leaves a message that me_last_error() hands to the caller; nothing is
// launched in that case, so a refused size never produces a wrong result.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define ME_WAVE 64

extern "C" const char* me_last_error();
int me_fail(const char* fmt, ...);
int me_check_launch(const char* what);

enum MeDtype { ME_F32 = 0, ME_BF16 = 1 };

// ------------------------------------------------------------------ bfloat16 as raw 16 bits
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }

// Round to nearest, ties to even; NaN stays NaN: the hardware's conversion (gfx950 has one; by integer arithmetic this
// is six instructions a value, which the tails and inner loops of the small kernels feel).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ float from_float<float>(float f) {
  return f;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(f);
  return r;
}

// ------------------------------------------------------------------ loads of data that is read once
// A buffer that a kernel reads once streams at 7.1-7.2 TB/s through non-temporal loads (the `nt` bit) where ordinary
// loads reach 6.1-6.5 (4 GiB read by 2,048 to 131,072 blocks of 256 lanes, 16 bytes a lane). Decode attention takes
// the keys and values of large launches that way. Weights do not gain: the head's 311 MB at one row and the
// projections of the 8B and 32B shapes took 1-11% longer (what a step reads again the step after seems to be served
// better by ordinary loads).
typedef unsigned me_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned me_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 stream_load16(const void* p) {
  const me_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const me_u32x4*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ me_u32x2 stream_load8(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const me_u32x2*>(p));
}

// ------------------------------------------------------------------ the activation of a gated feed-forward
// act(gate) * up: the codes that the entry points' `gated` arguments take (0: the product is not gated).
enum MeGate { ME_GATE_NONE = 0, ME_GATE_SILU = 1, ME_GATE_GELU_TANH = 2 };

__device__ __forceinline__ float gate_act(float g, int code) {
  if (code == ME_GATE_GELU_TANH) {  // 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))
    const float u = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.f + tanhf(u));
  }
  return g / (1.f + expf(-g));  // silu
}
// The same for results that are rounded to bfloat16: the exponential and the reciprocal as one instruction each (a
// correctly rounded division and expf are two dozen instructions at the tail of every gated product).
__device__ __forceinline__ float gate_act_bf16(float g, int code) {
  if (code == ME_GATE_GELU_TANH) return gate_act(g, code);
  return g * __builtin_amdgcn_rcpf(1.f + __expf(-g));
}

// ------------------------------------------------------------------ wave and block reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, ME_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, ME_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads. `scratch` holds 16 floats of LDS. Every thread gets
// the result; the order of additions is fixed by the thread layout alone.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (ME_WAVE - 1), wave = threadIdx.x / ME_WAVE;
  const int nwaves = (blockDim.x + ME_WAVE - 1) / ME_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

// ------------------------------------------------------------------ a norm carried from one product to the next
// A product that is a delta of the float32 residual stream can add itself to the stream in its epilogue and leave,
// for the RMS norm behind it, bf16(stream * w_norm) (not yet divided by the row's root mean square) and the sums of
// squares of what its blocks added up, `blocks` partial sums a row. The product behind the norm multiplies its rows
// by rsqrt(sum / dim + eps): a row's scale is a common factor of its products. No kernel of its own adds and norms.
struct CarryOut {   // what the first product leaves (x == nullptr: an ordinary product)
  float* x;         // [M, N] the residual stream, added to in place
  bf16_t* h;        // [M, N] bf16(x * w_norm)
  float* ss;        // [M, blocks] partial sums of squares of the rows of x
  const float* w_norm;  // [N]
  int blocks;
};
struct RowScale {   // what the second product reads (ss == nullptr: rows are not scaled)
  const float* ss;  // [M, blocks]
  int blocks;
  float inv_dim, eps;
};

// scale[m] = rsqrt(sum_b ss[m, b] / dim + eps) for rows m < M, by the waves of a block in turn, in two halves: the loads
// at a kernel's head (row_ss_fetch: wave w takes rows w, w + waves, ..; a lane sums every 64th partial sum), the rest
// when the kernel's own work is done (row_scales_finish), so that the loads' latency hides behind it. The order of the
// additions follows from the number of partial sums alone. The caller puts a barrier before it reads `scale`.
template <int ROWS_PER_WAVE>
__device__ __forceinline__ void row_ss_fetch(const RowScale& rs, int M, float (&part)[ROWS_PER_WAVE], int wave, int lane, int waves) {
#pragma unroll
  for (int i = 0; i < ROWS_PER_WAVE; ++i) {
    const int m = wave + i * waves;
    // (one load per lane and row in the usual case, and nothing computed on it here: no wait at the kernel's head)
    float s = m < M && lane < rs.blocks ? rs.ss[(size_t)m * rs.blocks + lane] : 0.f;
    if (rs.blocks > ME_WAVE && m < M)
      for (int b = lane + ME_WAVE; b < rs.blocks; b += ME_WAVE) s += rs.ss[(size_t)m * rs.blocks + b];
    part[i] = s;
  }
}
template <int ROWS_PER_WAVE>
__device__ __forceinline__ void row_scales_finish(const RowScale& rs, int M, const float (&part)[ROWS_PER_WAVE], float* scale,
                                                  int wave, int lane, int waves) {
#pragma unroll
  for (int i = 0; i < ROWS_PER_WAVE; ++i) {
    const int m = wave + i * waves;
    const float s = wave_sum(part[i]);
    if (m < M && lane == 0) scale[m] = rsqrtf(s * rs.inv_dim + rs.eps);
  }
}
