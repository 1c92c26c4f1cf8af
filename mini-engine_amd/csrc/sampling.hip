// Token choice from float32 logits [R, V], one block per row:
//   temperature == 0: argmax (the lowest index among equal maxima);
//   temperature  > 0: argmax of logits / max(temperature, 1e-5) + g_i with g_i independent standard
//     Gumbel noise, which draws index i with probability softmax(logits / temperature)_i.
// The noise for (row, i) is a pure function of the row's 64-bit key and i, so a request's draw does
// not depend on what else is in the batch. The host derives the key from (seed, request, number of
// the output token).
#include "common.h"

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

// Uniform in (0, 1) from the top 32 bits: (r + 0.5) / 2^32.
__device__ __forceinline__ float gumbel_noise(uint64_t key, int i) {
  const uint64_t h = mix64(key ^ mix64((uint64_t)(uint32_t)i));
  const float u = ((float)(uint32_t)(h >> 32) + 0.5f) * 2.3283064365386963e-10f;
  const float uc = fminf(u, 0.99999994f);
  return -logf(-logf(uc));
}

__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                      const float* __restrict__ temperatures,
                                                      const uint64_t* __restrict__ keys, int* __restrict__ out) {
  __shared__ float best_v[16];
  __shared__ int best_i[16];
  const int row = blockIdx.x;
  const float* lr = logits + (size_t)row * vocab;
  const float temp = temperatures ? temperatures[row] : 0.f;
  const uint64_t key = keys ? keys[row] : 0;
  const float inv_t = temp > 0.f ? 1.f / fmaxf(temp, 1e-5f) : 1.f;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    float v = lr[i];
    if (temp > 0.f) v = v * inv_t + gumbel_noise(key, i);
    if (v > bv || (v == bv && i < bi)) {
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, ME_WAVE);
    const int oi = __shfl_xor(bi, off, ME_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) {
      bv = ov;
      bi = oi;
    }
  }
  const int lane = threadIdx.x & (ME_WAVE - 1), wave = threadIdx.x / ME_WAVE;
  if (lane == 0) {
    best_v[wave] = bv;
    best_i[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int nwaves = blockDim.x / ME_WAVE;
    for (int w = 1; w < nwaves; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
        bv = best_v[w];
        bi = best_i[w];
      }
    out[row] = bi == 0x7fffffff ? 0 : bi;  // a row of NaNs picks token 0 rather than an invalid id
  }
}

extern "C" int me_sample(const float* logits, int num_rows, int vocab, const float* temperatures,
                         const uint64_t* keys, int* out, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (vocab <= 0) return me_fail("me_sample: vocab=%d", vocab);
  const int threads = vocab >= 8192 ? 1024 : (vocab >= 1024 ? 256 : 64);
  sample_kernel<<<num_rows, threads, 0, stream>>>(logits, vocab, temperatures, keys, out);
  return me_check_launch("me_sample");
}
