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

// Stage 1: block (row, chunk) scans a contiguous slice of the vocabulary and writes its best
// (value, index). Stage 2: one wave per row picks the best of the chunks. Ties go to the lowest index
// at both stages, so the result is that of a single scan.
struct Best {
  float v;
  int i;
};

__device__ __forceinline__ void take_better(float& bv, int& bi, float ov, int oi) {
  if (ov > bv || (ov == bv && oi < bi)) {
    bv = ov;
    bi = oi;
  }
}

__device__ __forceinline__ void wave_best(float& bv, int& bi) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, ME_WAVE);
    const int oi = __shfl_xor(bi, off, ME_WAVE);
    take_better(bv, bi, ov, oi);
  }
}

__global__ __launch_bounds__(256) void sample_stage1_kernel(const float* __restrict__ logits, int vocab,
                                                            const float* __restrict__ temperatures,
                                                            const uint64_t* __restrict__ keys, Best* __restrict__ part,
                                                            int chunks, int chunk_len) {
  __shared__ float best_v[4];
  __shared__ int best_i[4];
  const int row = blockIdx.x, chunk = blockIdx.y;
  const float* lr = logits + (size_t)row * vocab;
  const float temp = temperatures ? temperatures[row] : 0.f;
  const uint64_t key = keys ? keys[row] : 0;
  const float inv_t = temp > 0.f ? 1.f / fmaxf(temp, 1e-5f) : 1.f;
  const int begin = chunk * chunk_len, end = min(vocab, begin + chunk_len);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    float v = lr[i];
    if (temp > 0.f) v = v * inv_t + gumbel_noise(key, i);
    take_better(bv, bi, v, i);
  }
  wave_best(bv, bi);
  const int lane = threadIdx.x & (ME_WAVE - 1), wave = threadIdx.x / ME_WAVE;
  if (lane == 0) {
    best_v[wave] = bv;
    best_i[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) take_better(bv, bi, best_v[w], best_i[w]);
    part[(size_t)row * chunks + chunk].v = bv;
    part[(size_t)row * chunks + chunk].i = bi;
  }
}

__global__ __launch_bounds__(64) void sample_stage2_kernel(const Best* __restrict__ part, int chunks,
                                                           int* __restrict__ out) {
  const int row = blockIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += ME_WAVE) take_better(bv, bi, part[(size_t)row * chunks + c].v,
                                                                  part[(size_t)row * chunks + c].i);
  wave_best(bv, bi);
  if (threadIdx.x == 0) out[row] = bi == 0x7fffffff ? 0 : bi;  // a row of NaNs picks token 0, not an invalid id
}

// Number of vocabulary slices per row; the workspace holds rows * chunks (float, int) pairs.
extern "C" int me_sample_chunks(int vocab) {
  const int c = (vocab + 2047) / 2048;
  return c < 1 ? 1 : (c > 128 ? 128 : c);
}

extern "C" int me_sample(const float* logits, int num_rows, int vocab, const float* temperatures,
                         const uint64_t* keys, int* out, void* workspace, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (vocab <= 0) return me_fail("me_sample: vocab=%d", vocab);
  if (num_rows > 65535) return me_fail("me_sample: %d rows exceed the grid", num_rows);
  const int chunks = me_sample_chunks(vocab);
  const int chunk_len = (vocab + chunks - 1) / chunks;
  sample_stage1_kernel<<<dim3(num_rows, chunks), 256, 0, stream>>>(logits, vocab, temperatures, keys, (Best*)workspace,
                                                                   chunks, chunk_len);
  if (me_check_launch("me_sample stage 1")) return 1;
  sample_stage2_kernel<<<num_rows, 64, 0, stream>>>((const Best*)workspace, chunks, out);
  return me_check_launch("me_sample stage 2");
}

// ---------------------------------------------------------------- the entry point that allocates nothing
// me_sample_static: me_sample without a workspace argument. The (value, index) pairs that stage 1
// hands to stage 2 live in a file-scope device array instead of memory the caller allocates. See
// no_alloc.h for who this is for and what it asks of the caller.
#include "no_alloc.h"

#include <mutex>

static __device__ __align__(256) unsigned char scratch[ME_SAMPLE_STATIC_SCRATCH_BYTES];

#define ME_MAX_DEVICES 64
static void* g_scratch_ptr[ME_MAX_DEVICES];  // this library's copy of `scratch` on each device, once looked up
static std::mutex g_scratch_mutex;

// The device address of `scratch` on the current device. In host code the array's name is only a
// handle for this lookup; kernels and copies get the address it returns.
static int static_scratch(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return me_fail("me_sample_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= ME_MAX_DEVICES) return me_fail("me_sample_static: device %d is beyond %d", dev, ME_MAX_DEVICES);
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return me_fail("me_sample_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" int me_sample_static_max_pairs() { return ME_SAMPLE_STATIC_SCRATCH_BYTES / (int)sizeof(Best); }

extern "C" int me_sample_static(const float* logits, int num_rows, int vocab, const float* temperatures,
                                const uint64_t* keys, int* out, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (vocab <= 0) return me_fail("me_sample_static: vocab=%d", vocab);
  const int chunks = me_sample_chunks(vocab);
  if ((long long)num_rows * chunks > me_sample_static_max_pairs())
    return me_fail("me_sample_static: %d rows of %d vocabulary slices need %lld pairs of scratch, the static "
                   "buffer holds %d (use me_sample with a workspace of your own)",
                   num_rows, chunks, (long long)num_rows * chunks, me_sample_static_max_pairs());
  void* ws = nullptr;
  if (static_scratch(&ws)) return 1;
  // Stage 1 writes every pair that stage 2 reads (rows x chunks of them), so what the last call left
  // in the buffer needs no clearing.
  return me_sample(logits, num_rows, vocab, temperatures, keys, out, ws, stream);
}
