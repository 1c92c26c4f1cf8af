// Causal grouped-query attention over the paged cache, for any mix of items in a step: one wave
// per (new token, query head). It takes every size the cache allows (any page size, any group
// size, head sizes up to 256 in steps of 2) in float32 or bfloat16 storage, and is the kernel of
// the 32-bit path; the bfloat16 path uses the matrix-core kernels where their size limits hold.
//
// A token at absolute position p of item b sees keys lo..p of item b, lo = max(0, p - window + 1)
// (window == 0: lo = 0). Keys are visited in tiles of 64 aligned to absolute position (tile t holds
// positions 64t .. 64t+63), so the order of every sum depends on p, lo and the head alone, never on
// how the sequence was cut into steps or on what else is in the batch.
//
// Cache layout per layer: keys K[page, kv_head, slot, d]; values transposed V[page, kv_head, d, slot].
#include "common.h"

#define AG_MAX_D 256

template <typename T>
__global__ __launch_bounds__(256) void attention_general_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table,
    int table_width, T* __restrict__ out, int num_tokens, int nh, int nkv, int d, int bs, int window, float scale) {
  __shared__ float qs[4][AG_MAX_D];
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const long long unit = (long long)blockIdx.x * 4 + wave;
  if (unit >= (long long)num_tokens * nh) return;
  const int t = (int)(unit / nh), head = (int)(unit % nh);
  const int kvh = head / (nh / nkv);
  const int p = positions[t];
  const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int* table = block_table + (size_t)token_item[t] * table_width;

  const T* qrow = q + ((size_t)t * nh + head) * d;
  float* qw = qs[wave];
  for (int i = lane; i < d; i += ME_WAVE) qw[i] = to_float(qrow[i]) * scale;
  __builtin_amdgcn_wave_barrier();

  float m = -INFINITY, l = 0.f;
  float acc[AG_MAX_D / ME_WAVE];
#pragma unroll
  for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) acc[k] = 0.f;

  for (int tile = (lo / 64) * 64; tile <= p; tile += 64) {
    const int key = tile + lane;
    const bool valid = key >= lo && key <= p;
    float s = -INFINITY;
    if (valid) {
      const int page = table[key / bs];
      const T* krow = k_cache + (((size_t)page * nkv + kvh) * bs + key % bs) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(qw[i], to_float(krow[i]), dot);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));  // at least one key of the tile is visible
    const float pr = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // exp(-inf) = 0 on the first tile
    l = l * alpha + wave_sum(pr);
#pragma unroll
    for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) acc[k] *= alpha;
    m = m_new;
    const int j_lo = lo > tile ? lo - tile : 0;
    const int j_hi = p - tile < 63 ? p - tile : 63;
    for (int j = j_lo; j <= j_hi; ++j) {
      const float pj = __shfl(pr, j, ME_WAVE);
      const int kj = tile + j;
      const int page = table[kj / bs];
      const T* vbase = v_cache + ((size_t)page * nkv + kvh) * d * bs + kj % bs;
#pragma unroll
      for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) {
        const int i = lane + k * ME_WAVE;
        if (i < d) acc[k] = fmaf(pj, to_float(vbase[(size_t)i * bs]), acc[k]);
      }
    }
  }
  T* orow = out + ((size_t)t * nh + head) * d;
  const float inv = 1.f / l;
#pragma unroll
  for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) {
    const int i = lane + k * ME_WAVE;
    if (i < d) orow[i] = from_float<T>(acc[k] * inv);
  }
}

extern "C" int me_attention_general(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                    const int* token_item, const int* block_table, int table_width, void* out,
                                    int num_tokens, int nh, int nkv, int d, int bs, int window, float scale,
                                    int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (d <= 0 || d > AG_MAX_D) return me_fail("me_attention_general: head_dim=%d must be in 1..%d", d, AG_MAX_D);
  if (nh <= 0 || nkv <= 0 || nh % nkv)
    return me_fail("me_attention_general: %d query heads are not a multiple of %d key/value heads", nh, nkv);
  if (bs <= 0 || table_width <= 0 || window < 0)
    return me_fail("me_attention_general: block_size=%d table_width=%d window=%d", bs, table_width, window);
  const long long units = (long long)num_tokens * nh;
  const unsigned blocks = (unsigned)((units + 3) / 4);
  if (dtype == ME_F32)
    attention_general_kernel<float><<<blocks, 256, 0, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, positions, token_item, block_table,
        table_width, (float*)out, num_tokens, nh, nkv, d, bs, window, scale);
  else
    attention_general_kernel<bf16_t><<<blocks, 256, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, token_item, block_table,
        table_width, (bf16_t*)out, num_tokens, nh, nkv, d, bs, window, scale);
  return me_check_launch("me_attention_general");
}
