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
  const long long unit = (long long)blockIdx.x * (blockDim.x / ME_WAVE) + wave;
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

  const bool vec_k = sizeof(T) == 4 && d % 4 == 0 && ((uintptr_t)k_cache & 15) == 0;   // a key row in 16-byte pieces
  const bool vec_v = sizeof(T) == 4 && bs % 4 == 0 && ((uintptr_t)v_cache & 15) == 0;  // four keys of a value row at once
  for (int tile = (lo / 64) * 64; tile <= p; tile += 64) {
    const int key = tile + lane;
    const bool valid = key >= lo && key <= p;
    float s = -INFINITY;
    if (valid) {
      const int page = table[key / bs];
      const T* krow = k_cache + (((size_t)page * nkv + kvh) * bs + key % bs) * d;
      float dot = 0.f;
      if (vec_k) {  // the same products in the same order; 128 elements of the row are requested before the first is used
        const float4* k4 = reinterpret_cast<const float4*>(krow);
        const int n4 = d / 4;
        for (int base = 0; base < n4; base += 32) {
          float4 kv[32];
#pragma unroll
          for (int u = 0; u < 32; ++u) kv[u] = base + u < n4 ? k4[base + u] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
          for (int u = 0; u < 32; ++u)
            if (base + u < n4) {
              const int i = 4 * (base + u);
              dot = fmaf(qw[i], kv[u].x, dot);
              dot = fmaf(qw[i + 1], kv[u].y, dot);
              dot = fmaf(qw[i + 2], kv[u].z, dot);
              dot = fmaf(qw[i + 3], kv[u].w, dot);
            }
        }
      } else {
        for (int i = 0; i < d; ++i) dot = fmaf(qw[i], to_float(krow[i]), dot);
      }
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
    int j = j_lo;
    if (vec_v) {
      // whole groups of four keys that lie in one page (tiles and groups are aligned to 4, pages hold a multiple of
      // 4): one 16-byte load per group and element of the head, the sums in the order of the keys as below
      for (; j <= j_hi && (j & 3); ++j) {
        const float pj = __shfl(pr, j, ME_WAVE);
        const int kj = tile + j;
        const T* vbase = v_cache + ((size_t)table[kj / bs] * nkv + kvh) * d * bs + kj % bs;
#pragma unroll
        for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) {
          const int i = lane + k * ME_WAVE;
          if (i < d) acc[k] = fmaf(pj, to_float(vbase[(size_t)i * bs]), acc[k]);
        }
      }
      // eight groups of four keys at a time: their values are requested before the first is used
      const int groups = j <= j_hi ? (j_hi + 1 - j) / 4 : 0;  // whole groups from j on
      for (int g0 = 0; g0 < groups; g0 += 8) {
        float4 vv[8][AG_MAX_D / ME_WAVE];
#pragma unroll
        for (int gq = 0; gq < 8; ++gq) {
          const bool there = g0 + gq < groups;
          const int kj = tile + j + 4 * (there ? g0 + gq : 0);
          const T* vbase = v_cache + ((size_t)table[kj / bs] * nkv + kvh) * d * bs + kj % bs;
#pragma unroll
          for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) {
            const int i = lane + k * ME_WAVE;
            vv[gq][k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (there && i < d) vv[gq][k] = *reinterpret_cast<const float4*>(vbase + (size_t)i * bs);
          }
        }
#pragma unroll
        for (int gq = 0; gq < 8; ++gq) {
          if (g0 + gq < groups) {
            const int jj = j + 4 * (g0 + gq);
            const float p0 = __shfl(pr, jj, ME_WAVE), p1 = __shfl(pr, jj + 1, ME_WAVE), p2 = __shfl(pr, jj + 2, ME_WAVE),
                        p3 = __shfl(pr, jj + 3, ME_WAVE);
#pragma unroll
            for (int k = 0; k < AG_MAX_D / ME_WAVE; ++k) {
              if (lane + k * ME_WAVE < d) {
                acc[k] = fmaf(p0, vv[gq][k].x, acc[k]);
                acc[k] = fmaf(p1, vv[gq][k].y, acc[k]);
                acc[k] = fmaf(p2, vv[gq][k].z, acc[k]);
                acc[k] = fmaf(p3, vv[gq][k].w, acc[k]);
              }
            }
          }
        }
      }
      j += 4 * groups;
    }
    for (; j <= j_hi; ++j) {
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
  const int waves = units < 2048 ? 1 : 4;  // few units (decode steps): a compute unit each
  const unsigned blocks = (unsigned)((units + waves - 1) / waves);
  if (dtype == ME_F32)
    attention_general_kernel<float><<<blocks, waves * 64, 0, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, positions, token_item, block_table,
        table_width, (float*)out, num_tokens, nh, nkv, d, bs, window, scale);
  else
    attention_general_kernel<bf16_t><<<blocks, waves * 64, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, token_item, block_table,
        table_width, (bf16_t*)out, num_tokens, nh, nkv, d, bs, window, scale);
  return me_check_launch("me_attention_general");
}
