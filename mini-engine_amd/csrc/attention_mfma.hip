// bfloat16 attention over the paged cache on the matrix cores (v_mfma_f32_16x16x16_bf16), for
// head sizes that are multiples of 32 and page sizes that are multiples of 16.
//
// Both kernels compute the transposed products, so that every operand is read along the direction
// in which it is contiguous in memory and the scores never leave their registers:
//
//   S^T[key, q] = sum_d K[key, d] Q[q, d]        A = K page rows (along d), B = Q rows (along d)
//   O^T[d, q]  += sum_key V^T[d, key] P^T[key, q] A = transposed value page (along keys), B = P^T
//
// The 16x16 result of the first product leaves lane l with S^T[(l/16)*4 .. +4][l%16]: four keys of
// one query column. That is exactly the B-operand layout of the second product, so exp(S - max)
// is rounded to bfloat16 in place and fed back. A query column is one (token, head of the group);
// its running maximum and sum live in the four lanes l%16 + {0,16,32,48}.
//
// Scores are scaled in float32 after the product (the query is not rounded a second time);
// softmax statistics and the output accumulator are float32; exponentials are base 2 with the
// scale folded in.
//
//  * me_attention_decode_bf16: one new token per item. Grid (items, kv heads x head chunks, splits);
//    each wave handles one split of the context for the heads of one group and writes an
//    unnormalised partial result; me_attention_decode_combine merges the splits.
//  * me_attention_prefill_bf16: any number of new tokens per item (causal within the new tokens,
//    earlier keys from the cache). Grid (query tiles, kv heads); four waves of 32 query columns.
#include "common.h"

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

union Frag8 {  // eight bfloat16: one 16-byte load feeding two matrix-core steps
  uint4 u;
  short4_t h[2];
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ short4_t pack_bf16x4(float a, float b, float c, float d) {
  short4_t r;
  r[0] = (short)f32_to_bf16_bits(a);
  r[1] = (short)f32_to_bf16_bits(b);
  r[2] = (short)f32_to_bf16_bits(c);
  r[3] = (short)f32_to_bf16_bits(d);
  return r;
}

// max / sum over the four lanes that share a query column (l%16 fixed, l/16 = 0..3)
__device__ __forceinline__ float column_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, ME_WAVE));
  return fmaxf(v, __shfl_xor(v, 32, ME_WAVE));
}
__device__ __forceinline__ float column_sum(float v) {
  v += __shfl_xor(v, 16, ME_WAVE);
  return v + __shfl_xor(v, 32, ME_WAVE);
}

#define LOG2E 1.4426950408889634f

// One 16-key tile for NB blocks of 16 query columns. `kbase` points at K[page, kvh, off, 0], `vbase`
// at V^T[page, kvh, 0, off]. key0 is the absolute position of the tile's first key. A key is
// visible to column nb if lo <= key <= qpos[nb].
template <int D, int NB>
__device__ __forceinline__ void attend_tile(const bf16_t* __restrict__ kbase, const bf16_t* __restrict__ vbase,
                                            int bs, int key0, int lo, const int (&qpos)[NB], bool need_mask,
                                            const Frag8 (&qf)[NB][D / 32], float scale_log2,
                                            float (&m)[NB], float (&lsum)[NB], float4_t (&acc)[NB][D / 16]) {
  const int lane = threadIdx.x & (ME_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  Frag8 kf[D / 32];
#pragma unroll
  for (int c = 0; c < D / 32; ++c) kf[c].u = *reinterpret_cast<const uint4*>(kbase + (size_t)r * D + c * 32 + g * 8);
  short4_t vf[D / 16];
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
    vf[dt] = *reinterpret_cast<const short4_t*>(vbase + (size_t)(dt * 16 + r) * bs + g * 4);

  short4_t pf[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf[c].h[0], qf[nb][c].h[0], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf[c].h[1], qf[nb][c].h[1], s, 0, 0, 0);
    }
    float sv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sv[i] = s[i] * scale_log2;
      if (need_mask) {
        const int key = key0 + g * 4 + i;
        if (key < lo || key > qpos[nb]) sv[i] = -INFINITY;
      }
    }
    float tmax = column_max(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
    const float m_new = fmaxf(m[nb], tmax);
    // a column that has seen no visible key yet keeps m = -inf; use 0 as the reference then
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m[nb] - m_ref);
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = fast_exp2(sv[i] - m_ref);
    lsum[nb] = lsum[nb] * alpha + column_sum((p[0] + p[1]) + (p[2] + p[3]));
    m[nb] = m_new;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      acc[nb][dt][0] *= alpha;
      acc[nb][dt][1] *= alpha;
      acc[nb][dt][2] *= alpha;
      acc[nb][dt][3] *= alpha;
    }
    pf[nb] = pack_bf16x4(p[0], p[1], p[2], p[3]);
  }
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      acc[nb][dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[dt], pf[nb], acc[nb][dt], 0, 0, 0);
}

// ------------------------------------------------------------------------------------- decode
// Partial results: part_o [items, nh, splits, D] (unnormalised), part_ml [items, nh, splits, 2].
template <int D>
__global__ __launch_bounds__(64) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ item_ctx, const int* __restrict__ block_table, int table_width,
    float* __restrict__ part_o, float* __restrict__ part_ml, int nh, int nkv, int bs, int window, float scale_log2,
    int split_keys, int num_splits, int head_chunks) {
  const int item = blockIdx.x;
  const int kvh = blockIdx.y / head_chunks, chunk = blockIdx.y % head_chunks;
  const int split = blockIdx.z;
  const int group = nh / nkv;
  const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
  const int heads_here = min(16, group - chunk * 16);
  const int head0 = kvh * group + chunk * 16;
  const int ctx = item_ctx[item];
  const int lo = window > 0 ? max(ctx - window, 0) : 0;
  const int begin = max(split * split_keys, (lo / 16) * 16);
  const int end = min((split + 1) * split_keys, ctx);

  float m[1] = {-INFINITY}, lsum[1] = {0.f};
  float4_t acc[1][D / 16];
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt) acc[0][dt] = (float4_t){0.f, 0.f, 0.f, 0.f};

  if (begin < end) {
    Frag8 qf[1][D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      qf[0][c].u = make_uint4(0, 0, 0, 0);
      if (r < heads_here)
        qf[0][c].u = *reinterpret_cast<const uint4*>(q + ((size_t)item * nh + head0 + r) * D + c * 32 + g * 8);
    }
    const int qpos[1] = {ctx - 1};
    const int* table = block_table + (size_t)item * table_width;
    for (int key0 = begin; key0 < end; key0 += 16) {
      int page = table[key0 / bs];
      page = page < 0 ? 0 : page;
      const int off = key0 % bs;
      const bf16_t* kbase = k_cache + (((size_t)page * nkv + kvh) * bs + off) * D;
      const bf16_t* vbase = v_cache + ((size_t)page * nkv + kvh) * D * bs + off;
      const bool need_mask = key0 < lo || key0 + 16 > ctx;
      attend_tile<D, 1>(kbase, vbase, bs, key0, lo, qpos, need_mask, qf, scale_log2, m, lsum, acc);
    }
  }
  if (r < heads_here) {
    const size_t slot = ((size_t)item * nh + head0 + r) * num_splits + split;
    if (g == 0) {
      part_ml[slot * 2] = m[0];
      part_ml[slot * 2 + 1] = lsum[0];
    }
    float* po = part_o + slot * D;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      *reinterpret_cast<float4_t*>(po + dt * 16 + g * 4) = acc[0][dt];
  }
}

// out[item, head, :] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s. One block of 256 threads per
// (item, head): the weights of all splits first (every split's statistics are loaded at once), then
// the weighted sum with thread -> (four output elements, one of 256 / (d/4) groups of splits), so
// that the loads of different splits are independent of each other.
#define ME_MAX_SPLITS 1024
__global__ __launch_bounds__(256) void attention_decode_combine_kernel(const float* __restrict__ part_o,
                                                                       const float* __restrict__ part_ml,
                                                                       bf16_t* __restrict__ out, int num_splits, int d) {
  __shared__ float wgt[ME_MAX_SPLITS];
  __shared__ float red_max[4], red_sum[4];
  __shared__ float4_t partial[256];
  const size_t unit = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & (ME_WAVE - 1), wave = tid / ME_WAVE;
  const float* ml = part_ml + unit * num_splits * 2;
  float big = -INFINITY;
  for (int s = tid; s < num_splits; s += 256)
    if (ml[s * 2 + 1] > 0.f) big = fmaxf(big, ml[s * 2]);
  big = wave_max(big);
  if (lane == 0) red_max[wave] = big;
  __syncthreads();
  big = fmaxf(fmaxf(red_max[0], red_max[1]), fmaxf(red_max[2], red_max[3]));
  float part_denom = 0.f;
  for (int s = tid; s < num_splits; s += 256) {
    const float l = ml[s * 2 + 1];
    const float w = l > 0.f ? fast_exp2(ml[s * 2] - big) : 0.f;  // an empty split has no weight
    wgt[s] = w;
    part_denom += w * l;
  }
  part_denom = wave_sum(part_denom);
  if (lane == 0) red_sum[wave] = part_denom;
  __syncthreads();
  const float denom = (red_sum[0] + red_sum[1]) + (red_sum[2] + red_sum[3]);

  const int quads = d / 4;          // d is a multiple of 32, so quads <= 64
  const int groups = 256 / quads;   // groups of splits handled side by side
  const int qd = tid % quads, grp = tid / quads;
  float4_t accv = {0.f, 0.f, 0.f, 0.f};
  if (grp < groups) {
    const float* po = part_o + unit * num_splits * d + qd * 4;
    for (int s = grp; s < num_splits; s += groups) {
      const float w = wgt[s];
      const float4_t v = *reinterpret_cast<const float4_t*>(po + (size_t)s * d);
      accv[0] += w * v[0];
      accv[1] += w * v[1];
      accv[2] += w * v[2];
      accv[3] += w * v[3];
    }
  }
  partial[tid] = accv;
  __syncthreads();
  if (tid < quads) {
    float4_t total = partial[tid];
    for (int gi = 1; gi < groups; ++gi) {
      const float4_t v = partial[gi * quads + tid];
      total[0] += v[0];
      total[1] += v[1];
      total[2] += v[2];
      total[3] += v[3];
    }
    const float inv = 1.f / denom;
    *reinterpret_cast<short4_t*>(out + unit * d + tid * 4) =
        pack_bf16x4(total[0] * inv, total[1] * inv, total[2] * inv, total[3] * inv);
  }
}

template <int D>
static void launch_decode(const bf16_t* q, const bf16_t* kc, const bf16_t* vc, const int* item_ctx, const int* table,
                          int width, float* part_o, float* part_ml, int items, int nh, int nkv, int bs, int window,
                          float scale_log2, int split_keys, int num_splits, hipStream_t stream) {
  const int chunks = (nh / nkv + 15) / 16;
  dim3 grid(items, nkv * chunks, num_splits);
  attention_decode_kernel<D><<<grid, 64, 0, stream>>>(q, kc, vc, item_ctx, table, width, part_o, part_ml, nh, nkv, bs,
                                                      window, scale_log2, split_keys, num_splits, chunks);
}

extern "C" int me_attention_mfma_supported(int d, int bs) {
  return (d == 32 || d == 64 || d == 96 || d == 128 || d == 192 || d == 256) && bs > 0 && bs % 16 == 0;
}

// q [items, nh, d] (one token per item), item_ctx[i] = keys of item i including the new one,
// workspace: part_o float [items * nh * num_splits * d], part_ml float [items * nh * num_splits * 2].
// Split s covers keys [s * split_keys, (s+1) * split_keys); num_splits * split_keys must cover every
// context the step can hold (max_ctx).
extern "C" int me_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                                        const int* block_table, int table_width, void* out, float* part_o,
                                        float* part_ml, int items, int nh, int nkv, int d, int bs, int window,
                                        float scale, int split_keys, int num_splits, int max_ctx,
                                        hipStream_t stream) {
  if (items <= 0) return 0;
  if (!me_attention_mfma_supported(d, bs))
    return me_fail("me_attention_decode_bf16: head_dim=%d / block_size=%d not supported by the matrix-core kernels", d, bs);
  if (nh <= 0 || nkv <= 0 || nh % nkv) return me_fail("me_attention_decode_bf16: nh=%d nkv=%d", nh, nkv);
  if (split_keys <= 0 || split_keys % 16 || num_splits <= 0 || (long long)split_keys * num_splits < max_ctx)
    return me_fail("me_attention_decode_bf16: %d splits of %d keys do not cover %d keys", num_splits, split_keys, max_ctx);
  if (table_width * bs < max_ctx)
    return me_fail("me_attention_decode_bf16: block table of %d pages of %d cannot hold %d keys", table_width, bs, max_ctx);
  if (num_splits > ME_MAX_SPLITS) return me_fail("me_attention_decode_bf16: %d splits exceed %d", num_splits, ME_MAX_SPLITS);
  if (num_splits > 65535 || nkv * ((nh / nkv + 15) / 16) > 65535) return me_fail("me_attention_decode_bf16: grid too large");
  const float sl = scale * LOG2E;
  const bf16_t *qq = (const bf16_t*)q, *kc = (const bf16_t*)k_cache, *vc = (const bf16_t*)v_cache;
#define ME_DECODE_CASE(DD)                                                                                      \
  case DD:                                                                                                      \
    launch_decode<DD>(qq, kc, vc, item_ctx, block_table, table_width, part_o, part_ml, items, nh, nkv, bs, window, sl, \
                      split_keys, num_splits, stream);                                                          \
    break;
  switch (d) {
    ME_DECODE_CASE(32)
    ME_DECODE_CASE(64)
    ME_DECODE_CASE(96)
    ME_DECODE_CASE(128)
    ME_DECODE_CASE(192)
    ME_DECODE_CASE(256)
  }
#undef ME_DECODE_CASE
  if (me_check_launch("me_attention_decode_bf16")) return 1;
  attention_decode_combine_kernel<<<items * nh, 256, 0, stream>>>(part_o, part_ml, (bf16_t*)out, num_splits, d);
  return me_check_launch("me_attention_decode_combine");
}

// ------------------------------------------------------------------------------------ prefill
// Block = 4 waves; a block owns the query columns of `tokens_per_block = 128 / group` consecutive
// new tokens of one item for one kv head (column c -> token c / group, head c % group); wave w owns
// columns 32w .. 32w+31 as two blocks of 16. Blocks are numbered over all items: item i has
// ceil(qlen_i / tokens_per_block) of them.
template <int D>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ item_start, int num_items,
    const int* __restrict__ block_table, int table_width, bf16_t* __restrict__ out, int nh, int nkv, int bs,
    int window, float scale_log2, int tokens_per_block) {
  __shared__ int s_item, s_tile;
  if (threadIdx.x == 0) {
    int left = blockIdx.x, it = 0;
    for (; it < num_items; ++it) {
      const int tiles = (item_start[it + 1] - item_start[it] + tokens_per_block - 1) / tokens_per_block;
      if (left < tiles) break;
      left -= tiles;
    }
    s_item = it;
    s_tile = left;
  }
  __syncthreads();
  const int item = s_item;
  if (item >= num_items) return;
  const int kvh = blockIdx.y;
  const int group = nh / nkv;
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int t_begin = item_start[item] + s_tile * tokens_per_block;
  const int t_end = min(item_start[item + 1], t_begin + tokens_per_block);

  // this lane's query column in each of the wave's two blocks
  int tok[2], head[2], qpos[2];
  bool col_ok[2];
  int wave_max_pos = -1, wave_min_pos = 0x7fffffff;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int c = wave * 32 + nb * 16 + r;
    tok[nb] = t_begin + c / group;
    head[nb] = kvh * group + c % group;
    col_ok[nb] = c < tokens_per_block * group && tok[nb] < t_end;
    qpos[nb] = col_ok[nb] ? positions[tok[nb]] : -1;
  }
  {
    int mx = max(qpos[0], qpos[1]);
    int mn = min(col_ok[0] ? qpos[0] : 0x7fffffff, col_ok[1] ? qpos[1] : 0x7fffffff);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      mx = max(mx, __shfl_xor(mx, off, ME_WAVE));
      mn = min(mn, __shfl_xor(mn, off, ME_WAVE));
    }
    wave_max_pos = mx;
    wave_min_pos = mn;
  }
  if (wave_max_pos < 0) return;  // no column of this wave is in use

  Frag8 qf[2][D / 32];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      qf[nb][c].u = make_uint4(0, 0, 0, 0);
      if (col_ok[nb])
        qf[nb][c].u = *reinterpret_cast<const uint4*>(q + ((size_t)tok[nb] * nh + head[nb]) * D + c * 32 + g * 8);
    }
  float m[2] = {-INFINITY, -INFINITY}, lsum[2] = {0.f, 0.f};
  float4_t acc[2][D / 16];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) acc[nb][dt] = (float4_t){0.f, 0.f, 0.f, 0.f};

  // every column of the wave sees keys from its own lo; the lowest one bounds the loop
  const int lo_min = window > 0 ? max(wave_min_pos - window + 1, 0) : 0;
  const int* table = block_table + (size_t)item * table_width;
  // the four values a lane holds belong to one column, so the window's lower bound is per lane too
  int lo_col[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) lo_col[nb] = window > 0 ? max(qpos[nb] - window + 1, 0) : 0;

  for (int key0 = (lo_min / 16) * 16; key0 <= wave_max_pos; key0 += 16) {
    int page = table[key0 / bs];
    page = page < 0 ? 0 : page;
    const int off = key0 % bs;
    const bf16_t* kbase = k_cache + (((size_t)page * nkv + kvh) * bs + off) * D;
    const bf16_t* vbase = v_cache + ((size_t)page * nkv + kvh) * D * bs + off;
    const bool need_mask = key0 + 15 > wave_min_pos || window > 0;
    if (window > 0) {
      // per-column lower bounds differ: mask with the larger of the two inside attend_tile by
      // passing lo = 0 and folding the bound into qpos is not possible, so do the tile per block
      const int q0[1] = {qpos[0]}, q1[1] = {qpos[1]};
      attend_tile<D, 1>(kbase, vbase, bs, key0, lo_col[0], q0, true, reinterpret_cast<const Frag8(&)[1][D / 32]>(qf[0]),
                        scale_log2, reinterpret_cast<float(&)[1]>(m[0]), reinterpret_cast<float(&)[1]>(lsum[0]),
                        reinterpret_cast<float4_t(&)[1][D / 16]>(acc[0]));
      attend_tile<D, 1>(kbase, vbase, bs, key0, lo_col[1], q1, true, reinterpret_cast<const Frag8(&)[1][D / 32]>(qf[1]),
                        scale_log2, reinterpret_cast<float(&)[1]>(m[1]), reinterpret_cast<float(&)[1]>(lsum[1]),
                        reinterpret_cast<float4_t(&)[1][D / 16]>(acc[1]));
    } else {
      attend_tile<D, 2>(kbase, vbase, bs, key0, 0, qpos, need_mask, qf, scale_log2, m, lsum, acc);
    }
  }
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    if (!col_ok[nb]) continue;
    const float inv = 1.f / lsum[nb];
    bf16_t* orow = out + ((size_t)tok[nb] * nh + head[nb]) * D;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      const short4_t o = pack_bf16x4(acc[nb][dt][0] * inv, acc[nb][dt][1] * inv, acc[nb][dt][2] * inv,
                                     acc[nb][dt][3] * inv);
      *reinterpret_cast<short4_t*>(orow + dt * 16 + g * 4) = o;
    }
  }
}

// q [T, nh, d]; item_start int [items + 1] (offsets of the items' tokens); positions int [T];
// num_blocks = sum over items of ceil(qlen / (128 / group)), computed by the caller.
extern "C" int me_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                         const int* item_start, int num_items, const int* block_table, int table_width,
                                         void* out, int num_blocks, int nh, int nkv, int d, int bs, int window,
                                         float scale, hipStream_t stream) {
  if (num_items <= 0 || num_blocks <= 0) return 0;
  if (!me_attention_mfma_supported(d, bs))
    return me_fail("me_attention_prefill_bf16: head_dim=%d / block_size=%d not supported by the matrix-core kernels", d, bs);
  if (nh <= 0 || nkv <= 0 || nh % nkv) return me_fail("me_attention_prefill_bf16: nh=%d nkv=%d", nh, nkv);
  const int group = nh / nkv;
  if (group > 16) return me_fail("me_attention_prefill_bf16: group size %d exceeds 16", group);
  if (nkv > 65535) return me_fail("me_attention_prefill_bf16: %d kv heads exceed the grid", nkv);
  const int tpb = 128 / group;
  const float sl = scale * LOG2E;
  dim3 grid(num_blocks, nkv);
  const bf16_t *qq = (const bf16_t*)q, *kc = (const bf16_t*)k_cache, *vc = (const bf16_t*)v_cache;
#define ME_PREFILL_CASE(DD)                                                                                        \
  case DD:                                                                                                         \
    attention_prefill_kernel<DD><<<grid, 256, 0, stream>>>(qq, kc, vc, positions, item_start, num_items, block_table, \
                                                           table_width, (bf16_t*)out, nh, nkv, bs, window, sl, tpb); \
    break;
  switch (d) {
    ME_PREFILL_CASE(32)
    ME_PREFILL_CASE(64)
    ME_PREFILL_CASE(96)
    ME_PREFILL_CASE(128)
    ME_PREFILL_CASE(192)
    ME_PREFILL_CASE(256)
  }
#undef ME_PREFILL_CASE
  return me_check_launch("me_attention_prefill_bf16");
}
