// Causal grouped-query attention over the paged cache, for any mix of items in a step: one wave, or a
// block of eight, per (new token, query head). It takes every size the cache allows (any page size, any group
// size, head sizes up to 256 in steps of 2) in float32 or bfloat16 storage, and is the kernel of
// the 32-bit path; the bfloat16 path uses the matrix-core kernels where their size limits hold.
//
// A token at absolute position p of item b sees keys lo..p of item b, lo = max(0, p - window + 1)
// (window == 0: lo = 0). Keys are visited in tiles of 64 aligned to absolute position (tile t holds
// positions 64t .. 64t+63), four tiles to a chunk (chunk c holds positions 256c .. 256c+255): the tiles of a
// chunk update a running (maximum, sum, weighted values) from nothing, and the chunks' results are merged in
// ascending order. So the order of every sum depends on p, lo and the head alone, never on how the sequence
// was cut into steps, on what else is in the batch, or on how many waves share the chunks of a token.
//
// Cache layout per layer: keys K[page, kv_head, slot, d]; values transposed V[page, kv_head, d, slot].
#include "common.h"

#define AG_MAX_D 256

#define AG_CHUNK 256  // keys per chunk

// One chunk's result into the running one, the same operations wherever it is called. With nothing before
// (mt = -inf, lt = 0, acct = 0) the chunk's result comes through unchanged: exp(-inf) = 0 and exp(0) = 1.
template <int KMAX>
__device__ __forceinline__ void ag_merge(float& mt, float& lt, float (&acct)[KMAX], float mc, float lc,
                                         const float (&accc)[KMAX]) {
  const float mn = fmaxf(mt, mc);
  const float at = expf(mt - mn), ac = expf(mc - mn);
  lt = fmaf(lt, at, lc * ac);
#pragma unroll
  for (int k = 0; k < KMAX; ++k) acct[k] = fmaf(acct[k], at, accc[k] * ac);
  mt = mn;
}

// `wpu` waves per (token, head): 1 (a block of four waves serves four of them), or all waves of the block for one,
// which then take the chunks in turns, a round of wpu chunks at a time, and wave 0 merges the round's results in order.
template <typename T>
__global__ __launch_bounds__(512) void attention_general_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table,
    int table_width, T* __restrict__ out, int num_tokens, int nh, int nkv, int d, int bs, int window, float scale, int wpu) {
  constexpr int KMAX = AG_MAX_D / ME_WAVE;
  __shared__ float qs[8][AG_MAX_D];
  __shared__ float parts[8][AG_MAX_D + 2];  // with several waves per unit: a round's results (values, maximum, sum)
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int w = wave % wpu;
  const long long unit = (long long)blockIdx.x * (blockDim.x / ME_WAVE / wpu) + wave / wpu;
  if (unit >= (long long)num_tokens * nh) return;  // (with several waves per unit: the whole block)
  const int t = (int)(unit / nh), head = (int)(unit % nh);
  const int kvh = head / (nh / nkv);
  const int p = positions[t];
  const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int* table = block_table + (size_t)token_item[t] * table_width;

  const T* qrow = q + ((size_t)t * nh + head) * d;
  float* qw = qs[wave];
  for (int i = lane; i < d; i += ME_WAVE) qw[i] = to_float(qrow[i]) * scale;
  __builtin_amdgcn_wave_barrier();

  float mt = -INFINITY, lt = 0.f;
  float acct[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; ++k) acct[k] = 0.f;

  const bool vec_k = sizeof(T) == 4 && d % 4 == 0 && ((uintptr_t)k_cache & 15) == 0;   // a key row in 16-byte pieces
  const bool vec_v = sizeof(T) == 4 && bs % 4 == 0 && ((uintptr_t)v_cache & 15) == 0;  // four keys of a value row at once
  const int first_chunk = lo / AG_CHUNK, n_chunks = p / AG_CHUNK - first_chunk + 1;
  for (int round = 0; round * wpu < n_chunks; ++round) {
    const int ci = round * wpu + w;  // this wave's chunk of the round, if there is one
    float m = -INFINITY, l = 0.f;
    float acc[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) acc[k] = 0.f;
    const int chunk0 = (first_chunk + ci) * AG_CHUNK;
    const int tile_first = ci < n_chunks ? max(chunk0, (lo / 64) * 64) : 1;  // (no chunk left for this wave: no tiles)
    const int tile_last = ci < n_chunks ? min(p, chunk0 + AG_CHUNK - 1) : 0;
    for (int tile = tile_first; tile <= tile_last; tile += 64) {
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
    if (wpu == 1) {
      ag_merge<KMAX>(mt, lt, acct, m, l, acc);
    } else {  // the round's results go through LDS to wave 0, which merges them in the order of their chunks
      if (ci < n_chunks) {
#pragma unroll
        for (int k = 0; k < KMAX; ++k) parts[w][lane + k * ME_WAVE] = acc[k];
        if (lane == 0) parts[w][AG_MAX_D] = m, parts[w][AG_MAX_D + 1] = l;
      }
      __syncthreads();
      if (w == 0)
        for (int o = 0; o < wpu && round * wpu + o < n_chunks; ++o) {
          float accc[KMAX];
#pragma unroll
          for (int k = 0; k < KMAX; ++k) accc[k] = parts[o][lane + k * ME_WAVE];
          ag_merge<KMAX>(mt, lt, acct, parts[o][AG_MAX_D], parts[o][AG_MAX_D + 1], accc);
        }
      __syncthreads();
    }
  }
  if (w != 0) return;
  T* orow = out + ((size_t)t * nh + head) * d;
  const float inv = 1.f / lt;
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int i = lane + k * ME_WAVE;
    if (i < d) orow[i] = from_float<T>(acct[k] * inv);
  }
}

// The same attention for steps that bring several tokens per item (prompts, portions): a block takes up to
// `tq` consecutive tokens of the step and the heads of one kv head, a wave per (token, head), and stages each tile of
// 64 keys and values in LDS once for all of them, where the kernel above has every wave fetch its own copy (a 2,048-token
// prompt: 34 GB a layer from the L2). Tokens of a block that belong to different items are served one item after the
// other. Every wave does the arithmetic of the kernel above in the same order (the products of a score in ascending
// element, the keys of a tile in ascending position, the same reductions across lanes), so the two kernels give the same
// bits and a step may use either. float32, head sizes that are a multiple of 4, pages that hold a multiple of 4 keys.
constexpr int AS_KPAD = 4, AS_VROW = 68;  // LDS rows: a key's d + 4 floats, an element's 64 + 4 keys (16-byte reads of consecutive
                                           // rows by consecutive lanes without bank conflicts; 8 and 72 measured slower)

// DT: the head size if it is 64, 128 or 256 (loops unroll, no guards), else 0 (any multiple of 4 up to 256).
template <int DT>
__global__ __launch_bounds__(1024) void attention_shared_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k_cache, const float* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table,
    int table_width, float* __restrict__ out, int num_tokens, int nh, int nkv, int d_any, int bs, int bs_shift, int window,
    float scale, int tq) {
  constexpr int KMAX = DT ? DT / ME_WAVE : AG_MAX_D / ME_WAVE;  // elements of the output per lane
  const int d = DT ? DT : d_any, d4 = d / 4;
  extern __shared__ __attribute__((aligned(16))) float as_lds[];
  const int waves = blockDim.x / ME_WAVE;
  float* Ks = as_lds;                      // [64][d + AS_KPAD]
  float* Vs = Ks + 64 * (d + AS_KPAD);     // [d][AS_VROW]
  float* qs = Vs + (size_t)d * AS_VROW;    // [waves][d]
  float* ps = qs + (size_t)waves * d;      // [waves][64]: a tile's weights, for every lane to read
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / ME_WAVE), lane = threadIdx.x & (ME_WAVE - 1);
  const int group = nh / nkv, kvh = blockIdx.y;
  // (the step's last tokens first: they are the ones with the most keys before them, and blocks start in this order)
  const int first = (gridDim.x - 1 - blockIdx.x) * tq, limit = min(first + tq, num_tokens);
  const int t = first + wave / group, head = kvh * group + wave % group;
  const bool mine = wave < tq * group && t < limit;
  float* qw = qs + (size_t)wave * d;
  float* pw = ps + wave * 64;
  const int krow_floats = d + AS_KPAD;
  // staging: a wave copies whole key rows, 64 / dp rows at a time (dp: d4 rounded up to a power of two, lanes beyond d4 idle)
  int dp_shift = 0;
  while ((1 << dp_shift) < d4) ++dp_shift;
  const int k_rows_per_wave = ME_WAVE >> dp_shift, k_row_in_wave = lane >> dp_shift, k_piece = lane & ((1 << dp_shift) - 1);
  auto page_of = [&](int key, int& slot) {
    if (bs_shift >= 0) {
      slot = key & (bs - 1);
      return key >> bs_shift;
    }
    slot = key % bs;
    return key / bs;
  };

  for (int seg = first; seg < limit;) {  // runs of tokens of one item (every thread walks the same runs)
    const int item = token_item[seg];
    int seg_end = seg + 1;
    while (seg_end < limit && token_item[seg_end] == item) ++seg_end;
    const int* table = block_table + (size_t)item * table_width;
    int p_first = positions[seg], p_last = p_first;  // the run's lowest and highest position (a portion's are consecutive)
    for (int i = seg + 1; i < seg_end; ++i) p_first = min(p_first, positions[i]), p_last = max(p_last, positions[i]);
    const int lo_first = window > 0 ? max(p_first - window + 1, 0) : 0;
    const bool active = mine && t >= seg && t < seg_end;
    const int p = active ? __builtin_amdgcn_readfirstlane(positions[t]) : 0;
    const int lo = window > 0 ? max(p - window + 1, 0) : 0;
    if (active) {
      const float* qrow = q + ((size_t)t * nh + head) * d;
      for (int i = lane; i < d; i += ME_WAVE) qw[i] = qrow[i] * scale;
    }
    float m = -INFINITY, l = 0.f, mt = -INFINITY, lt = 0.f;  // the chunk in hand, and the chunks before it merged
    float acc[KMAX], acct[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) acc[k] = 0.f, acct[k] = 0.f;

    for (int tile = (lo_first / 64) * 64; tile <= p_last; tile += 64) {
      __syncthreads();  // every wave has left the tile before (and the q rows are written)
      for (int row = wave * k_rows_per_wave + k_row_in_wave; row < 64; row += waves * k_rows_per_wave) {
        const int key = tile + row;  // keys up to the last position of the run
        if (key <= p_last && k_piece < d4) {
          int slot;
          const int page = table[page_of(key, slot)];
          const float* src = k_cache + (((size_t)page * nkv + kvh) * bs + slot) * d + 4 * k_piece;
          *reinterpret_cast<float4*>(Ks + row * krow_floats + 4 * k_piece) = *reinterpret_cast<const float4*>(src);
        }
      }
      for (int idx = threadIdx.x; idx < d * 16; idx += blockDim.x) {  // four keys of an element at a time (they share a page)
        const int i = idx >> 4, key = tile + 4 * (idx & 15);
        if (key <= p_last) {
          int slot;
          const int page = table[page_of(key, slot)];
          const float* src = v_cache + ((size_t)page * nkv + kvh) * d * bs + (size_t)i * bs + slot;
          *reinterpret_cast<float4*>(Vs + i * AS_VROW + 4 * (idx & 15)) = *reinterpret_cast<const float4*>(src);
        }
      }
      __syncthreads();
      if (!active || tile > p || tile < (lo / 64) * 64) continue;
      if (tile % AG_CHUNK == 0 && tile > lo) {  // a chunk begins behind another one of this token: that one is complete
        ag_merge<KMAX>(mt, lt, acct, m, l, acc);
        m = -INFINITY, l = 0.f;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) acc[k] = 0.f;
      }
      const int key = tile + lane;
      const bool valid = key >= lo && key <= p;
      float s = -INFINITY;
      if (valid) {
        const float4* k4 = reinterpret_cast<const float4*>(Ks + lane * krow_floats);
        const float4* q4 = reinterpret_cast<const float4*>(qw);
        float dot = 0.f;
        for (int base = 0; base < d4; base += 8) {  // eight pieces of the row and of q are requested before the first is used
          float4 kv[8], qv[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int at = DT || base + u < d4 ? base + u : d4 - 1;
            kv[u] = k4[at], qv[u] = q4[at];
          }
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (DT || base + u < d4) {
              dot = fmaf(qv[u].x, kv[u].x, dot);
              dot = fmaf(qv[u].y, kv[u].y, dot);
              dot = fmaf(qv[u].z, kv[u].z, dot);
              dot = fmaf(qv[u].w, kv[u].w, dot);
            }
        }
        s = dot;
      }
      const float m_new = fmaxf(m, wave_max(s));
      const float pr = valid ? expf(s - m_new) : 0.f;
      const float alpha = expf(m - m_new);
      l = l * alpha + wave_sum(pr);
#pragma unroll
      for (int k = 0; k < KMAX; ++k) acc[k] *= alpha;
      m = m_new;
      pw[lane] = pr;
      __builtin_amdgcn_wave_barrier();
      const int j_lo = lo > tile ? lo - tile : 0;
      const int j_hi = p - tile < 63 ? p - tile : 63;
      int j = j_lo;
      for (; j <= j_hi && (j & 3); ++j) {
        const float pj = pw[j];
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (DT || i < d) acc[k] = fmaf(pj, Vs[i * AS_VROW + j], acc[k]);
        }
      }
      for (; j + 15 <= j_hi; j += 16) {  // four groups of four keys: their values are requested before the first is used
        float4 vv[4][KMAX], pv[4];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          pv[gq] = *reinterpret_cast<const float4*>(pw + j + 4 * gq);
#pragma unroll
          for (int k = 0; k < KMAX; ++k) {
            const int i = lane + k * ME_WAVE;
            vv[gq][k] = *reinterpret_cast<const float4*>(Vs + (DT || i < d ? i : 0) * AS_VROW + j + 4 * gq);
          }
        }
#pragma unroll
        for (int gq = 0; gq < 4; ++gq)
#pragma unroll
          for (int k = 0; k < KMAX; ++k)
            if (DT || lane + k * ME_WAVE < d) {
              acc[k] = fmaf(pv[gq].x, vv[gq][k].x, acc[k]);
              acc[k] = fmaf(pv[gq].y, vv[gq][k].y, acc[k]);
              acc[k] = fmaf(pv[gq].z, vv[gq][k].z, acc[k]);
              acc[k] = fmaf(pv[gq].w, vv[gq][k].w, acc[k]);
            }
      }
      for (; j + 3 <= j_hi; j += 4) {
        const float4 pv = *reinterpret_cast<const float4*>(pw + j);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (DT || i < d) {
            const float4 vv = *reinterpret_cast<const float4*>(Vs + i * AS_VROW + j);
            acc[k] = fmaf(pv.x, vv.x, acc[k]);
            acc[k] = fmaf(pv.y, vv.y, acc[k]);
            acc[k] = fmaf(pv.z, vv.z, acc[k]);
            acc[k] = fmaf(pv.w, vv.w, acc[k]);
          }
        }
      }
      for (; j <= j_hi; ++j) {
        const float pj = pw[j];
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (DT || i < d) acc[k] = fmaf(pj, Vs[i * AS_VROW + j], acc[k]);
        }
      }
    }
    if (active) {
      ag_merge<KMAX>(mt, lt, acct, m, l, acc);  // the last chunk
      float* orow = out + ((size_t)t * nh + head) * d;
      const float inv = 1.f / lt;
#pragma unroll
      for (int k = 0; k < KMAX; ++k) {
        const int i = lane + k * ME_WAVE;
        if (DT || i < d) orow[i] = acct[k] * inv;
      }
    }
    seg = seg_end;
  }
}

// `items`: how many items the step's tokens belong to (0: unknown). Steps with two and more tokens per item on
// average go to the kernel that shares the tiles of keys and values among the tokens of a block; the results are
// the same bits either way.
extern "C" int me_attention_general(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                    const int* token_item, const int* block_table, int table_width, void* out,
                                    int num_tokens, int nh, int nkv, int d, int bs, int window, float scale,
                                    int dtype, int items, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (d <= 0 || d > AG_MAX_D) return me_fail("me_attention_general: head_dim=%d must be in 1..%d", d, AG_MAX_D);
  if (nh <= 0 || nkv <= 0 || nh % nkv)
    return me_fail("me_attention_general: %d query heads are not a multiple of %d key/value heads", nh, nkv);
  if (bs <= 0 || table_width <= 0 || window < 0)
    return me_fail("me_attention_general: block_size=%d table_width=%d window=%d", bs, table_width, window);
  const int group = nh / nkv;
  if (dtype == ME_F32 && items > 0 && num_tokens >= 2 * items && d % 4 == 0 && bs % 4 == 0 && group <= 16 &&
      (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0) {
    const int tq = 16 / group > 0 ? 16 / group : 1, waves = tq * group;
    const size_t lds = ((size_t)64 * (d + AS_KPAD) + (size_t)d * AS_VROW + (size_t)waves * (d + 64)) * sizeof(float);
    int bs_shift = -1;
    if ((bs & (bs - 1)) == 0)
      for (bs_shift = 0; (1 << bs_shift) < bs;) ++bs_shift;
    const dim3 grid((num_tokens + tq - 1) / tq, nkv);
#define ME_SHARED_LAUNCH(DT)                                                                                                     \
  do {                                                                                                                           \
    static size_t allowed = 0; /* grows to the most this head size has asked for */                                             \
    if (lds > allowed) {                                                                                                         \
      if (hipFuncSetAttribute((const void*)attention_shared_f32_kernel<DT>, hipFuncAttributeMaxDynamicSharedMemorySize,          \
                              (int)lds) != hipSuccess)                                                                           \
        return me_fail("me_attention_general: %zu bytes of block memory for head_dim=%d are refused", lds, d);                   \
      allowed = lds;                                                                                                             \
    }                                                                                                                            \
    attention_shared_f32_kernel<DT><<<grid, waves * 64, lds, stream>>>(                                                          \
        (const float*)q, (const float*)k_cache, (const float*)v_cache, positions, token_item, block_table, table_width,         \
        (float*)out, num_tokens, nh, nkv, d, bs, bs_shift, window, scale, tq);                                                   \
  } while (0)
    if (d == 64)
      ME_SHARED_LAUNCH(64);
    else if (d == 128)
      ME_SHARED_LAUNCH(128);
    else if (d == 256)
      ME_SHARED_LAUNCH(256);
    else
      ME_SHARED_LAUNCH(0);
#undef ME_SHARED_LAUNCH
    return me_check_launch("me_attention_general");
  }
  const long long units = (long long)num_tokens * nh;
  // few units (decode steps): a block of eight waves each, which share a token's chunks of keys; else four units a block
  const int wpu = units < 2048 ? 8 : 1, waves = units < 2048 ? 8 : 4;
  const unsigned blocks = (unsigned)((units + waves / wpu - 1) / (waves / wpu));
  if (dtype == ME_F32)
    attention_general_kernel<float><<<blocks, waves * 64, 0, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, positions, token_item, block_table,
        table_width, (float*)out, num_tokens, nh, nkv, d, bs, window, scale, wpu);
  else
    attention_general_kernel<bf16_t><<<blocks, waves * 64, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, token_item, block_table,
        table_width, (bf16_t*)out, num_tokens, nh, nkv, d, bs, window, scale, wpu);
  return me_check_launch("me_attention_general");
}
