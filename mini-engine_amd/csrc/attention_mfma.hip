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

// Four values rounded to bfloat16 (to nearest even) by the hardware's conversion, two per instruction (rounded by
// integer arithmetic, six instructions a value, the decode kernel's tile took a fifth longer: a decode step at batch 8
// 1.704 -> 1.657 ms, at batch 64 5.94 -> 5.75, at batch 1 0.991 -> 0.972).
__device__ __forceinline__ short4_t pack_bf16x4(float a, float b, float c, float d) {
  typedef __bf16 packed_t __attribute__((ext_vector_type(4)));
  const packed_t r = {(__bf16)a, (__bf16)b, (__bf16)c, (__bf16)d};
  return __builtin_bit_cast(short4_t, r);
}

// max / sum over the four lanes that share a query column (l%16 fixed, l/16 = 0..3). The row swaps
// of gfx950 (v_permlane16_swap, v_permlane32_swap) hand every lane its partner's value at vector-ALU
// speed: after a swap of a register with a copy of itself, the two results hold, in every lane, the
// lane's own value and that of lane ^ 16 (resp. lane ^ 32), in one order or the other.
typedef unsigned uint2v_t __attribute__((ext_vector_type(2)));
typedef unsigned uint4v_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float column_max(float v) {
  unsigned u = __float_as_uint(v);
  uint2v_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  u = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
  a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
}
__device__ __forceinline__ float column_sum(float v) {
  unsigned u = __float_as_uint(v);
  uint2v_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  u = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(a[0]) + __uint_as_float(a[1]);
}

#define LOG2E 1.4426950408889634f

// One 16-key tile for NB blocks of 16 query columns, in two halves so that a caller can have the
// loads of the next tile in flight while it computes on this one. `kbase` points at
// K[page, kvh, off, 0], `vbase` at V^T[page, kvh, 0, off]. key0 is the absolute position of the tile's
// first key. A key is visible to column nb if lo <= key <= qpos[nb].
template <int D>
struct KvTile {
  Frag8 kf[D / 32];
  short4_t vf[D / 16];
};

template <int D, bool STREAMED>
__device__ __forceinline__ void load_tile(KvTile<D>& t, const bf16_t* __restrict__ kbase,
                                          const bf16_t* __restrict__ vbase, int bs) {
  const int lane = threadIdx.x & (ME_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  if constexpr (STREAMED) {  // non-temporal loads: for launches that stream hundreds of megabytes once (the host decides)
#pragma unroll
    for (int c = 0; c < D / 32; ++c) t.kf[c].u = stream_load16(kbase + (size_t)r * D + c * 32 + g * 8);
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      t.vf[dt] = __builtin_bit_cast(short4_t, stream_load8(vbase + (size_t)(dt * 16 + r) * bs + g * 4));
    return;
  }
#pragma unroll
  for (int c = 0; c < D / 32; ++c) t.kf[c].u = *reinterpret_cast<const uint4*>(kbase + (size_t)r * D + c * 32 + g * 8);
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
    t.vf[dt] = *reinterpret_cast<const short4_t*>(vbase + (size_t)(dt * 16 + r) * bs + g * 4);
}

template <int D, int NB>
__device__ __forceinline__ void compute_tile(const KvTile<D>& t, int key0, int lo, const int (&qpos)[NB],
                                             bool need_mask, const Frag8 (&qf)[NB][D / 32], float scale_log2,
                                             float (&m)[NB], float (&lsum)[NB], float4_t (&acc)[NB][D / 16]) {
  const int lane = threadIdx.x & (ME_WAVE - 1);
  const int g = lane >> 4;
  short4_t pf[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.kf[c].h[0], qf[nb][c].h[0], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.kf[c].h[1], qf[nb][c].h[1], s, 0, 0, 0);
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
    // (the column's sum per tile: with the four lanes of a column keeping sums of their own until the split is done,
    // as the prefill kernel does, steps at batch 1 and 64 are 0.5-0.9% longer and only long contexts gain)
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
      acc[nb][dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.vf[dt], pf[nb], acc[nb][dt], 0, 0, 0);
}

// ------------------------------------------------------------------------------------- decode
// Partial results: part_o [items, nh, splits, D] (unnormalised), part_ml [items, nh, splits, 2].
//
// FUSED: the kernel starts from the raw output of the q/k/v projection, qkv [items, (nh + 2 nkv) D],
// and does the per-head RMSNorm and the rotary encoding itself (what me_qk_norm_rope_scatter does
// for steps with longer items), in float32 with one rounding at the end:
//   * every block norms and rotates the query heads it owns, straight into matrix-core operands
//     (a lane's eight dims of a 32-wide chunk and their rotary partners, half a head away, sit in
//     the same lane when D is a multiple of 64);
//   * the block whose split holds the item's newest position also norms and rotates the new key,
//     writes it and the new value into their page, and waits for those stores before it reads that
//     page. No other block of the step reads that slot.
struct DecodeFusedArgs {
  const float* q_w;         // [D] or null: no q/k norm
  const float* k_w;         // [D] or null
  const float* rope_table;  // [positions, 2, D/2] or null: no rotary
  float eps;
  int write_kv;             // 0: a layer that reads another layer's cache
  bf16_t* k_cache_w;
  bf16_t* v_cache_w;
};

// Tiles of a split from which on a wave fetches one tile at a time, whatever DEPTH says: with five tiles and more of its own
// a wave streams best without a tile requested ahead, since the other waves of its SIMD fill the gaps (measured with 16, 12,
// 8, 4 and 1 here: batch 8 at contexts of 4,096 / 2,304 1.881 / 1.526 ms a step with 16, 1.851 / 1.505 with 4; batch 16 at
// 1,024 1.538 -> 1.512; batch 64 at 512 2.047 -> 2.031; with 1, splits of two tiles lose: batch 1 1.040 -> 1.079).
#define LONG_RUN 4

// Most splits that one block takes on, a wave each. Heads beyond 128 need more than 256 registers a lane
// with two tiles in flight, which only blocks of at most four waves (one per SIMD) may have.
#define DECODE_BLOCK_WAVES(D) ((D) <= 128 ? 8 : 4)

template <int D, bool FUSED, int DEPTH, bool STREAMED>
__device__ __forceinline__ void attention_decode_body(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ item_ctx, const int* __restrict__ block_table, int table_width,
    float* __restrict__ part_o, float* __restrict__ part_ml, bf16_t* __restrict__ out, int nh, int nkv, int bs_shift,
    int window, float scale_log2, int num_splits, int head_chunks, const DecodeFusedArgs& fa,
    const int* __restrict__ live_items, int waves_wanted) {
  extern __shared__ float decode_lds[];  // only with several waves a block: their results, to be added up
  const int bs = 1 << bs_shift;
  const int item = blockIdx.x;
  const int kvh = blockIdx.y / head_chunks, chunk = blockIdx.y % head_chunks;
  // the wave's number as a scalar: everything that follows from it (the split, its keys, the loop over them)
  // stays uniform for the compiler
  const int block_waves = blockDim.x / ME_WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / ME_WAVE);
  const int split = blockIdx.z * block_waves + wave;  // num_splits = gridDim.z * block_waves
  const int group = nh / nkv;
  const int lane = threadIdx.x & (ME_WAVE - 1), r = lane & 15, g = lane >> 4;
  const int heads_here = min(16, group - chunk * 16);
  const int head0 = kvh * group + chunk * 16;
  const int* table = block_table + (size_t)item * table_width;
  auto fetch = [&](KvTile<D>& t, int key0) {
    int page = table[min(key0 >> bs_shift, table_width - 1)];
    page = page < 0 ? 0 : page;
    const int off = key0 & (bs - 1);
    load_tile<D, STREAMED>(t, k_cache + (((size_t)page * nkv + kvh) * bs + off) * D,
                           v_cache + ((size_t)page * nkv + kvh) * D * bs + off, bs);
  };
  KvTile<D> t[DEPTH];
  // The keys of an item, from its window's first (rounded down to a tile of 16) to its newest, are dealt
  // to the splits in equal runs of whole tiles: every split has work whatever the item's length is
  // (the grid is sized for the longest context the step may hold, often many times the actual one).
  const int ctx = item_ctx[item];
  // A launch that was laid out for fewer items than the grid holds (a replayed graph whose last items
  // are padding) has more splits than this step needs: the live items share `waves_wanted` waves, and
  // the splits beyond that come out empty.
  int splits = num_splits;
  if (live_items) {
    const int units = max(live_items[0], 1) * (int)gridDim.y;
    splits = min(num_splits, max(1, (waves_wanted + units - 1) / units));
  }
  const int lo = window > 0 ? max(ctx - window, 0) : 0;
  const int lo16 = (lo / 16) * 16;
  int tiles_per_split = ((ctx - lo16 + 15) / 16 + splits - 1) / splits;
  // With 16 splits and more per item, runs of 16, 32, 48 or 64 tiles (the waves of an item then start at keys a multiple of 256
  // apart and walk them in step) measured slower than runs one tile longer with a split less at work, on the same GPU in turns:
  // batch 8 at a context of 8,192 2.78 -> 2.44 ms a step, batch 4 at 8,192 1.98 -> 1.76, batch 8 at 4,096 1.83 -> 1.78 in a
  // pool of 2,304 pages and 1.766 -> 1.775 in one of 16,640; contexts that give other runs: no change. The cause is not
  // established (it depends on where the pages lie: a context of 3,968, whose runs are as long but whose last split is short,
  // shows no such loss; walking each run from a tile of its own and around its end, which takes the waves out of step
  // altogether, is slower everywhere but at 8,192). Longer runs gain nothing (128 tiles: 5.96 -> 6.09), and with fewer splits
  // the longer runs cost what they are longer (batch 16 at 4,096, 8 splits of 32 tiles: 2.374 -> 2.430), so those keep
  // theirs, and so do blocks that add up their own waves' splits.
  if (block_waves == 1 && splits >= 16 && tiles_per_split % 16 == 0 && tiles_per_split <= 64) ++tiles_per_split;
  const int begin = lo16 + split * tiles_per_split * 16;
  const int end = min(begin + tiles_per_split * 16, ctx);

  float m[1] = {-INFINITY}, lsum[1] = {0.f};
  float4_t acc[1][D / 16];
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt) acc[0][dt] = (float4_t){0.f, 0.f, 0.f, 0.f};

  if (begin < end) {
    // the first tile is requested before the query is prepared, unless it holds the slot that this
    // block is about to write
    const bool early = !FUSED || begin + 16 < ctx;
    if (early) fetch(t[0], begin);
    Frag8 qf[1][D / 32];
    if (FUSED) {
      constexpr int HC = D / 64;  // chunks per half head
      const int pos = ctx - 1;
      const size_t row = (size_t)item * (fa.write_kv ? nh + 2 * nkv : nh) * D;
      // ---- the new key and value of this kv head, by the block that will read them
      if (fa.write_kv && end == ctx) {
        const int page = table[pos >> bs_shift];
        if (page >= 0) {
          const int slot = pos & (bs - 1);
          const bf16_t* ksrc = q + row + (size_t)(nh + kvh) * D;
          const bf16_t* vsrc = q + row + (size_t)(nh + nkv + kvh) * D;
          float k1[(D / 2 + 63) / 64], k2[(D / 2 + 63) / 64];
          float ss = 0.f;
#pragma unroll
          for (int p = 0; p < (D / 2 + 63) / 64; ++p) {
            const int j = lane + 64 * p;
            k1[p] = j < D / 2 ? to_float(ksrc[j]) : 0.f;
            k2[p] = j < D / 2 ? to_float(ksrc[j + D / 2]) : 0.f;
            ss += k1[p] * k1[p] + k2[p] * k2[p];
          }
          const float inv = fa.k_w ? rsqrtf(wave_sum(ss) / (float)D + fa.eps) : 1.f;
          bf16_t* kdst = fa.k_cache_w + (((size_t)page * nkv + kvh) * bs + slot) * D;
          bf16_t* vdst = fa.v_cache_w + ((size_t)page * nkv + kvh) * D * bs + slot;
#pragma unroll
          for (int p = 0; p < (D / 2 + 63) / 64; ++p) {
            const int j = lane + 64 * p;
            if (j < D / 2) {
              float a = k1[p], b = k2[p];
              if (fa.k_w) {
                a = a * inv * fa.k_w[j];
                b = b * inv * fa.k_w[j + D / 2];
              }
              if (fa.rope_table) {
                const float c = fa.rope_table[(size_t)pos * D + j], sn = fa.rope_table[(size_t)pos * D + D / 2 + j];
                const float ra = a * c - b * sn, rb = b * c + a * sn;
                a = ra;
                b = rb;
              }
              kdst[j] = from_float<bf16_t>(a);
              kdst[j + D / 2] = from_float<bf16_t>(b);
              vdst[(size_t)j * bs] = vsrc[j];
              vdst[(size_t)(j + D / 2) * bs] = vsrc[j + D / 2];
            }
          }
          __threadfence_block();  // the stores have landed before this wave reads the page below
        }
      }
      // ---- this block's query heads: norm, rotate, round once, as matrix-core operands
      float qv[D / 32][8];
      float ss = 0.f;
#pragma unroll
      for (int c = 0; c < D / 32; ++c) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (r < heads_here) raw = *reinterpret_cast<const uint4*>(q + row + (size_t)(head0 + r) * D + c * 32 + g * 8);
        const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          qv[c][2 * i] = __uint_as_float(w4[i] << 16);
          qv[c][2 * i + 1] = __uint_as_float(w4[i] & 0xffff0000u);
          ss += qv[c][2 * i] * qv[c][2 * i] + qv[c][2 * i + 1] * qv[c][2 * i + 1];
        }
      }
      if (fa.q_w) {
        const float inv = rsqrtf(column_sum(ss) / (float)D + fa.eps);
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
#pragma unroll
          for (int i = 0; i < 8; ++i) qv[c][i] = qv[c][i] * inv * fa.q_w[c * 32 + g * 8 + i];
      }
      if (fa.rope_table) {
#pragma unroll
        for (int c = 0; c < HC; ++c)
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int j = c * 32 + g * 8 + i;
            const float cs = fa.rope_table[(size_t)pos * D + j], sn = fa.rope_table[(size_t)pos * D + D / 2 + j];
            const float a = qv[c][i], b = qv[c + HC][i];
            qv[c][i] = a * cs - b * sn;
            qv[c + HC][i] = b * cs + a * sn;
          }
      }
#pragma unroll
      for (int c = 0; c < D / 32; ++c) {
        qf[0][c].h[0] = pack_bf16x4(qv[c][0], qv[c][1], qv[c][2], qv[c][3]);
        qf[0][c].h[1] = pack_bf16x4(qv[c][4], qv[c][5], qv[c][6], qv[c][7]);
      }
    } else {
#pragma unroll
      for (int c = 0; c < D / 32; ++c) {
        qf[0][c].u = make_uint4(0, 0, 0, 0);
        if (r < heads_here)
          qf[0][c].u = *reinterpret_cast<const uint4*>(q + ((size_t)item * nh + head0 + r) * D + c * 32 + g * 8);
      }
    }
    const int qpos[1] = {ctx - 1};
    if (!early) fetch(t[0], begin);
    // DEPTH tiles in flight per wave: tile i + DEPTH - 1 is requested before the products of tile i. Short
    // splits (few waves, each waiting on memory) want two (four measured no better); with long splits the
    // chip is full of waves and fewer registers, one more wave per SIMD, serve better. A tile past `end` is a valid page that
    // nobody computes on.
    if (DEPTH > 1 && tiles_per_split > LONG_RUN) {
      // a long run of this wave's own (the chip is full of such waves): one tile at a time streams best
      for (int k = begin; k < end; k += 16) {
        if (k > begin) fetch(t[0], k);
        compute_tile<D, 1>(t[0], k, lo, qpos, k < lo || k + 16 > ctx, qf, scale_log2, m, lsum, acc);
      }
    } else {
#pragma unroll
      for (int j = 1; j < DEPTH - 1; ++j) fetch(t[j], begin + 16 * j);
      for (int key0 = begin; key0 < end; key0 += 16 * DEPTH) {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
          const int k = key0 + 16 * j;
          if (DEPTH > 1) fetch(t[(j + DEPTH - 1) % DEPTH], k + 16 * (DEPTH - 1));
          else if (k > begin) fetch(t[0], k);
          if (j == 0 || k < end)
            compute_tile<D, 1>(t[j], k, lo, qpos, k < lo || k + 16 > ctx, qf, scale_log2, m, lsum, acc);
        }
      }
    }
  }
  if (block_waves == 1) {
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
    return;
  }
  // Several waves a block, each with a split of its own: their results meet in LDS and are added up
  // here, with the weights 2^(m_w - M). A block that holds all splits of its heads (gridDim.z == 1)
  // writes the finished output; else one partial result for the block, as a single wave would.
  float* lds_o = decode_lds;                                        // [waves][heads_here][D]
  float* lds_ml = decode_lds + (size_t)block_waves * heads_here * D;  // [waves][heads_here][2]
  if (r < heads_here) {
    float* po = lds_o + ((size_t)wave * heads_here + r) * D;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      *reinterpret_cast<float4_t*>(po + dt * 16 + g * 4) = acc[0][dt];
    if (g == 0) {
      lds_ml[(wave * heads_here + r) * 2] = m[0];
      lds_ml[(wave * heads_here + r) * 2 + 1] = lsum[0];
    }
  }
  __syncthreads();
  const int blocks_z = gridDim.z;
  for (int idx = threadIdx.x; idx < heads_here * (D / 4); idx += blockDim.x) {
    const int hr = idx / (D / 4), quad = idx % (D / 4);
    float big = -INFINITY;
    for (int w = 0; w < block_waves; ++w)
      if (lds_ml[(w * heads_here + hr) * 2 + 1] > 0.f) big = fmaxf(big, lds_ml[(w * heads_here + hr) * 2]);
    float denom = 0.f;
    float4_t total = {0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < block_waves; ++w) {
      const float l = lds_ml[(w * heads_here + hr) * 2 + 1];
      const float wgt = l > 0.f ? fast_exp2(lds_ml[(w * heads_here + hr) * 2] - big) : 0.f;  // an empty split has no weight
      denom += wgt * l;
      const float4_t v = *reinterpret_cast<const float4_t*>(lds_o + ((size_t)w * heads_here + hr) * D + quad * 4);
      total[0] += wgt * v[0];
      total[1] += wgt * v[1];
      total[2] += wgt * v[2];
      total[3] += wgt * v[3];
    }
    const size_t head = (size_t)item * nh + head0 + hr;
    if (blocks_z == 1) {
      const float inv = denom > 0.f ? 1.f / denom : 0.f;  // no visible key at all: zeros, not NaN
      *reinterpret_cast<short4_t*>(out + head * D + quad * 4) =
          pack_bf16x4(total[0] * inv, total[1] * inv, total[2] * inv, total[3] * inv);
    } else {
      const size_t slot = head * blocks_z + blockIdx.z;
      *reinterpret_cast<float4_t*>(part_o + slot * D + quad * 4) = total;
      if (quad == 0) {
        part_ml[slot * 2] = big;
        part_ml[slot * 2 + 1] = denom;
      }
    }
  }
}

// STREAMED: the launch is large enough for non-temporal loads of its keys and values to pay (the host decides by its
// size). They pay where every item reads pages of its own; items that share their pages (a prefix served from the
// cache) read them out of each other's cache lines, which ordinary loads keep: the step says which it is (bit 0 of
// step_flags[0]), and the kernel holds both bodies.
template <int D, bool FUSED, int DEPTH, bool STREAMED>
__global__ __launch_bounds__(DECODE_BLOCK_WAVES(D) * 64) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ item_ctx, const int* __restrict__ block_table, int table_width,
    float* __restrict__ part_o, float* __restrict__ part_ml, bf16_t* __restrict__ out, int nh, int nkv, int bs_shift,
    int window, float scale_log2, int num_splits, int head_chunks, DecodeFusedArgs fa,
    const int* __restrict__ live_items, int waves_wanted, const int* __restrict__ step_flags) {
  if constexpr (STREAMED) {
    if (!(step_flags && (step_flags[0] & 1))) {
      attention_decode_body<D, FUSED, DEPTH, true>(q, k_cache, v_cache, item_ctx, block_table, table_width, part_o, part_ml, out, nh,
                                                   nkv, bs_shift, window, scale_log2, num_splits, head_chunks, fa, live_items,
                                                   waves_wanted);
      return;
    }
  }
  attention_decode_body<D, FUSED, DEPTH, false>(q, k_cache, v_cache, item_ctx, block_table, table_width, part_o, part_ml, out, nh, nkv,
                                                bs_shift, window, scale_log2, num_splits, head_chunks, fa, live_items, waves_wanted);
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
  // the first partial results of this thread are requested before the weights are known: their loads
  // and those of the statistics are in flight together
  constexpr int EARLY = 8;
  const int quads = d / 4;          // d is a multiple of 32, so quads <= 64
  const int groups = 256 / quads;   // groups of splits handled side by side
  const int qd = tid % quads, grp = tid / quads;
  const float* po = part_o + unit * num_splits * d + qd * 4;
  float4_t early[EARLY];
#pragma unroll
  for (int i = 0; i < EARLY; ++i) {
    const int sp = grp + i * groups;
    early[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
    if (grp < groups && sp < num_splits) early[i] = *reinterpret_cast<const float4_t*>(po + (size_t)sp * d);
  }
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

  float4_t accv = {0.f, 0.f, 0.f, 0.f};
  if (grp < groups) {
#pragma unroll
    for (int i = 0; i < EARLY; ++i) {
      const int sp = grp + i * groups;
      const float w = sp < num_splits ? wgt[sp] : 0.f;
      accv[0] += w * early[i][0];
      accv[1] += w * early[i][1];
      accv[2] += w * early[i][2];
      accv[3] += w * early[i][3];
    }
    for (int s = grp + EARLY * groups; s < num_splits; s += groups) {
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
                          float scale_log2, int depth, int num_splits, int block_waves, bf16_t* out,
                          const DecodeFusedArgs* fused, const int* live_items, int waves_wanted, int streamed,
                          const int* step_flags, hipStream_t stream) {
  const int chunks = (nh / nkv + 15) / 16;
  dim3 grid(items, nkv * chunks, num_splits / block_waves);  // num_splits is a multiple of block_waves
  const int heads_most = nh / nkv < 16 ? nh / nkv : 16;
  const size_t lds = block_waves > 1 ? (size_t)block_waves * heads_most * (D + 2) * sizeof(float) : 0;
  int bs_shift = 0;
  while ((1 << bs_shift) < bs) ++bs_shift;
#define ME_DECODE_LAUNCH_AS(FUSED, DEPTH, STREAMED, ARGS)                                                                  \
  attention_decode_kernel<D, FUSED, DEPTH, STREAMED><<<grid, 64 * block_waves, lds, stream>>>(                             \
      q, kc, vc, item_ctx, table, width, part_o, part_ml, out, nh, nkv, bs_shift, window, scale_log2, num_splits, chunks,  \
      ARGS, live_items, waves_wanted, step_flags)
#define ME_DECODE_LAUNCH(FUSED, DEPTH, ARGS)                \
  do {                                                      \
    if (streamed)                                           \
      ME_DECODE_LAUNCH_AS(FUSED, DEPTH, true, ARGS);        \
    else                                                    \
      ME_DECODE_LAUNCH_AS(FUSED, DEPTH, false, ARGS);       \
  } while (0)
  if constexpr (D % 64 == 0) {
    if (fused) {
      if (depth == 2)
        ME_DECODE_LAUNCH(true, 2, *fused);
      else
        ME_DECODE_LAUNCH(true, 1, *fused);
      return;
    }
  }
  if (depth == 2)
    ME_DECODE_LAUNCH(false, 2, DecodeFusedArgs{});
  else
    ME_DECODE_LAUNCH(false, 1, DecodeFusedArgs{});
#undef ME_DECODE_LAUNCH_AS
#undef ME_DECODE_LAUNCH
}

// Head sizes that are multiples of 32 (instantiated: 32, 64, 96, 128, 192, 256) and pages of a power
// of two of at least 16 keys.
extern "C" int me_attention_mfma_supported(int d, int bs) {
  return (d == 32 || d == 64 || d == 96 || d == 128 || d == 192 || d == 256) && bs >= 16 && (bs & (bs - 1)) == 0;
}

// q [items, nh, d] (one token per item), item_ctx[i] = keys of item i including the new one,
// workspace: part_o float [items * nh * num_splits * d], part_ml float [items * nh * num_splits * 2].
// Every item's keys are dealt to the num_splits splits in equal runs; split_keys (a multiple of 16) says
// how long a run is at the longest context the step can hold (max_ctx): num_splits * split_keys must
// cover it. live_items (device, or null): how many of the items are live, for a launch whose grid was
// laid out for fewer items than it holds; then full_splits is the number of splits of a step with every
// item live and waves_wanted the number of waves that the live items' splits should come to.
// How many splits one block of a decode launch takes on, a wave each (1: a wave a block, and a second kernel or the
// product behind adds up the splits).
// Few splits (a step of many items): one block takes all splits of its heads, a wave each, adds their
// results up itself and writes the output; the second kernel is not needed then. Such a block is a whole
// (item, kv head) of work and a compute unit takes in only so much per microsecond, so this pays only where the
// blocks divide evenly among the compute units: 512 blocks on 256 units yes (batch 64: 5% ahead of one wave a
// block and the second kernel), and up to 256 (a block a unit: 17 to 32 items, 3-7% ahead), but 320 or 384 no
// (batch 40: 8,280 -> 8,850 tokens/s with a wave a block: a unit had one block or two, and the step waited for
// the units with two).
static int decode_compute_units() {
  static int cus = 0;
  if (cus <= 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0)
      cus = 256;
  }
  return cus;
}

static int decode_block_waves(int items, int nh, int nkv, int d, int num_splits) {
  int block_waves = (num_splits > 1 && num_splits <= DECODE_BLOCK_WAVES(d)) ? num_splits : 1;
  const int heads_most = nh / nkv < 16 ? nh / nkv : 16;
  if ((size_t)block_waves * heads_most * (d + 2) * sizeof(float) > 48 * 1024) block_waves = 1;  // LDS for the sum
  const int cus = decode_compute_units();
  const long long blocks = (long long)items * nkv * ((nh / nkv + 15) / 16);  // with every split of an (item, kv head) in one block
  if (block_waves > 1) {
    const long long rounds = (blocks + cus - 1) / cus;
    if (blocks > cus && blocks * 10 < rounds * cus * 9) block_waves = 1;  // rounds that are less than nine tenths full
  }
  return block_waves;
}

// Whether a decode launch of these sizes leaves one partial result per split in part_o / part_ml (which the second
// kernel, or me_attention_out_product_bf16 in its place, adds up): the launches that may be given no `out`.
extern "C" int me_attention_decode_leaves_parts(int items, int nh, int nkv, int d, int num_splits) {
  if (items <= 0 || nh <= 0 || nkv <= 0 || nh % nkv) return 0;
  return decode_block_waves(items, nh, nkv, d, num_splits) == 1;
}

static int decode_common(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                         const int* block_table, int table_width, void* out, float* part_o, float* part_ml, int items,
                         int nh, int nkv, int d, int bs, int window, float scale, int split_keys, int num_splits,
                         int max_ctx, const DecodeFusedArgs* fused, const int* live_items, int full_splits,
                         int waves_wanted, const int* step_flags, hipStream_t stream);

extern "C" int me_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                                        const int* block_table, int table_width, void* out, float* part_o,
                                        float* part_ml, int items, int nh, int nkv, int d, int bs, int window,
                                        float scale, int split_keys, int num_splits, int max_ctx,
                                        const int* live_items, int full_splits, int waves_wanted,
                                        const int* step_flags, hipStream_t stream) {
  return decode_common(q, k_cache, v_cache, item_ctx, block_table, table_width, out, part_o, part_ml, items, nh, nkv, d,
                       bs, window, scale, split_keys, num_splits, max_ctx, nullptr, live_items, full_splits, waves_wanted,
                       step_flags, stream);
}

// Head sizes and groupings for which the decode kernel can take the norm, the rotary encoding and
// the page write as its prologue: a multiple of 64, full-width rotary or none, at most 16 heads per
// kv head.
extern "C" int me_attention_decode_fused_supported(int d, int bs, int rotary_dim, int group) {
  return me_attention_mfma_supported(d, bs) && d % 64 == 0 && (rotary_dim == 0 || rotary_dim == d) && group <= 16;
}

// As me_attention_decode_bf16, from the raw projection qkv [items, (nh + 2 nkv) d] (or [items, nh d]
// with write_kv == 0). rope_table must cover position max_ctx - 1.
extern "C" int me_attention_decode_fused_bf16(const void* qkv, const float* q_w, const float* k_w,
                                              const float* rope_table, int rotary_dim, float eps, int write_kv,
                                              void* k_cache, void* v_cache, const int* item_ctx,
                                              const int* block_table, int table_width, void* out, float* part_o,
                                              float* part_ml, int items, int nh, int nkv, int d, int bs, int window,
                                              float scale, int split_keys, int num_splits, int max_ctx,
                                              const int* live_items, int full_splits, int waves_wanted,
                                              const int* step_flags, hipStream_t stream) {
  if (nkv <= 0 || nh <= 0 || nh % nkv || !me_attention_decode_fused_supported(d, bs, rope_table ? rotary_dim : 0, nh / nkv))
    return me_fail("me_attention_decode_fused_bf16: head_dim=%d block_size=%d rotary_dim=%d heads=%d/%d not supported", d,
                   bs, rotary_dim, nh, nkv);
  DecodeFusedArgs fa;
  fa.q_w = q_w;
  fa.k_w = k_w;
  fa.rope_table = rope_table;
  fa.eps = eps;
  fa.write_kv = write_kv;
  fa.k_cache_w = (bf16_t*)k_cache;
  fa.v_cache_w = (bf16_t*)v_cache;
  return decode_common(qkv, k_cache, v_cache, item_ctx, block_table, table_width, out, part_o, part_ml, items, nh, nkv, d,
                       bs, window, scale, split_keys, num_splits, max_ctx, &fa, live_items, full_splits, waves_wanted, step_flags,
                       stream);
}

static int decode_common(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                         const int* block_table, int table_width, void* out, float* part_o, float* part_ml, int items,
                         int nh, int nkv, int d, int bs, int window, float scale, int split_keys, int num_splits,
                         int max_ctx, const DecodeFusedArgs* fused, const int* live_items, int full_splits,
                         int waves_wanted, const int* step_flags, hipStream_t stream) {
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
  // How many tiles a wave keeps in flight goes by the splits that a step with every item live uses
  // (full_splits; the grid's num_splits when no count of live items is given).
  if (live_items && (full_splits <= 0 || full_splits > num_splits || waves_wanted <= 0))
    return me_fail("me_attention_decode_bf16: %d splits for a full step out of %d, %d waves wanted", full_splits, num_splits,
                   waves_wanted);
  const int run_splits = live_items ? full_splits : num_splits;
  const int run_keys = (((max_ctx + run_splits - 1) / run_splits + 15) / 16) * 16;
  const long long run_waves = (long long)items * nkv * ((nh / nkv + 15) / 16) * run_splits;
  const int depth = (run_keys <= 256 || run_waves <= 1024) ? 2 : 1;
  const int block_waves = decode_block_waves(items, nh, nkv, d, num_splits);
  if (!out && block_waves > 1)
    return me_fail("me_attention_decode_bf16: a launch whose blocks add up their splits themselves needs `out`");
  const int cus = decode_compute_units();
  const long long blocks = (long long)items * nkv * ((nh / nkv + 15) / 16);
  // Keys and values pass through once: loaded as non-temporal they arrive faster where the launch streams hundreds of
  // megabytes over a full chip (batch 64 at 4,096: 6.21 -> 5.97 ms a step; batch 8 and 16 at 16,384: 3.54 -> 3.41 and
  // 6.0 -> 5.6), and no faster or slower where it does not (batch 8 at 4,096, 134 MB: level; 33 MB and less: 0.4-0.8% slower;
  // 160 to 224 blocks of 5 to 7 waves on 256 compute units, batch 20 to 28: 1-5% slower). The size goes by the longest context
  // the launch may hold. (Instances of the kernel of their own: as a branch around every load of one kernel it cost steps that
  // do not take it up to 4%.)
  const long long kv_bytes = (long long)items * max_ctx * nkv * d * 4;
  const int streamed = kv_bytes >= (256ll << 20) && (block_waves == 1 || blocks >= cus);
  const float sl = scale * LOG2E;
  const bf16_t *qq = (const bf16_t*)q, *kc = (const bf16_t*)k_cache, *vc = (const bf16_t*)v_cache;
#define ME_DECODE_CASE(DD)                                                                                      \
  case DD:                                                                                                      \
    launch_decode<DD>(qq, kc, vc, item_ctx, block_table, table_width, part_o, part_ml, items, nh, nkv, bs, window, sl, \
                      depth, num_splits, block_waves, (bf16_t*)out, fused, live_items, waves_wanted, streamed, step_flags, \
                      stream);                                                                                  \
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
  if (block_waves > 1) return 0;  // the blocks held all splits of their heads and wrote the output themselves
  if (!out) return 0;             // the caller adds up the splits (me_attention_out_product_bf16)
  attention_decode_combine_kernel<<<items * nh, 256, 0, stream>>>(part_o, part_ml, (bf16_t*)out, num_splits, d);
  return me_check_launch("me_attention_decode_combine");
}

// ------------------------------------------------------------------------------------ prefill
// A block owns the query columns of `tokens_per_block = columns / group` consecutive
// new tokens of one item for one kv head (column c -> token c / group, head c % group); wave w owns
// NB blocks of 16 columns. Measured on 2,048-token prompts of the 0.6B shape: 8 waves x 1 block of
// columns (128 columns a block) beats 4 x 2 (register pressure pushes the accumulators out of the
// vector registers) and 4 x 1 (64 columns a block, twice the LDS traffic per product, also when a long and
// a short tile share a compute unit). What a block does is an entry of a work list that the host lays
// out once per step, longest first: which tokens, which range of keys. Causal prompts give tiles of
// very different lengths; a block costs about 3 us plus 1.5 us per 64 keys, so at 2,048 tokens (one block
// per compute unit) the last tile's 32 key tiles set the time. Cutting long tiles into ranges, whose
// partial results a second kernel adds up, evens that out but pays the fixed cost and the partial
// results again: measured worth it only where the step has fewer blocks than the chip has compute
// units (a short portion of a prompt over a long context), which is where the host does it.
//
// Keys and values are staged through LDS in tiles of 64 keys, double-buffered: while the waves
// multiply tile i out of one buffer, the loads of tile i+1 fill the other, straight from the pages
// (global_load_lds_dwordx4: no registers hold a tile and no LDS write instructions are issued; with the
// tile in registers on its way a 2,048-token prompt took 38.6 us a layer, now 37.2, and 32,704 tokens
// 161 ms in all, now 153); one barrier per tile. Products use v_mfma_f32_16x16x32_bf16 (the
// full-rate bfloat16 instruction of gfx950; the 16x16x16 form runs at half its rate):
//   S^T (16 keys x 16 columns) += K[16 keys, 32 d] . Q^T[32 d, 16 columns]
//   O^T (16 d x 16 columns)   += V^T[16 d, 32 keys] . P^T[32 keys, 16 columns]
// A lane holds four rows of every score tile. The rows of the four score tiles of a 64-key tile are dealt
// to the keys so that these come to eight consecutive keys per 32 (PrefillLds below): the lane's B operand
// of the second product then pairs with one 16-byte piece of a value row as it lies in its page.
//
// A 16-byte LDS read is served in four groups of lanes (0-3 with 12-15 and 20-27, 4-11 with 16-19 and
// 28-31, and the same in the upper half); the layouts below keep each group on distinct banks
// (measured: 5.3 cycles per wave instruction against 8 with two lanes a bank).
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

#define PF_KT 64  // keys per LDS tile

// One LDS buffer holds a 64-key tile as the global loads deliver it (a wave's load instruction writes 64
// consecutive 16-byte pieces, one per lane, wherever in memory each lane reads): no rows can be padded, so
// the key rows are swizzled instead.
//   keys:   [64 keys][D/8 pieces]; the piece at physical column pc of key row k holds the eight dims from
//           (pc ^ swizzle(k)) * 8. Row t*16.. of the first product's A operand is not key t*16 + r but
//           key 32 (t/2) + 8 (r/4) + 4 (t%2) + r%4, so that a lane ends up with the scores of eight
//           consecutive keys per 32 (four of score tile 2h, four of tile 2h+1): the B operand of the second
//           product then pairs with eight consecutive keys of a value row, one 16-byte piece as it lies in
//           the page. swizzle(k) = (k % 4) + 4 ((k / 8) % 4) is the row r that reads key k: with a row
//           stride of 256 bytes (d = 128) the 16-byte reads of a wave's four groups of lanes hit every bank once.
//   values: [4 sub-tiles of 16 keys][D dims][2 pieces]: the layout of a transposed page of 16 slots; rows 32
//           bytes apart, read by lane % 16 with the piece chosen by the lane's upper bits, are free of conflicts as they are.
template <int D>
struct PrefillLds {
  static constexpr int P = D / 8;                // 16-byte pieces per key row
  static constexpr int REGION = PF_KT * D;       // elements of the keys of a tile, and of its values
  static constexpr int BUF_ELEMS = 2 * REGION;
  static constexpr int BUFFERS = 2;
  static constexpr int BYTES = BUFFERS * BUF_ELEMS * 2;
  static constexpr int LOW = (P & -P) < 16 ? (P & -P) : 16;  // the swizzle stays inside an aligned group of pieces that every row has
  static constexpr int SWIZZLE_MASK = LOW - 1;
  __device__ static constexpr int swizzle(int key) { return ((key & 3) | (((key >> 3) & 3) << 2)) & SWIZZLE_MASK; }
};

typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// What a lane fetches of every tile: a wave's load instruction j of a region (j = wave, wave + WAVES, ...: D/8
// instructions for the keys, as many for the values) brings pieces 64 j .. 64 j + 63 of the region. The pieces of
// one instruction lie in one 16-key sub-tile, hence in one page: the page's address is scalar arithmetic and a
// lane only adds its own offset, which is the same for every tile.
template <int D, int WAVES>
struct PfStage {
  static constexpr int P = D / 8;
  static constexpr int SLOTS = (P + WAVES - 1) / WAVES;
  unsigned k_off[SLOTS], v_off[SLOTS];  // bytes from the sub-tile's first key (first slot) in its page
  int page[SLOTS];                      // block-table entries of the tile to be fetched next: scalar
};

template <int D, int WAVES>
__device__ __forceinline__ void pf_stage_init(PfStage<D, WAVES>& st, int wave, int lane, int bs_shift) {
  using L = PrefillLds<D>;
#pragma unroll
  for (int sl = 0; sl < PfStage<D, WAVES>::SLOTS; ++sl) {
    const int n = 64 * (wave + sl * WAVES) + lane;  // piece of the region
    const int key = (n / L::P) & (PF_KT - 1), pc = n % L::P;
    st.k_off[sl] = (unsigned)(((key & 15) * D + ((pc ^ L::swizzle(key)) * 8)) * 2);
    const int d = (n % (2 * D)) >> 1, piece = n & 1;
    st.v_off[sl] = (((unsigned)d << bs_shift) * 2u) + (unsigned)piece * 16u;
  }
}

// Block-table entries of the pages that the wave's instructions of tile `key0` read. Scalar loads, issued an
// iteration before pf_issue_tile uses them.
template <int D, int WAVES>
__device__ __forceinline__ void pf_fetch_pages(PfStage<D, WAVES>& st, int key0, int wave, const int* __restrict__ table,
                                               int table_width, int bs_shift) {
  constexpr int P = D / 8;
#pragma unroll
  for (int sl = 0; sl < PfStage<D, WAVES>::SLOTS; ++sl) {
    const int sub = min((wave + sl * WAVES) / (P / 4), 3);
    st.page[sl] = table[min((key0 + 16 * sub) >> bs_shift, table_width - 1)];
  }
}

// Requests tile `key0` from the pages straight into the LDS buffer `buf`; the data is there after the next
// __syncthreads() (which waits for the wave's outstanding loads before the barrier).
template <int D, int WAVES>
__device__ __forceinline__ void pf_issue_tile(const PfStage<D, WAVES>& st, int key0, int wave, bf16_t* buf, int bs_shift, int nkv,
                                              int kvh, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache) {
  using L = PrefillLds<D>;
  constexpr int P = D / 8;
  const int bs_mask = (1 << bs_shift) - 1;
  char* kdst = reinterpret_cast<char*>(buf);
  char* vdst = reinterpret_cast<char*>(buf + L::REGION);
#pragma unroll
  for (int sl = 0; sl < PfStage<D, WAVES>::SLOTS; ++sl) {
    const int j = wave + sl * WAVES;
    if (P % WAVES != 0 && j >= P) break;  // the same for the whole wave
    const int sub = j / (P / 4);
    int page = st.page[sl];
    page = page < 0 ? 0 : page;
    const int off = (key0 + 16 * sub) & bs_mask;  // of the sub-tile's first key in its page
    const char* kb = reinterpret_cast<const char*>(k_cache + ((((size_t)page * nkv + kvh) << bs_shift) + off) * D);
    const char* vb = reinterpret_cast<const char*>(v_cache + ((((size_t)page * nkv + kvh) * D) << bs_shift) + off);
    __builtin_amdgcn_global_load_lds((global_ptr_t)(kb + st.k_off[sl]), (lds_ptr_t)(kdst + j * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((global_ptr_t)(vb + st.v_off[sl]), (lds_ptr_t)(vdst + j * 1024), 16, 0, 0);
  }
}


// Maximum without the quieting of signalling NaNs that fmaxf brings along (an extra instruction per
// operand): scores are finite or -inf here.
__device__ __forceinline__ float max_raw(float a, float b) {
  float d;
  asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}
__device__ __forceinline__ float column_max_raw(float v) {
  unsigned u = __float_as_uint(v);
  uint2v_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  u = __float_as_uint(max_raw(__uint_as_float(a[0]), __uint_as_float(a[1])));
  a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return max_raw(__uint_as_float(a[0]), __uint_as_float(a[1]));
}

// First product of one 64-key tile: four 16-key score tiles against NB blocks of 16 query columns,
// out of the key half of one LDS buffer.
template <int D, int NB>
__device__ __forceinline__ void pf_scores64(const bf16_t* __restrict__ ks, int r, int g, const bf16x8_t (&qf)[NB][D / 32],
                                            float4_t (&s)[NB][4]) {
  using L = PrefillLds<D>;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int t = 0; t < 4; ++t) s[nb][t] = (float4_t){0.f, 0.f, 0.f, 0.f};
  const int key_r = 8 * (r >> 2) + (r & 3);  // the lane's key row of score tile 0; swizzle(key of any tile) = swizzle(key_r)
#pragma unroll
  for (int c = 0; c < D / 32; ++c) {
    const bf16_t* col = ks + key_r * D + ((c * 4 + g) ^ L::swizzle(key_r)) * 8;
    bf16x8_t kf[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) kf[t] = *reinterpret_cast<const bf16x8_t*>(col + (32 * (t >> 1) + 4 * (t & 1)) * D);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int t = 0; t < 4; ++t) s[nb][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t], qf[nb][c], s[nb][t], 0, 0, 0);
  }
}

// One pass of the running softmax over the 64 scores of each column, then the second product out of the
// value half of the LDS buffer. MASK is a compile-time switch: tiles that every column of the wave
// sees whole skip the compares.
template <int D, int NB, bool MASK>
__device__ __forceinline__ void pf_softmax_pv64(const bf16_t* __restrict__ vs, int key_base, int r, int g,
                                                const float4_t (&s)[NB][4], const int (&qpos)[NB], const int (&lo_col)[NB],
                                                float scale_log2, float (&m)[NB], float (&lsum)[NB],
                                                float4_t (&acc)[NB][D / 16]) {
  using L = PrefillLds<D>;
  bf16x8_t pf[NB][2];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float sv[16];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) sv[t * 4 + i] = s[nb][t][i];
    if (MASK) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = key_base + (i >> 3) * 32 + g * 8 + ((i >> 2) & 1) * 4 + (i & 3);  // score tile i / 4, row 4g + i % 4
        if (key < lo_col[nb] || key > qpos[nb]) sv[i] = -INFINITY;
      }
    }
    // statistics are kept in units of the raw score times scale*log2(e): one fused multiply-add per
    // score feeds the exponential
    float tmax = max3_raw(max3_raw(sv[0], sv[1], sv[2]), max3_raw(sv[3], sv[4], sv[5]), max3_raw(sv[6], sv[7], sv[8]));
    tmax = max3_raw(tmax, max3_raw(sv[9], sv[10], sv[11]), max3_raw(sv[12], sv[13], sv[14]));
    tmax = column_max_raw(max_raw(tmax, sv[15])) * scale_log2;
    const float m_new = max_raw(m[nb], tmax);
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;  // a column with no visible key so far
    const float alpha = fast_exp2(m[nb] - m_ref);
    float p[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) p[i] = fast_exp2(fmaf(sv[i], scale_log2, -m_ref));
    const float psum = (((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]))) +
                       (((p[8] + p[9]) + (p[10] + p[11])) + ((p[12] + p[13]) + (p[14] + p[15])));
    // the lane's own keys: the four lanes of a column scale their sums alike (the maximum is the column's) and add them
    // up once, behind the loop over keys (8,192 and 32,704 tokens 1.9% faster than with the column's sum per tile)
    lsum[nb] = fmaf(lsum[nb], alpha, psum);
    m[nb] = m_new;
    // The running maximum rarely moves after the first tiles: the rescale of the accumulator is skipped
    // when no column of the wave needs it. The multiplication is written as instructions that work in
    // place: as plain C++ under a branch the accumulator ends up in two sets of registers and is copied
    // on the path that does not multiply, which costs more than multiplying always.
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) {
        float a0 = acc[nb][dt][0], a1 = acc[nb][dt][1], a2 = acc[nb][dt][2], a3 = acc[nb][dt][3];
        asm volatile("v_mul_f32 %0, %0, %4\n v_mul_f32 %1, %1, %4\n v_mul_f32 %2, %2, %4\n v_mul_f32 %3, %3, %4"
                     : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3) : "v"(alpha));
        acc[nb][dt] = (float4_t){a0, a1, a2, a3};
      }
    }
    // the B operand of the second product: for each half of 32 keys, the lane's four keys of the first
    // score tile and then those of the second
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 8; ++i) pf[nb][h][i] = (__bf16)p[h * 8 + i];  // round to nearest even in hardware
  }
  // halves outermost: the two products into one accumulator are D/16 instructions apart
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(vs + ((2 * h + (g >> 1)) * D + dt * 16 + r) * 16 + (g & 1) * 8);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[nb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[nb][h], acc[nb][dt], 0, 0, 0);
    }
  }
}

// One entry of the work list that the host lays out for a step: a tile of consecutive query tokens of one
// item and a range of keys. The positions of an item's tokens are consecutive, so the first one's stands
// for all. A tile whose keys are cut into several ranges gives partial results that
// attention_prefill_combine_kernel adds up; `chunk` is -1 for a tile in one piece. A block runs the
// entries from its first one (bundle_first[block]) up to and including the next one marked `last`: the
// host packs entries into bundles of about equal work when a step has too few tiles to go round.
struct PrefillWork {
  int item;
  int token_begin, token_count;  // the tile's tokens among the packed tokens of the step
  int pos_first;                 // position of the first of them
  int key_begin;                 // first key, a multiple of 64
  int key_last;                  // last key, inclusive
  int chunk;
  int last;
};

// WAVES waves per block, NB blocks of 16 query columns per wave: WAVES * NB * 16 = 128 columns.
template <int D, int NB, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const PrefillWork* __restrict__ work, const int* __restrict__ bundle_first, const int* __restrict__ block_table,
    int table_width, bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int max_chunks,
    int nh, int nkv, int bs_shift, int window, float scale_log2, int tokens_per_block) {
  constexpr int THREADS = WAVES * 64;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16_t* lds = reinterpret_cast<bf16_t*>(lds_raw);
  using L = PrefillLds<D>;
  const int kvh = blockIdx.x % nkv;
  const int group = nh / nkv;
  const int tid = threadIdx.x, lane = tid & (ME_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / ME_WAVE);  // scalar: what a wave fetches follows from it
  const int r = lane & 15, g = lane >> 4;
  PfStage<D, WAVES> stage;
  pf_stage_init<D, WAVES>(stage, wave, lane, bs_shift);
  for (int wi = bundle_first[blockIdx.x / nkv];; ++wi) {
  const PrefillWork w = work[wi];  // the same for every lane: scalar loads
  const int item = w.item;
  const int t_begin = w.token_begin, t_end = w.token_begin + w.token_count;
  const int* table = block_table + (size_t)item * table_width;

  // this lane's query column in each of the wave's blocks
  int tok[NB], head[NB], qpos[NB], lo_col[NB];
  bool col_ok[NB];
  int wave_max_pos = -1, wave_min_pos = 0x7fffffff;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int c = (wave * NB + nb) * 16 + r;
    tok[nb] = t_begin + c / group;
    head[nb] = kvh * group + c % group;
    col_ok[nb] = c < tokens_per_block * group && tok[nb] < t_end;
    qpos[nb] = col_ok[nb] ? w.pos_first + c / group : -1;
    lo_col[nb] = window > 0 ? max(qpos[nb] - window + 1, 0) : 0;
    wave_max_pos = max(wave_max_pos, qpos[nb]);
    if (col_ok[nb]) wave_min_pos = min(wave_min_pos, qpos[nb]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    wave_max_pos = max(wave_max_pos, __shfl_xor(wave_max_pos, off, ME_WAVE));
    wave_min_pos = min(wave_min_pos, __shfl_xor(wave_min_pos, off, ME_WAVE));
  }

  bf16x8_t qf[NB][D / 32];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      qf[nb][c] = bf16x8_t{};
      if (col_ok[nb])
        qf[nb][c] = *reinterpret_cast<const bf16x8_t*>(q + ((size_t)tok[nb] * nh + head[nb]) * D + c * 32 + g * 8);
    }
  float m[NB], lsum[NB];
  float4_t acc[NB][D / 16];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    m[nb] = -INFINITY;
    lsum[nb] = 0.f;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) acc[nb][dt] = (float4_t){0.f, 0.f, 0.f, 0.f};
  }

  // ---- staging of 64-key tiles: global memory -> LDS without a stop in registers (pf_issue_tile). While tile i
  // is multiplied out of LDS buffer i % 2, the loads of tile i+1 fill the other buffer: it was last read
  // before the barrier that ended iteration i-1, and the barrier that ends iteration i waits for the loads.
  const int first_tile = w.key_begin;
  const int last_key = w.key_last;
  pf_fetch_pages<D, WAVES>(stage, first_tile, wave, table, table_width, bs_shift);
  pf_issue_tile<D, WAVES>(stage, first_tile, wave, lds, bs_shift, nkv, kvh, k_cache, v_cache);
  pf_fetch_pages<D, WAVES>(stage, first_tile + PF_KT, wave, table, table_width, bs_shift);
  __syncthreads();
  int buf = 0;
  for (int key0 = first_tile; key0 <= last_key; key0 += PF_KT, buf ^= 1) {
    const bf16_t* ks = lds + (size_t)buf * L::BUF_ELEMS;
    const bf16_t* vs = ks + L::REGION;
    const bool active = key0 <= wave_max_pos;  // else every column of the wave lies before this tile
    // Tiles are fetched unconditionally (the page index is clamped to the table, so a tile past the last
    // key reads valid memory that nobody uses).
    pf_issue_tile<D, WAVES>(stage, key0 + PF_KT, wave, lds + (size_t)(buf ^ 1) * L::BUF_ELEMS, bs_shift, nkv, kvh, k_cache, v_cache);
    pf_fetch_pages<D, WAVES>(stage, key0 + 2 * PF_KT, wave, table, table_width, bs_shift);  // for the next iteration
    float4_t s[NB][4];
    pf_scores64<D, NB>(ks, r, g, qf, s);  // also by a wave that will not use them: no control flow around s
    if (active) {
      const bool need_mask = key0 + PF_KT - 1 > wave_min_pos || window > 0;
      if (need_mask)
        pf_softmax_pv64<D, NB, true>(vs, key0, r, g, s, qpos, lo_col, scale_log2, m, lsum, acc);
      else
        pf_softmax_pv64<D, NB, false>(vs, key0, r, g, s, qpos, lo_col, scale_log2, m, lsum, acc);
    }
    __syncthreads();
  }
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) lsum[nb] = column_sum(lsum[nb]);
  if (w.chunk >= 0) {
    // one range of several: the unnormalised sums and the statistics of every column
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if (!col_ok[nb]) continue;
      const size_t slot = ((size_t)tok[nb] * nh + head[nb]) * max_chunks + w.chunk;
      if (g == 0) {
        part_ml[slot * 2] = m[nb];
        part_ml[slot * 2 + 1] = lsum[nb];
      }
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) *reinterpret_cast<float4_t*>(part_o + slot * D + dt * 16 + g * 4) = acc[nb][dt];
    }
  } else {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
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
  if (w.last) break;  // (the loop over keys ended with a barrier: LDS is free for the next entry)
  }
}

// Adds up the ranges of the tokens whose keys were cut: out[token, head, :] = sum_c 2^(m_c - M) o_c /
// sum_c 2^(m_c - M) l_c over the token's chunks (token_chunks[token]; tokens with one chunk were written
// by the attention kernel itself). One block per token; a thread owns four consecutive outputs of a head
// at a time, so that all loads of a block are independent of each other.
__global__ __launch_bounds__(256) void attention_prefill_combine_kernel(const float* __restrict__ part_o,
                                                                        const float* __restrict__ part_ml,
                                                                        const int* __restrict__ token_chunks,
                                                                        bf16_t* __restrict__ out, int nh, int d,
                                                                        int max_chunks) {
  const int tok = blockIdx.x;
  const int nc = token_chunks[tok];
  if (nc <= 1) return;
  const int quads = nh * d / 4;  // d is a multiple of 32
  for (int v = threadIdx.x; v < quads; v += 256) {
    const int head = v * 4 / d, e = v * 4 % d;
    const size_t unit = (size_t)tok * nh + head;
    const float* ml = part_ml + unit * max_chunks * 2;
    const float* po = part_o + unit * max_chunks * d + e;
    float big = -INFINITY;
    for (int c = 0; c < nc; ++c)
      if (ml[c * 2 + 1] > 0.f) big = fmaxf(big, ml[c * 2]);
    float denom = 0.f;
    float4_t total = {0.f, 0.f, 0.f, 0.f};
    for (int c = 0; c < nc; ++c) {
      const float l = ml[c * 2 + 1];
      if (l > 0.f) {  // a range with no visible key has no weight
        const float wgt = fast_exp2(ml[c * 2] - big);
        const float4_t o = *reinterpret_cast<const float4_t*>(po + (size_t)c * d);
        denom += wgt * l;
        total[0] = fmaf(wgt, o[0], total[0]);
        total[1] = fmaf(wgt, o[1], total[1]);
        total[2] = fmaf(wgt, o[2], total[2]);
        total[3] = fmaf(wgt, o[3], total[3]);
      }
    }
    const float inv = 1.f / denom;
    *reinterpret_cast<short4_t*>(out + unit * d + e) =
        pack_bf16x4(total[0] * inv, total[1] * inv, total[2] * inv, total[3] * inv);
  }
}

#define PF_WAVES 8
// Query columns (token, head of the group) per block: 16 or 32 per wave. The wider block reads each key
// and value fragment once for two products and stages half as many tiles per product, which pays when a
// step still gives every compute unit several blocks (long prompts).
#define PF_COLUMNS_NARROW (PF_WAVES * 16)
#define PF_COLUMNS_WIDE (2 * PF_WAVES * 16)

extern "C" int me_attention_prefill_columns(int wide) { return wide ? PF_COLUMNS_WIDE : PF_COLUMNS_NARROW; }

template <int D, int NB>
static int launch_prefill(dim3 grid, const bf16_t* q, const bf16_t* kc, const bf16_t* vc, const PrefillWork* work,
                          const int* bundle_first, const int* table, int width, bf16_t* out,
                          float* part_o, float* part_ml, int max_chunks, int nh, int nkv, int bs_shift, int window,
                          float sl, int tpb, hipStream_t stream) {
  static bool configured = false;  // raise the dynamic LDS limit of this instantiation once
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<D, NB, PF_WAVES>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, PrefillLds<D>::BYTES);
    if (e != hipSuccess) return me_fail("me_attention_prefill_bf16: cannot reserve %d bytes of LDS: %s",
                                        PrefillLds<D>::BYTES, hipGetErrorString(e));
    configured = true;
  }
  attention_prefill_kernel<D, NB, PF_WAVES><<<grid, PF_WAVES * 64, PrefillLds<D>::BYTES, stream>>>(
      q, kc, vc, work, bundle_first, table, width, out, part_o, part_ml, max_chunks, nh, nkv, bs_shift, window, sl, tpb);
  return 0;
}

// q [T, nh, d], packed new tokens. columns: query columns per block, me_attention_prefill_columns(0) or (1).
// work: entries of eight ints laid out by the caller (item, first token and
// number of tokens of the tile (at most columns / group), position of the first
// token, first key (a multiple of 64), last key, chunk or -1, 1 on the last entry of a bundle);
// bundle_first int [num_bundles]: the first entry of each bundle. Every bundle is run by one block per kv
// head. When a tile's keys are cut into chunks (max_chunks > 1), part_o float [T, nh, max_chunks, d] and
// part_ml float [T, nh, max_chunks, 2] take the partial results and token_chunks int [T] says how many
// chunks each token's tile has (1: in one piece).
extern "C" int me_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, int num_items,
                                         const int* block_table, int table_width, void* out, const int* work,
                                         const int* bundle_first, int num_bundles, float* part_o, float* part_ml,
                                         const int* token_chunks, int max_chunks, int num_tokens, int nh, int nkv,
                                         int d, int bs, int window, float scale, int columns, hipStream_t stream) {
  const int num_work = num_bundles;
  if (num_items <= 0 || num_work <= 0) return 0;
  if (!me_attention_mfma_supported(d, bs))
    return me_fail("me_attention_prefill_bf16: head_dim=%d / block_size=%d not supported by the matrix-core kernels", d, bs);
  if (nh <= 0 || nkv <= 0 || nh % nkv) return me_fail("me_attention_prefill_bf16: nh=%d nkv=%d", nh, nkv);
  // the kernel takes the tile maximum on unscaled scores and scales afterwards: right for a positive scale only
  if (!(scale > 0.f) || scale > 3.0e38f) return me_fail("me_attention_prefill_bf16: scale=%g must be positive and finite", scale);
  const int group = nh / nkv;
  if (group > 16) return me_fail("me_attention_prefill_bf16: group size %d exceeds 16", group);
  if ((long long)num_work * nkv > 0x7fffffffLL) return me_fail("me_attention_prefill_bf16: %d x %d blocks exceed the grid", num_work, nkv);
  if (table_width <= 0) return me_fail("me_attention_prefill_bf16: empty block table");
  if (!work || !bundle_first) return me_fail("me_attention_prefill_bf16: no work list");
  if (max_chunks < 1 || (max_chunks > 1 && (!part_o || !part_ml || !token_chunks || num_tokens <= 0)))
    return me_fail("me_attention_prefill_bf16: %d chunks need the partial buffers and the chunk counts", max_chunks);
  if (columns != PF_COLUMNS_NARROW && columns != PF_COLUMNS_WIDE)
    return me_fail("me_attention_prefill_bf16: %d query columns per block (%d or %d)", columns, PF_COLUMNS_NARROW, PF_COLUMNS_WIDE);
  const bool wide = columns == PF_COLUMNS_WIDE;
  const int tpb = columns / group;
  const float sl = scale * LOG2E;
  int bs_shift = 0;
  while ((1 << bs_shift) < bs) ++bs_shift;
  dim3 grid((unsigned)num_work * nkv);
  const bf16_t *qq = (const bf16_t*)q, *kc = (const bf16_t*)k_cache, *vc = (const bf16_t*)v_cache;
  int rc = 0;
#define ME_PREFILL_CASE(DD)                                                                                        \
  case DD:                                                                                                         \
    rc = wide ? launch_prefill<DD, 2>(grid, qq, kc, vc, (const PrefillWork*)work, bundle_first, block_table,       \
                                      table_width, (bf16_t*)out, part_o, part_ml, max_chunks, nh, nkv, bs_shift,   \
                                      window, sl, tpb, stream)                                                     \
              : launch_prefill<DD, 1>(grid, qq, kc, vc, (const PrefillWork*)work, bundle_first, block_table,       \
                                      table_width, (bf16_t*)out, part_o, part_ml, max_chunks, nh, nkv, bs_shift,   \
                                      window, sl, tpb, stream);                                                    \
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
  if (rc) return rc;
  if (me_check_launch("me_attention_prefill_bf16")) return 1;
  if (max_chunks > 1) {
    attention_prefill_combine_kernel<<<num_tokens, 256, 0, stream>>>(part_o, part_ml, token_chunks, (bf16_t*)out, nh, d,
                                                                     max_chunks);
    return me_check_launch("me_attention_prefill_combine");
  }
  return 0;
}

// ------------------------------------------------------------------------------------ the splits' sum inside the output projection
// For steps of very few items: the output projection behind decode attention reads the splits' partial results itself,
// so that the kernel that adds them up is not launched (a launch costs such a step more than the kernel's work). The
// heads are dealt to runs of k (HPR heads a run); a block owns one run and 64 output columns, for all rows. It asks
// for everything at its head (its weights, its heads' partial results, their statistics: one trip to memory), adds up
// the splits of each (row, head) pair as attention_decode_combine_kernel does, rounds the result to bfloat16 as that
// kernel's output is, and multiplies: parts[run][row][n] = sum over the run's k of out[row][k] W[n][k], float32, for the
// next add-and-norm to add up in their order. Every block of a run adds up the run's heads again, so this pays for narrow
// products only (measured on 16 heads of 128 and 1,024 columns, one row, 64 splits: 16 runs x 16 blocks of columns 2.8%
// of a step ahead of the two kernels, 8 runs x 16 1.7%, 16 x 8 blocks of 128 columns 1.2%, 8 x 8 0.5% behind; with
// two rows 1.4% behind at best).
#define OUT_MAX_SPLITS 128  // splits a (row, head) pair may have here
#define OUT_MAX_ROWS 4
#define OUT_EARLY 16        // partial results a thread asks for before it knows their weights

template <int D, int HPR>
__global__ __launch_bounds__(256) void attention_out_product_kernel(const float* __restrict__ part_o,
                                                                    const float* __restrict__ part_ml, int num_splits,
                                                                    const bf16_t* __restrict__ W, float* __restrict__ parts,
                                                                    int items, int nh, int N, int gpp) {
  constexpr int QUADS = D / 4;         // threads across a head's outputs, four each
  constexpr int GROUPS = 256 / QUADS;  // groups of such threads; gpp of them share the splits of one (row, head) pair
  constexpr int XROW = HPR * D + 8;    // LDS row stride in elements: 16 bytes off a multiple of 128
  __shared__ float2 ml[GROUPS][OUT_MAX_SPLITS];  // statistics by pair and split (pairs <= GROUPS)
  __shared__ float red[8];                        // maxima of the half-waves
  __shared__ float4_t partial[256];
  __shared__ float pdenom[GROUPS];
  __shared__ __attribute__((aligned(16))) uint16_t xs[OUT_MAX_ROWS][XROW];
  const int run = blockIdx.x, head0 = run * HPR;
  const int heads_here = min(HPR, nh - head0);
  const int tid = threadIdx.x, lane = tid & (ME_WAVE - 1), wave = tid / ME_WAVE, r = lane & 15, g = lane >> 4;
  const size_t K = (size_t)nh * D;
  const int n0 = ((int)blockIdx.y * 4 + wave) * 16;

  // ---- the wave's weights, as the first product operand: lane -> row n0 + r, eight k from 32 c + 8 g
  bf16x8_t w[HPR][D / 32];
#pragma unroll
  for (int hl = 0; hl < HPR; ++hl)
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      w[hl][c] = bf16x8_t{};
      if (n0 + r < N && hl < heads_here)
        w[hl][c] = *reinterpret_cast<const bf16x8_t*>(W + (size_t)(n0 + r) * K + (size_t)(head0 + hl) * D + c * 32 + g * 8);
    }

  // ---- this thread's (row, head) pair and its share of the pair's splits
  const int qd = tid % QUADS, grp = tid / QUADS;
  const int pair = grp / gpp, sub = grp % gpp;
  const int row = pair / HPR, hl_own = pair % HPR;
  const bool pair_ok = row < items && hl_own < heads_here;
  const size_t unit = (size_t)row * nh + head0 + hl_own;
  const float* po = part_o + unit * num_splits * D + qd * 4;
  float4_t early[OUT_EARLY];
#pragma unroll
  for (int i = 0; i < OUT_EARLY; ++i) {
    const int sp = sub + i * gpp;
    early[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
    if (pair_ok && sp < num_splits) early[i] = *reinterpret_cast<const float4_t*>(po + (size_t)sp * D);
  }
  // the statistics of the pair's splits, dealt to the pair's threads; their maximum over the pair
  const int pair_threads = QUADS * gpp, in_pair = sub * QUADS + qd;  // 32 or more threads
  float big = -INFINITY;
  for (int sp = in_pair; sp < num_splits; sp += pair_threads) {
    float2 st = make_float2(-INFINITY, 0.f);
    if (pair_ok) st = *reinterpret_cast<const float2*>(part_ml + (unit * num_splits + sp) * 2);
    ml[pair][sp] = st;
    if (st.y > 0.f) big = fmaxf(big, st.x);  // an empty split has no weight
  }
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) big = fmaxf(big, __shfl_xor(big, off, ME_WAVE));  // over the half-wave
  if ((lane & 31) == 0) red[tid / 32] = big;
  __syncthreads();
  {
    const int first = pair * pair_threads / 32;
    big = red[first];
    for (int i = 1; i < pair_threads / 32; ++i) big = fmaxf(big, red[first + i]);
  }
  float4_t accv = {0.f, 0.f, 0.f, 0.f};
  float dsum = 0.f;
  if (pair_ok) {
#pragma unroll
    for (int i = 0; i < OUT_EARLY; ++i) {
      const int sp = sub + i * gpp;
      if (sp < num_splits) {
        const float2 st = ml[pair][sp];
        const float wgt = st.y > 0.f ? fast_exp2(st.x - big) : 0.f;
        dsum += wgt * st.y;
        accv[0] += wgt * early[i][0];
        accv[1] += wgt * early[i][1];
        accv[2] += wgt * early[i][2];
        accv[3] += wgt * early[i][3];
      }
    }
    for (int sp = sub + OUT_EARLY * gpp; sp < num_splits; sp += gpp) {
      const float2 st = ml[pair][sp];
      const float wgt = st.y > 0.f ? fast_exp2(st.x - big) : 0.f;
      const float4_t v = *reinterpret_cast<const float4_t*>(po + (size_t)sp * D);
      dsum += wgt * st.y;
      accv[0] += wgt * v[0];
      accv[1] += wgt * v[1];
      accv[2] += wgt * v[2];
      accv[3] += wgt * v[3];
    }
  }
  partial[tid] = accv;
  if (qd == 0) pdenom[grp] = dsum;
  __syncthreads();
  if (pair_ok && sub == 0) {
    float4_t total = accv;
    float denom = dsum;
    for (int i = 1; i < gpp; ++i) {
      const float4_t v = partial[(grp + i) * QUADS + qd];
      total[0] += v[0];
      total[1] += v[1];
      total[2] += v[2];
      total[3] += v[3];
      denom += pdenom[grp + i];
    }
    const float inv = denom > 0.f ? 1.f / denom : 0.f;  // no visible key at all: zeros, not NaN
    *reinterpret_cast<short4_t*>(&xs[row][hl_own * D + qd * 4]) =
        pack_bf16x4(total[0] * inv, total[1] * inv, total[2] * inv, total[3] * inv);
  }
  __syncthreads();

  // ---- parts[run][m][n] = sum_k W[n][k] out[m][k]: lane -> out row r (rows beyond the items are zeros)
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int hl = 0; hl < HPR; ++hl) {
    if (hl >= heads_here) break;
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
      bf16x8_t xf = bf16x8_t{};
      if (r < items) xf = *reinterpret_cast<const bf16x8_t*>(&xs[r][hl * D + c * 32 + g * 8]);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[hl][c], xf, acc, 0, 0, 0);
    }
  }
  if (r < items) {
    const int n = n0 + g * 4;
    if (n < N) *reinterpret_cast<float4_t*>(parts + ((size_t)run * items + r) * N + n) = acc;  // N is a multiple of 4
  }
}

// Heads per run of k, for at most `OUT_RUNS` runs.
#define OUT_RUNS 16
static int out_heads_per_run(int nh) {
  int hpr = 1;
  while ((nh + hpr - 1) / hpr > OUT_RUNS) hpr *= 2;
  return hpr;
}

// How many runs of k (float32 partial sums) me_attention_out_product_bf16 writes for nh heads.
extern "C" int me_attention_out_product_runs(int nh) {
  if (nh <= 0) return 0;
  const int hpr = out_heads_per_run(nh);
  return (nh + hpr - 1) / hpr;
}

// Sizes that me_attention_out_product_bf16 takes: up to 4 rows, heads of 64 or 128, up to 128 splits, a width that is
// a multiple of 8, and at most 8 (row, head) pairs a block.
extern "C" int me_attention_out_product_supported(int items, int nh, int d, int n, int num_splits) {
  if (items <= 0 || items > OUT_MAX_ROWS || nh <= 0 || (d != 64 && d != 128) || n <= 0 || n % 8) return 0;
  if (num_splits <= 0 || num_splits > OUT_MAX_SPLITS) return 0;
  const int hpr = out_heads_per_run(nh);
  if (hpr > 4) return 0;
  int pairs = 1;
  while (pairs < items * hpr) pairs *= 2;
  return pairs <= 8;  // 32 threads or more a pair, whatever the head size
}

// part_o float [items * nh, num_splits, d], part_ml float [items * nh, num_splits, 2]: what a decode attention launch
// without `out` left. W bf16 [n, nh * d]. parts float [runs, items, n] (runs: me_attention_out_product_runs(nh)).
extern "C" int me_attention_out_product_bf16(const float* part_o, const float* part_ml, int num_splits, const void* W,
                                             float* parts, int items, int nh, int d, int n, hipStream_t stream) {
  if (!me_attention_out_product_supported(items, nh, d, n, num_splits))
    return me_fail("me_attention_out_product_bf16: items=%d heads=%d head_dim=%d width=%d splits=%d not supported", items, nh,
                   d, n, num_splits);
  if (!part_o || !part_ml || !W || !parts) return me_fail("me_attention_out_product_bf16: null operand");
  if (((uintptr_t)W | (uintptr_t)part_o | (uintptr_t)parts) & 15 || (uintptr_t)part_ml & 7)
    return me_fail("me_attention_out_product_bf16: operands must start at multiples of 16 bytes (the statistics: of 8)");
  const int hpr = out_heads_per_run(nh);
  const int runs = (nh + hpr - 1) / hpr;
  int pairs = 1;
  while (pairs < items * hpr) pairs *= 2;
  const int groups = 256 / (d / 4);
  const int gpp = groups / pairs;
  dim3 grid(runs, (n + 63) / 64);
  const bf16_t* w = (const bf16_t*)W;
#define ME_OUT_CASE(DD, HH) \
  if (d == DD && hpr == HH) attention_out_product_kernel<DD, HH><<<grid, 256, 0, stream>>>(part_o, part_ml, num_splits, w, parts, items, nh, n, gpp);
  ME_OUT_CASE(64, 1)
  ME_OUT_CASE(64, 2)
  ME_OUT_CASE(64, 4)
  ME_OUT_CASE(128, 1)
  ME_OUT_CASE(128, 2)
  ME_OUT_CASE(128, 4)
#undef ME_OUT_CASE
  return me_check_launch("me_attention_out_product_bf16");
}
