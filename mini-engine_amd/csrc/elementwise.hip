// Row-wise kernels around the matrix products: embedding lookup, residual add + RMSNorm,
// SwiGLU, and the fused per-head q/k RMSNorm + rotary encoding + key/value page write.
//
// All arithmetic is float32; T is the storage type of activations (float or bf16_t). The residual
// stream and the norm weights are float32 in both modes.
#include "common.h"

// ---------------------------------------------------------------------------------- embedding
// x[t, :] = table[ids[t], :] * scale as float32. One block per token.
template <typename T>
__global__ void embed_kernel(float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ ids,
                             int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // ids are validated on the host; never fault
  const T* row = table + (size_t)id * hidden;
  float* out = x + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = to_float(row[i]) * scale;
}

extern "C" int me_embed(void* x, const void* table, const int* ids, int num_tokens, int hidden, int vocab, float scale,
                        int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (hidden <= 0 || vocab <= 0) return me_fail("me_embed: hidden=%d vocab=%d", hidden, vocab);
  const int threads = hidden >= 256 ? 256 : 64;
  if (dtype == ME_F32)
    embed_kernel<float><<<num_tokens, threads, 0, stream>>>((float*)x, (const float*)table, ids, hidden, vocab, scale);
  else
    embed_kernel<bf16_t><<<num_tokens, threads, 0, stream>>>((float*)x, (const bf16_t*)table, ids, hidden, vocab, scale);
  return me_check_launch("me_embed");
}

// The same lookup for a step whose token ids are still on the device: where fed_rows[t] >= 0 the id of token t
// is fed_tokens[fed_rows[t]], what an earlier step's sampling kernel wrote there, not ids[t]. A decode step
// can then be launched before the host has read the tokens of the step before it.
template <typename T>
__global__ void embed_fed_kernel(float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ ids,
                                 const int* __restrict__ fed_rows, const int* __restrict__ fed_tokens, int hidden,
                                 int vocab, float scale) {
  const int t = blockIdx.x;
  const int from = fed_rows[t];
  int id = from >= 0 ? fed_tokens[from] : ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (size_t)id * hidden;
  float* out = x + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = to_float(row[i]) * scale;
}

extern "C" int me_embed_fed(void* x, const void* table, const int* ids, const int* fed_rows, const int* fed_tokens,
                            int num_tokens, int hidden, int vocab, float scale, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (hidden <= 0 || vocab <= 0) return me_fail("me_embed_fed: hidden=%d vocab=%d", hidden, vocab);
  if (!fed_rows || !fed_tokens) return me_fail("me_embed_fed: no fed rows or tokens");
  const int threads = hidden >= 256 ? 256 : 64;
  if (dtype == ME_F32)
    embed_fed_kernel<float><<<num_tokens, threads, 0, stream>>>((float*)x, (const float*)table, ids, fed_rows, fed_tokens,
                                                                hidden, vocab, scale);
  else
    embed_fed_kernel<bf16_t><<<num_tokens, threads, 0, stream>>>((float*)x, (const bf16_t*)table, ids, fed_rows, fed_tokens,
                                                                 hidden, vocab, scale);
  return me_check_launch("me_embed_fed");
}

// ---------------------------------------------------------------------- residual add + RMSNorm
// For output row r (input row src = rows ? rows[r] : r):
//   s = x[src] + (delta ? delta[src] : 0);  if (write_x) x[src] = s;
//   h[r] = s * rsqrt(mean(s^2) + eps) * w
// One block per row; the sum of squares is reduced in a fixed order.
// `parts` (float32 [num_parts, total rows, dim], or null) is a delta that still is a sum: partial
// products over runs of k, added here in the order of the runs.
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ delta, const float* __restrict__ parts,
                                   int num_parts, size_t part_stride, const float* __restrict__ w, T* __restrict__ h,
                                   const int* __restrict__ rows, int dim, float eps, int write_x) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + (size_t)src * dim;
  const T* dr = delta ? delta + (size_t)src * dim : nullptr;
  const float* pr = parts ? parts + (size_t)src * dim : nullptr;
  const bool adds = dr || pr;
  auto sum_at = [&](int i) {
    float s = xr[i];
    if (dr) s += to_float(dr[i]);
    if (pr) {
      float d = pr[i];
      for (int p = 1; p < num_parts; ++p) d += pr[p * part_stride + i];
      s += d;
    }
    return s;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const float s = sum_at(i);
    if (write_x && adds) xr[i] = s;
    ss += s * s;
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / (float)dim + eps);
  T* hr = h + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const float s = (adds && !write_x) ? sum_at(i) : xr[i];
    hr[i] = from_float<T>(s * inv * w[i]);
  }
}

// The same for rows whose length is a multiple of 4 and at most 16 elements per thread: a thread keeps its four
// vectors of 4 sums in registers (one pass over memory), loads 16 bytes at a time and has the loads of four
// partial sums in flight at once (a row of 5,120 with 7 partial sums: 41 -> 7 us). PB partial sums are requested
// together (4, or 8 where there are more than 4: a trip to memory for all of them instead of one for four and one for
// each of the rest); a run beyond the last reads the last one again and counts for nothing.
template <typename T, int PB>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ x, const T* __restrict__ delta, const float* __restrict__ parts,
                                       int num_parts, size_t part_stride, const float* __restrict__ w, T* __restrict__ h,
                                       const int* __restrict__ rows, int dim, float eps, int write_x) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + (size_t)src * dim;
  const T* dr = delta ? delta + (size_t)src * dim : nullptr;
  const float* pr = parts ? parts + (size_t)src * dim : nullptr;
  struct alignas(sizeof(T) * 4) Pack {
    T v[4];
  };
  const int nvec = dim / 4;
  float4 s[4], wv[4];  // (the norm's weight is requested with the row, not behind the sum over the block: the tail waits for nothing)
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int v = threadIdx.x + it * blockDim.x;
    s[it] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (v < nvec) {
      s[it] = *reinterpret_cast<const float4*>(xr + 4 * v);
      wv[it] = *reinterpret_cast<const float4*>(w + 4 * v);
      if (dr) {
        const Pack d = *reinterpret_cast<const Pack*>(dr + 4 * v);
        s[it].x += to_float(d.v[0]), s[it].y += to_float(d.v[1]), s[it].z += to_float(d.v[2]), s[it].w += to_float(d.v[3]);
      }
      if (pr) {  // in the order of the runs
        float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
        const float* at = pr + 4 * v;
        for (int q = 0; q < num_parts; q += PB) {
          float4 pv[PB];
#pragma unroll
          for (int i = 0; i < PB; ++i) pv[i] = *reinterpret_cast<const float4*>(at + (size_t)min(q + i, num_parts - 1) * part_stride);
#pragma unroll
          for (int i = 0; i < PB; ++i) {
            const float on = q + i < num_parts ? 1.f : 0.f;
            d.x += on * pv[i].x, d.y += on * pv[i].y, d.z += on * pv[i].z, d.w += on * pv[i].w;
          }
        }
        s[it].x += d.x, s[it].y += d.y, s[it].z += d.z, s[it].w += d.w;
      }
      if ((dr || pr) && write_x) *reinterpret_cast<float4*>(xr + 4 * v) = s[it];
      ss = fmaf(s[it].x, s[it].x, ss), ss = fmaf(s[it].y, s[it].y, ss), ss = fmaf(s[it].z, s[it].z, ss), ss = fmaf(s[it].w, s[it].w, ss);
    }
  }
  const float inv = rsqrtf(block_sum(ss, scratch) / (float)dim + eps);
  T* hr = h + (size_t)r * dim;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int v = threadIdx.x + it * blockDim.x;
    if (v < nvec) {
      Pack o;
      o.v[0] = from_float<T>(s[it].x * inv * wv[it].x), o.v[1] = from_float<T>(s[it].y * inv * wv[it].y);
      o.v[2] = from_float<T>(s[it].z * inv * wv[it].z), o.v[3] = from_float<T>(s[it].w * inv * wv[it].w);
      *reinterpret_cast<Pack*>(hr + 4 * v) = o;
    }
  }
}

template <typename T>
static bool launch_add_rmsnorm_vec(float* x, const T* delta, const float* parts, int num_parts, size_t part_stride,
                                   const float* w, T* h, const int* rows, int num_rows, int dim, float eps, int write_x,
                                   hipStream_t stream) {
  if (dim % 4 || dim > 16384) return false;
  if (((uintptr_t)x | (uintptr_t)parts | (uintptr_t)w) & 15 || ((uintptr_t)delta | (uintptr_t)h) & (sizeof(T) * 4 - 1) || part_stride % 4)
    return false;
  const int nvec = dim / 4;
  // a vector per thread where a block can have that many threads: all loads of a row are in flight at once (against a
  // wave per row with the row in its registers: 64 rows of 1,024 with 6 partial sums 3.1 us against 3.9, of 4,096 with 8
  // 4.1 against 9.8; 512 rows of 4,096 5.9 against 10.0; 2,048 rows of 1,024 5.5 against 6.2). A function of the row's
  // length alone: a row's sum of squares is added up in the same order whatever the number of rows.
  const int threads = nvec <= 64 ? 64 : (nvec <= 128 ? 128 : (nvec <= 256 ? 256 : (nvec <= 512 ? 512 : 1024)));
  if (parts && num_parts > 4)
    add_rmsnorm_vec_kernel<T, 8><<<num_rows, threads, 0, stream>>>(x, delta, parts, num_parts, part_stride, w, h, rows, dim, eps,
                                                                   write_x);
  else
    add_rmsnorm_vec_kernel<T, 4><<<num_rows, threads, 0, stream>>>(x, delta, parts, num_parts, part_stride, w, h, rows, dim, eps,
                                                                   write_x);
  return true;
}

// x *= scale over `count` float32 elements (a model's scale on its logits).
__global__ void scale_kernel(float* __restrict__ x, float scale, size_t count) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) x[i] *= scale;
}

extern "C" int me_scale_f32(float* x, float scale, long long count, hipStream_t stream) {
  if (count <= 0) return 0;
  const size_t want = ((size_t)count + 255) / 256;
  scale_kernel<<<(int)(want < 4096 ? want : 4096), 256, 0, stream>>>(x, scale, (size_t)count);
  return me_check_launch("me_scale_f32");
}

// The residual add alone, for a norm that is not of this shape and runs as a part of its own:
// x += delta (+ the partial sums, in the order of the runs).
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ delta, const float* __restrict__ parts,
                                    int num_parts, size_t part_stride, size_t count) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    float s = x[i];
    if (delta) s += to_float(delta[i]);
    if (parts) {
      float d = parts[i];
      for (int p = 1; p < num_parts; ++p) d += parts[p * part_stride + i];
      s += d;
    }
    x[i] = s;
  }
}

extern "C" int me_residual_add(void* x, const void* delta, const float* parts, int num_parts, long long part_stride,
                               int num_rows, int dim, int dtype, hipStream_t stream) {
  if (num_rows <= 0 || dim <= 0) return 0;
  if (!delta && !parts) return 0;
  if (parts && num_parts < 1) return me_fail("me_residual_add: partial sums without parts");
  const size_t count = (size_t)num_rows * dim;
  const size_t want = (count + 255) / 256;
  const int blocks = (int)(want < 4096 ? want : 4096);
  if (dtype == ME_F32)
    residual_add_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, (const float*)delta, parts, num_parts,
                                                           (size_t)part_stride, count);
  else
    residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>((float*)x, (const bf16_t*)delta, parts, num_parts,
                                                            (size_t)part_stride, count);
  return me_check_launch("me_residual_add");
}

extern "C" int me_add_rmsnorm(void* x, const void* delta, const float* parts, int num_parts, long long part_stride,
                              const float* w, void* h, const int* rows, int num_rows, int dim, float eps, int write_x,
                              int dtype, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (dim <= 0) return me_fail("me_add_rmsnorm: dim=%d", dim);
  if (parts && (num_parts < 1 || part_stride < (long long)dim)) return me_fail("me_add_rmsnorm: %d partial sums", num_parts);
  if (dtype == ME_F32 ? launch_add_rmsnorm_vec<float>((float*)x, (const float*)delta, parts, num_parts, (size_t)part_stride, w,
                                                      (float*)h, rows, num_rows, dim, eps, write_x, stream)
                      : launch_add_rmsnorm_vec<bf16_t>((float*)x, (const bf16_t*)delta, parts, num_parts, (size_t)part_stride,
                                                       w, (bf16_t*)h, rows, num_rows, dim, eps, write_x, stream))
    return me_check_launch("me_add_rmsnorm");
  const int threads = dim >= 2048 ? 512 : (dim >= 512 ? 256 : (dim >= 128 ? 128 : 64));
  if (dtype == ME_F32)
    add_rmsnorm_kernel<float><<<num_rows, threads, 0, stream>>>((float*)x, (const float*)delta, parts, num_parts,
                                                                (size_t)part_stride, w, (float*)h, rows, dim, eps, write_x);
  else
    add_rmsnorm_kernel<bf16_t><<<num_rows, threads, 0, stream>>>((float*)x, (const bf16_t*)delta, parts, num_parts,
                                                                 (size_t)part_stride, w, (bf16_t*)h, rows, dim, eps,
                                                                 write_x);
  return me_check_launch("me_add_rmsnorm");
}

// Plain RMSNorm over rows of T (used by parts tests and by mixers that norm activations):
// out[r] = in[r] * rsqrt(mean(in[r]^2) + eps) * w
template <typename T>
__global__ void rmsnorm_kernel(const T* __restrict__ in, const float* __restrict__ w, T* __restrict__ out, int dim,
                               float eps) {
  __shared__ float scratch[16];
  const T* xr = in + (size_t)blockIdx.x * dim;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const float s = to_float(xr[i]);
    ss += s * s;
  }
  const float inv = rsqrtf(block_sum(ss, scratch) / (float)dim + eps);
  T* o = out + (size_t)blockIdx.x * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = from_float<T>(to_float(xr[i]) * inv * w[i]);
}

extern "C" int me_rmsnorm(const void* in, const float* w, void* out, int num_rows, int dim, float eps, int dtype,
                          hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (dim <= 0) return me_fail("me_rmsnorm: dim=%d", dim);
  const int threads = dim >= 2048 ? 512 : (dim >= 512 ? 256 : (dim >= 128 ? 128 : 64));
  if (dtype == ME_F32)
    rmsnorm_kernel<float><<<num_rows, threads, 0, stream>>>((const float*)in, w, (float*)out, dim, eps);
  else
    rmsnorm_kernel<bf16_t><<<num_rows, threads, 0, stream>>>((const bf16_t*)in, w, (bf16_t*)out, dim, eps);
  return me_check_launch("me_rmsnorm");
}

// ------------------------------------------------------------------------------------ SwiGLU
// act[t, i] = a(gu[t, i]) * gu[t, inter + i], a = silu (z / (1 + exp(-z))) or tanh-gelu by `gate`. A thread handles VEC
// consecutive i (16-byte loads when the row length allows it).
template <typename T, int VEC>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ act, int inter, size_t total_vec, int gate) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_vec) return;
  const int per_row = inter / VEC;
  const size_t t = idx / per_row;
  const int i = (int)(idx - t * per_row) * VEC;
  struct alignas(sizeof(T) * VEC) Pack {
    T v[VEC];
  };
  const Pack g = *reinterpret_cast<const Pack*>(gu + t * 2 * inter + i);
  const Pack u = *reinterpret_cast<const Pack*>(gu + t * 2 * inter + inter + i);
  Pack o;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const float gf = to_float(g.v[k]);
    o.v[k] = from_float<T>((sizeof(T) == 2 ? gate_act_bf16(gf, gate) : gate_act(gf, gate)) * to_float(u.v[k]));
  }
  *reinterpret_cast<Pack*>(act + t * inter + i) = o;
}

template <typename T>
static void launch_swiglu(const T* gu, T* act, int num_tokens, int inter, int gate, hipStream_t stream) {
  constexpr int WIDE = 16 / sizeof(T);
  const bool wide = inter % WIDE == 0 && ((uintptr_t)gu % 16 == 0) && ((uintptr_t)act % 16 == 0);
  const int threads = 256;
  if (wide) {
    const size_t total = (size_t)num_tokens * (inter / WIDE);
    swiglu_kernel<T, WIDE><<<(unsigned)((total + threads - 1) / threads), threads, 0, stream>>>(gu, act, inter, total, gate);
  } else {
    const size_t total = (size_t)num_tokens * inter;
    swiglu_kernel<T, 1><<<(unsigned)((total + threads - 1) / threads), threads, 0, stream>>>(gu, act, inter, total, gate);
  }
}

extern "C" int me_swiglu(const void* gu, void* act, int num_tokens, int inter, int gate, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (inter <= 0) return me_fail("me_swiglu: intermediate=%d", inter);
  if (gate != ME_GATE_SILU && gate != ME_GATE_GELU_TANH) return me_fail("me_swiglu: unknown gate activation %d", gate);
  if (dtype == ME_F32)
    launch_swiglu<float>((const float*)gu, (float*)act, num_tokens, inter, gate, stream);
  else
    launch_swiglu<bf16_t>((const bf16_t*)gu, (bf16_t*)act, num_tokens, inter, gate, stream);
  return me_check_launch("me_swiglu");
}

// ------------------------------------------------------------------- rotary cos/sin table
// table[pos, 0, j] = cos(pos * inv_freq[j]), table[pos, 1, j] = sin(pos * inv_freq[j]) in float32, with
// the accurate library routines (angles reach tens of thousands of radians). Computed once per model;
// every kernel that rotates reads it, so all of them see the same bits for a position.
__global__ void rope_table_kernel(float* __restrict__ table, const float* __restrict__ inv_freq, int half,
                                  int num_positions) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= num_positions * half) return;
  const int pos = idx / half, j = idx % half;
  const float angle = (float)pos * inv_freq[j];
  table[((size_t)pos * 2) * half + j] = cosf(angle);
  table[((size_t)pos * 2 + 1) * half + j] = sinf(angle);
}

extern "C" int me_rope_table(float* table, const float* inv_freq, int half, int num_positions, hipStream_t stream) {
  if (half <= 0 || num_positions <= 0) return me_fail("me_rope_table: half=%d positions=%d", half, num_positions);
  const long long total = (long long)half * num_positions;
  rope_table_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(table, inv_freq, half, num_positions);
  return me_check_launch("me_rope_table");
}

// ------------------------------------------- per-head q/k RMSNorm + rotary + key/value page write
// qkv is [T, (nh + 2*nkv) * d]: q heads, then k heads, then v heads. Grid (token, group of heads),
// four waves per block, a wave per head at a time:
//   q heads: optional RMSNorm over d with q_w, rotary, written to q_out [T, nh, d];
//   k heads: optional RMSNorm with k_w, rotary, written to the key page   K[page, kvh, slot, d];
//   v heads: copied to the transposed value page                          V[page, kvh, d, slot].
// page = block_table[item, pos / bs], slot = pos % bs. Rotary: pairs (j, j + rd/2), j < rd/2, with
// cos/sin of pos * inv_freq[j] read from rope_table [positions, 2, rd/2]; dims >= rd pass through.
// rope_table == nullptr means no rotary.
// write_kv == 0: qkv is [T, nh * d] and only q is processed (a layer that reads another layer's cache).
#define ME_MAX_HEAD_DIM 256

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_scatter_kernel(
    const T* __restrict__ qkv, const float* __restrict__ q_w, const float* __restrict__ k_w,
    const float* __restrict__ rope_table, const int* __restrict__ positions, const int* __restrict__ token_item,
    const int* __restrict__ block_table, int table_width, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int nh, int nkv, int d, int rd, int bs, float eps, int write_kv, int heads_per_block,
    int skip_v) {
  __shared__ float stage[4][ME_MAX_HEAD_DIM];
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int t = blockIdx.x;
  const int heads_row = write_kv ? nh + 2 * nkv : nh;
  const int heads_total = skip_v ? nh + nkv : heads_row;  // value heads are written by the page-tile kernel
  const int width = heads_row * d;  // q-only rows when nothing is written
  const int pos = positions[t];
  const int half = rd / 2;
  const float* cs = rope_table ? rope_table + (size_t)pos * rd : nullptr;  // [2, half] of this position
  int page = 0, slot = 0;
  if (write_kv) {
    page = block_table[(size_t)token_item[t] * table_width + pos / bs];
    slot = pos % bs;
  }
  const int hd_end = min(heads_total, (int)(blockIdx.y + 1) * heads_per_block);
  for (int hd = blockIdx.y * heads_per_block + wave; hd < hd_end; hd += 4) {
    const T* src = qkv + (size_t)t * width + (size_t)hd * d;
    const int kind = hd < nh ? 0 : (hd < nh + nkv ? 1 : 2);
    float vals[ME_MAX_HEAD_DIM / ME_WAVE];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
      const int i = lane + k * ME_WAVE;
      vals[k] = i < d ? to_float(src[i]) : 0.f;
      ss += vals[k] * vals[k];
    }
    const float* w = kind == 0 ? q_w : (kind == 1 ? k_w : nullptr);
    if (w) {
      const float inv = rsqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
      for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
        const int i = lane + k * ME_WAVE;
        if (i < d) vals[k] = vals[k] * inv * w[i];
      }
    }
    if (kind != 2 && cs) {
      float* st = stage[wave];
      __builtin_amdgcn_wave_barrier();  // the previous head's reads of this wave's stage are done
#pragma unroll
      for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
        const int i = lane + k * ME_WAVE;
        if (i < d) st[i] = vals[k];
      }
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): LDS writes of this wave are visible
#pragma unroll
      for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
        const int i = lane + k * ME_WAVE;
        if (i < rd) {
          const int j = i < half ? i : i - half;
          const float c = cs[j], sn = cs[half + j];
          vals[k] = i < half ? st[i] * c - st[i + half] * sn : st[i] * c + st[i - half] * sn;
        }
      }
    }
    if (kind == 0) {
      T* dst = q_out + ((size_t)t * nh + hd) * d;
#pragma unroll
      for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
        const int i = lane + k * ME_WAVE;
        if (i < d) dst[i] = from_float<T>(vals[k]);
      }
    } else if (page >= 0) {
      if (kind == 1) {
        const int kvh = hd - nh;
        T* dst = k_cache + (((size_t)page * nkv + kvh) * bs + slot) * d;
#pragma unroll
        for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
          const int i = lane + k * ME_WAVE;
          if (i < d) dst[i] = from_float<T>(vals[k]);
        }
      } else {
        const int kvh = hd - nh - nkv;
        T* dst = v_cache + ((size_t)page * nkv + kvh) * d * bs + slot;
#pragma unroll
        for (int k = 0; k < ME_MAX_HEAD_DIM / ME_WAVE; ++k) {
          const int i = lane + k * ME_WAVE;
          if (i < d) dst[(size_t)i * bs] = from_float<T>(vals[k]);
        }
      }
    }
  }
}

// Eight consecutive elements, moved as one access.
template <typename T>
struct alignas(sizeof(T) * 8) Pack8 {
  T v[8];
};

// Values of many consecutive tokens: one block per (16-slot segment of a page that the step's tokens
// touch, kv head). The segment's tokens are read row by row into LDS and written transposed, 16 slots
// (32 bytes) per head dimension, instead of one 2-byte store per (token, dimension). Segments are
// numbered over all items; item i touches segments pos0/16 .. (pos0 + qlen - 1)/16 of its positions.
template <typename T>
struct VScatterLds {
  T tile[16][ME_MAX_HEAD_DIM + 2];
  int item, seg;
};

// The work of one block (256 threads, all of which call it): segment `segment` of the step, kv head `kvh`.
template <typename T>
__device__ __forceinline__ void v_scatter_segment(VScatterLds<T>& lds, int segment, int kvh, const T* __restrict__ qkv,
                                                  const int* __restrict__ positions, const int* __restrict__ item_start,
                                                  int num_items, const int* __restrict__ block_table, int table_width,
                                                  T* __restrict__ v_cache, int nh, int nkv, int d, int bs) {
  T(&tile)[16][ME_MAX_HEAD_DIM + 2] = lds.tile;
  int& s_item = lds.item;
  int& s_seg = lds.seg;
  if (threadIdx.x == 0) {
    int left = segment, it = 0;
    for (; it < num_items; ++it) {
      const int p0 = positions[item_start[it]], n = item_start[it + 1] - item_start[it];
      const int segs = (p0 + n - 1) / 16 - p0 / 16 + 1;
      if (left < segs) break;
      left -= segs;
    }
    s_item = it;
    s_seg = left;
  }
  __syncthreads();
  const int item = s_item;
  if (item >= num_items) return;
  const int t0 = item_start[item], n = item_start[item + 1] - t0;
  const int p0 = positions[t0];
  const int seg_pos = (p0 / 16 + s_seg) * 16;           // first position of the segment
  const int first = max(seg_pos, p0), last = min(seg_pos + 15, p0 + n - 1);  // positions present
  const int width = (nh + 2 * nkv) * d;
  const T* src = qkv + (size_t)(nh + nkv + kvh) * d;
  const bool wide = d % 8 == 0 && (((uintptr_t)qkv | (uintptr_t)v_cache) & (sizeof(T) * 8 - 1)) == 0;
  if (wide) {  // rows in pieces of eight elements
    for (int idx = threadIdx.x; idx < (last - first + 1) * (d / 8); idx += blockDim.x) {
      const int row = idx / (d / 8), col = idx % (d / 8) * 8;
      const Pack8<T> v = *reinterpret_cast<const Pack8<T>*>(src + (size_t)(t0 + first - p0 + row) * width + col);
#pragma unroll
      for (int j = 0; j < 8; ++j) tile[first - seg_pos + row][col + j] = v.v[j];
    }
  } else {
    for (int idx = threadIdx.x; idx < (last - first + 1) * d; idx += blockDim.x) {
      const int row = idx / d, col = idx % d;
      tile[first - seg_pos + row][col] = src[(size_t)(t0 + first - p0 + row) * width + col];
    }
  }
  __syncthreads();
  const int page = block_table[(size_t)item * table_width + seg_pos / bs];
  if (page < 0) return;
  T* dst = v_cache + ((size_t)page * nkv + kvh) * d * bs + seg_pos % bs;
  const int lo = first - seg_pos, hi = last - seg_pos;
  if (wide && lo == 0 && hi == 15) {  // a whole segment: eight slots of one dimension per store
    for (int idx = threadIdx.x; idx < d * 2; idx += blockDim.x) {
      const int dim = idx >> 1, half = idx & 1;
      Pack8<T> v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v.v[j] = tile[half * 8 + j][dim];
      *reinterpret_cast<Pack8<T>*>(dst + (size_t)dim * bs + half * 8) = v;
    }
    return;
  }
  for (int idx = threadIdx.x; idx < d * 16; idx += blockDim.x) {
    const int dim = idx / 16, slot = idx % 16;
    if (slot >= lo && slot <= hi) dst[(size_t)dim * bs + slot] = tile[slot][dim];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void v_scatter_tiles_kernel(const T* __restrict__ qkv, const int* __restrict__ positions,
                                                              const int* __restrict__ item_start, int num_items,
                                                              const int* __restrict__ block_table, int table_width,
                                                              T* __restrict__ v_cache, int nh, int nkv, int d, int bs) {
  __shared__ VScatterLds<T> lds;
  v_scatter_segment<T>(lds, blockIdx.x, blockIdx.y, qkv, positions, item_start, num_items, block_table, table_width,
                       v_cache, nh, nkv, d, bs);
}

// The same work for the common geometry (head size a power of two from 16 to 256, rotary over the
// whole head or none): a lane owns eight consecutive dims of the lower half of a head and their rotary
// partners half a head away, so no value has to cross lanes for the rotation, loads and stores are
// 8 elements wide (16 bytes in bfloat16), and a wave handles 64 / (d/16) heads at a time. Unit u of the
// grid is (token, head) = (u / heads, u % heads).
template <typename T, int LPH>  // LPH = d / 16 lanes per head
__global__ __launch_bounds__(256) void qk_norm_rope_scatter_wide_kernel(
    const T* __restrict__ qkv, const float* __restrict__ q_w, const float* __restrict__ k_w,
    const float* __restrict__ rope_table, const int* __restrict__ positions, const int* __restrict__ token_item,
    const int* __restrict__ block_table, int table_width, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int num_tokens, int nh, int nkv, int bs, float eps, int write_kv, int skip_v,
    const int* __restrict__ item_start, int num_items, unsigned own_blocks) {
  constexpr int D = LPH * 16, HALF = D / 2, HPW = 64 / LPH;  // heads per wave
  if (blockIdx.x >= own_blocks) {  // the blocks behind this kernel's own write the values, a page segment each
    __shared__ VScatterLds<T> lds;
    const unsigned v = blockIdx.x - own_blocks;
    v_scatter_segment<T>(lds, v / nkv, v % nkv, qkv, positions, item_start, num_items, block_table, table_width, v_cache,
                         nh, nkv, D, bs);
    return;
  }
  const int lane = threadIdx.x & (ME_WAVE - 1);
  const int sub = lane / LPH, p = lane % LPH;
  const int heads_row = write_kv ? nh + 2 * nkv : nh;
  const int heads = skip_v ? nh + nkv : heads_row;
  const long long unit = ((long long)blockIdx.x * (blockDim.x / ME_WAVE) + threadIdx.x / ME_WAVE) * HPW + sub;
  if (unit >= (long long)num_tokens * heads) return;
  const int t = (int)(unit / heads), hd = (int)(unit % heads);
  const int kind = hd < nh ? 0 : (hd < nh + nkv ? 1 : 2);
  const T* src = qkv + ((size_t)t * heads_row + hd) * D;
  const Pack8<T> lo = *reinterpret_cast<const Pack8<T>*>(src + 8 * p);
  const Pack8<T> hi = *reinterpret_cast<const Pack8<T>*>(src + 8 * p + HALF);
  float a[8], b[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = to_float(lo.v[j]);
    b[j] = to_float(hi.v[j]);
  }
  const int pos = positions[t];
  const float* w = kind == 0 ? q_w : (kind == 1 ? k_w : nullptr);
  if (w) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) ss = fmaf(a[j], a[j], fmaf(b[j], b[j], ss));
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, ME_WAVE);  // within the head's lanes
    const float inv = rsqrtf(ss / (float)D + eps);
    const float4 wa0 = *reinterpret_cast<const float4*>(w + 8 * p), wa1 = *reinterpret_cast<const float4*>(w + 8 * p + 4);
    const float4 wb0 = *reinterpret_cast<const float4*>(w + 8 * p + HALF),
                 wb1 = *reinterpret_cast<const float4*>(w + 8 * p + HALF + 4);
    const float wa[8] = {wa0.x, wa0.y, wa0.z, wa0.w, wa1.x, wa1.y, wa1.z, wa1.w};
    const float wb[8] = {wb0.x, wb0.y, wb0.z, wb0.w, wb1.x, wb1.y, wb1.z, wb1.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      a[j] *= inv * wa[j];
      b[j] *= inv * wb[j];
    }
  }
  if (kind != 2 && rope_table) {
    const float* cs = rope_table + (size_t)pos * D + 8 * p;  // [2, HALF]: cosines then sines
    const float4 c0 = *reinterpret_cast<const float4*>(cs), c1 = *reinterpret_cast<const float4*>(cs + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(cs + HALF), s1 = *reinterpret_cast<const float4*>(cs + HALF + 4);
    const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float ra = a[j] * c[j] - b[j] * sn[j], rb = b[j] * c[j] + a[j] * sn[j];
      a[j] = ra;
      b[j] = rb;
    }
  }
  Pack8<T> out_lo, out_hi;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    out_lo.v[j] = from_float<T>(a[j]);
    out_hi.v[j] = from_float<T>(b[j]);
  }
  if (kind == 0) {
    T* dst = q_out + ((size_t)t * nh + hd) * D;
    *reinterpret_cast<Pack8<T>*>(dst + 8 * p) = out_lo;
    *reinterpret_cast<Pack8<T>*>(dst + 8 * p + HALF) = out_hi;
    return;
  }
  const int page = block_table[(size_t)token_item[t] * table_width + pos / bs];
  if (page < 0) return;
  const int slot = pos % bs;
  if (kind == 1) {
    T* dst = k_cache + (((size_t)page * nkv + (hd - nh)) * bs + slot) * D;
    *reinterpret_cast<Pack8<T>*>(dst + 8 * p) = out_lo;
    *reinterpret_cast<Pack8<T>*>(dst + 8 * p + HALF) = out_hi;
  } else {
    T* dst = v_cache + ((size_t)page * nkv + (hd - nh - nkv)) * D * bs + slot;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      dst[(size_t)(8 * p + j) * bs] = out_lo.v[j];
      dst[(size_t)(8 * p + j + HALF) * bs] = out_hi.v[j];
    }
  }
}

template <typename T>
static bool launch_wide(const T* qkv, const float* q_w, const float* k_w, const float* rope_table, const int* positions,
                        const int* token_item, const int* block_table, int table_width, T* q_out, T* k_cache,
                        T* v_cache, int num_tokens, int nh, int nkv, int d, int bs, float eps, int write_kv, int skip_v,
                        const int* item_start, int num_items, int num_segments, hipStream_t stream) {
  // 8-element accesses need aligned bases (row lengths are multiples of the head size, itself one of 16)
  const uintptr_t align = sizeof(T) * 8 - 1;
  if (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_cache) & align) return false;
  if (((uintptr_t)q_w | (uintptr_t)k_w | (uintptr_t)rope_table) & 15) return false;
  const int heads = write_kv ? (skip_v ? nh + nkv : nh + 2 * nkv) : nh;
  const long long units = (long long)num_tokens * heads;
  // with skip_v the values are written by blocks of the same launch, one per (page segment, kv head)
  const long long value_blocks = skip_v ? (long long)num_segments * nkv : 0;
#define ME_WIDE(LPH)                                                                                                  \
  {                                                                                                                   \
    const long long per_block = 4 * (64 / LPH);                                                                       \
    const long long own = (units + per_block - 1) / per_block, all = own + value_blocks;                              \
    if (all > 0x7fffffffLL) return false;                                                                             \
    qk_norm_rope_scatter_wide_kernel<T, LPH><<<(unsigned)all, 256, 0, stream>>>(                                      \
        qkv, q_w, k_w, rope_table, positions, token_item, block_table, table_width, q_out, k_cache, v_cache,          \
        num_tokens, nh, nkv, bs, eps, write_kv, skip_v, item_start, num_items, (unsigned)own);                        \
    return true;                                                                                                      \
  }
  switch (d) {
    case 16: ME_WIDE(1)
    case 32: ME_WIDE(2)
    case 64: ME_WIDE(4)
    case 128: ME_WIDE(8)
    case 256: ME_WIDE(16)
  }
#undef ME_WIDE
  return false;
}

// One launch where the wide kernel takes the geometry (it writes the values' page segments with blocks of
// its own); else the general kernel, and the page-segment kernel behind it when `tiles`.
template <typename T>
static void launch_qk_scatter(const T* qkv, const float* q_w, const float* k_w, const float* rope_table,
                              const int* positions, const int* token_item, const int* block_table, int table_width,
                              T* q_out, T* k_cache, T* v_cache, int num_tokens, int nh, int nkv, int d, int rd, int bs,
                              float eps, int write_kv, bool wide, bool tiles, int hpb, dim3 grid, const int* item_start,
                              int num_items, int num_segments, hipStream_t stream) {
  if (wide && launch_wide<T>(qkv, q_w, k_w, rope_table, positions, token_item, block_table, table_width, q_out, k_cache,
                             v_cache, num_tokens, nh, nkv, d, bs, eps, write_kv, tiles ? 1 : 0, item_start, num_items,
                             tiles ? num_segments : 0, stream))
    return;
  qk_norm_rope_scatter_kernel<T><<<grid, 256, 0, stream>>>(qkv, q_w, k_w, rope_table, positions, token_item, block_table,
                                                           table_width, q_out, k_cache, v_cache, nh, nkv, d, rd, bs, eps,
                                                           write_kv, hpb, tiles ? 1 : 0);
  if (tiles)
    v_scatter_tiles_kernel<T><<<dim3(num_segments, nkv), 256, 0, stream>>>(qkv, positions, item_start, num_items,
                                                                         block_table, table_width, v_cache, nh, nkv, d, bs);
}

// rope_table: float32 [num_positions, 2, rd / 2] or null; every position of the step must be below
// num_positions (checked by the caller against the engine's length limit).
// item_start / num_items / num_segments: when given (num_segments > 0), the values are written by the
// page-tile kernel; num_segments is the sum over items of (pos0 + qlen - 1)/16 - pos0/16 + 1.
extern "C" int me_qk_norm_rope_scatter(const void* qkv, const float* q_w, const float* k_w, const float* rope_table,
                                       const int* positions, const int* token_item, const int* block_table,
                                       int table_width, void* q_out, void* k_cache, void* v_cache, int num_tokens,
                                       int nh, int nkv, int d, int rd, int bs, float eps, int write_kv, int dtype,
                                       const int* item_start, int num_items, int num_segments, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (d <= 0 || d > ME_MAX_HEAD_DIM || d % 2)
    return me_fail("me_qk_norm_rope_scatter: head_dim=%d must be even and at most %d", d, ME_MAX_HEAD_DIM);
  if (rd < 0 || rd > d || rd % 2) return me_fail("me_qk_norm_rope_scatter: rotary_dim=%d with head_dim=%d", rd, d);
  if (nh <= 0 || nkv <= 0 || bs <= 0 || table_width <= 0)
    return me_fail("me_qk_norm_rope_scatter: nh=%d nkv=%d block_size=%d table_width=%d", nh, nkv, bs, table_width);
  const bool tiles = write_kv && num_segments > 0 && item_start != nullptr && bs % 16 == 0;
  if (tiles && (num_items <= 0 || nkv > 65535)) return me_fail("me_qk_norm_rope_scatter: %d items, %d kv heads", num_items, nkv);
  const int heads_total = write_kv ? (tiles ? nh + nkv : nh + 2 * nkv) : nh;
  // few tokens: spread the heads over many blocks; many tokens: a block per token keeps its table rows hot
  const int hpb = num_tokens >= 512 ? heads_total : 4;
  dim3 grid(num_tokens, (heads_total + hpb - 1) / hpb);
  if (grid.y > 65535) return me_fail("me_qk_norm_rope_scatter: too many heads");
  const bool wide = (rd == d || rope_table == nullptr) && (d & (d - 1)) == 0 && d >= 16 && d <= 256;
  if (dtype == ME_F32)
    launch_qk_scatter<float>((const float*)qkv, q_w, k_w, rope_table, positions, token_item, block_table, table_width,
                             (float*)q_out, (float*)k_cache, (float*)v_cache, num_tokens, nh, nkv, d, rd, bs, eps,
                             write_kv, wide, tiles, hpb, grid, item_start, num_items, num_segments, stream);
  else
    launch_qk_scatter<bf16_t>((const bf16_t*)qkv, q_w, k_w, rope_table, positions, token_item, block_table, table_width,
                              (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, num_tokens, nh, nkv, d, rd, bs, eps,
                              write_kv, wide, tiles, hpb, grid, item_start, num_items, num_segments, stream);
  return me_check_launch("me_qk_norm_rope_scatter");
}
