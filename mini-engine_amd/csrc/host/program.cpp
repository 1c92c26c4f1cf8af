// Running a step program: the choice of kernel per operation and step size, and the launches.
#include "program.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <mutex>
#include <set>
#include <tuple>

#include "../kernels.h"

namespace me {

namespace {

constexpr int kF32 = 0, kBF16 = 1;
constexpr int kSmallMaxRows = 64;   // what the small matrix-core kernel accepts
constexpr int kSmallFastRows = 16;  // up to here it beats the GEMM library on every shape, the norm as its prologue too
constexpr int kNormStreamRows = 2;   // up to here the add-and-norm is the prologue of the weight-streaming kernel
constexpr int kTiledMinRows = 256;
constexpr int kStreamWholeRows = 32;   // up to here the weight-streaming kernel serves wide plain products whose blocks fill whole
                                       // rounds (gated ones up to 64)
constexpr int kStreamGroupRows = 256;  // what the weight-streaming kernel accepts, in groups of 64 rows
constexpr int kTiledMaxK = 3072;  // gate/up with the SwiGLU as the tiled kernel's epilogue against the library's product and a
                                  // SwiGLU kernel: at k = 1,024 (3,072 columns) 15-62 us against 21-67 for 512 to 4,096 rows; at
                                  // k = 4,096 (12,288 columns) 95-729 against 89-640; at k = 5,120 (25,600) 345-1,973 against
                                  // 293-1,767: the longer k is, the less a pass over the output weighs against the product
constexpr int kHeadStreamRows = 32;  // the head's logits (float32) come from the weight-streaming kernel up to here: at 151,936
                                     // rows of 1,024 / 4,096 / 5,120 it takes 62-75 / 245-272 / 291-341 us at 8 to 32 rows,
                                     // the library 62-79 / 260-276 / 319-362; from 48 rows on the library is ahead
constexpr int kDecodeWaves = 1024;  // waves that a decode attention launch aims at (four per compute unit of 256)
constexpr int64_t kStreamMinElements = 8ll << 20;  // weights from 16 MiB on: streaming them is the product's time
constexpr int64_t kStreamMaxBytes = 1ll << 31;     // what the weight-streaming kernel addresses

void ok(int code) {
  if (code) throw Error(kBadState, me_last_error());
}

struct Arena {
  char* base;
  size_t size, used = 0;
  void* take(size_t bytes) {
    const size_t at = (used + 255) & ~(size_t)255;
    if (at + bytes > size)
      throw Error(kBadState, "the step needs more workspace than the program's arena holds (" + std::to_string(at + bytes) +
                                 " of " + std::to_string(size) + " bytes)");
    used = at + bytes;
    return base + at;
  }
};

struct Pending {
  const void* delta = nullptr;
  const float* parts = nullptr;
  int num_parts = 0;
  long long stride = 0;
  bool any() const { return delta || parts; }
};

// Which kernel serves a bfloat16 product of m rows (measured on the layer sizes of a 0.6B, an 8B and a 32B model):
//   up to 16 rows, weights below 16 MiB: the small matrix-core kernel; the residual add and the norm are its prologue
//     where the delta in front is a tensor (a product whose k was not cut);
//   17 to 64 rows, weights below 16 MiB: the weight-streaming kernel (qkv 5.0-6.7 us, gate/up with SwiGLU 6.6-9.3
//     against 5.8-7.7 and 7.5-10.3 with the small kernel, 8.2-8.6 and 14.4-14.7 with the library and a SwiGLU kernel);
//   a delta of the residual stream, at any row count up to 64: the weight-streaming kernel with k cut into runs, so
//     that every compute unit streams a part of the weight (1,024 columns, 1 to 16 rows: 3.5 and 4.3 us against 4.7-6.1
//     and 5.8-7.8 with the small kernel; 17 to 64 rows: 3.9-5.3 against 7.9-16 and 7.6-9.8). The add-and-norm behind
//     it, a kernel of its own (2.9 us), adds the partial sums up; as the prologue of the next product, where every
//     block would read them, they cost more at every row count (one row: 853 -> 820 tokens/s);
//   everything else: the GEMM library, as the reference hands every projection to one.
bool small_serves(int m, int k) { return k % 8 == 0 && m <= kSmallFastRows; }

// Whether a product of up to 64 rows is bound by streaming its weight: the layers of wide models. Their
// deltas go to the weight-streaming kernel with k cut into runs (measured at 4,096 and 5,120 columns, k of 4,096
// to 25,600: 8.7-29 us and 21-80 us against 9.4-65 and 27-245 with the small kernel, 10-38 and 20-156 with
// the library); their other products go to the same kernel up to 16 rows (qkv and gate/up 14.7-43 and 24-117 us
// against 15-51 and 26-139 with the small kernel) and to the library from 17 to 64 rows (qkv 15-33 us against
// 21-56 with the streaming kernel, whose time grows with the rows). The norm before such a product is a kernel
// of its own: the partial sums it adds up are read once, not by every block of a product.
bool weight_bound(int m, int rows_of_w, int k) {
  const int64_t elements = (int64_t)rows_of_w * k;
  return m <= kSmallMaxRows && k % 8 == 0 && elements >= kStreamMinElements && elements * 2 < kStreamMaxBytes;
}

// What the weight-streaming kernel takes at all.
bool streams(int m, int rows_of_w, int k) {
  return m <= kSmallMaxRows && k % 8 == 0 && (int64_t)rows_of_w * k * 2 < kStreamMaxBytes;
}

int compute_units();

// Whether the weight-streaming kernel serves a wide product of 17 to 32 rows instead of the library: where its blocks fill
// whole rounds of the compute units (at least 15/16 of them) and the rows of the weight are a multiple of 4 KiB apart, which
// costs the library's kernels a quarter of their rate (2 x 12,288 x 4,096 with SwiGLU: 52 us, with k = 4,224 42; the streaming
// kernel 46 and 39). Measured at 17 and 32 rows: 2 x 12,288 x 4,096 46 us against 52; 6,144 x 4,096 14.1 and 15.6 against
// 16.3 and 15.9; 2 x 28,672 x 8,192 182 against 191 and 194; a decode step of the 8B shape at batch 20 to 32 4-5% shorter.
// Where the blocks do not fill their rounds the library is ahead (10,240 x 5,120 on 160 blocks: 32 and 35 against 27 and 30;
// 5,120 x 4,096: 13.4 against 12.0), with other k it is ahead or level (2 x 25,600 x 5,120: 101 and 105 against 99 and 102),
// and from 33 rows on it is ahead on as many shapes as not.
// With each block's walk over k starting at a step of its own (what the kernel does for such k) the gated products stay ahead
// up to 64 rows: 2 x 12,288 x 4,096 38-43 us against 48-50 at 17 to 64 rows, 2 x 14,336 x 4,096 45-48 against 58-65, 2 x 28,672
// x 8,192 169-180 against 192-216; the plain 6,144 x 4,096 up to 32 (14.3 and 15.1 against 15.1 and 15.4; 19.4 against 17.6 at 64).
bool stream_serves_mid_rows(int m, int n, int k, bool gated) {
  if (k % 2048 || m > (gated ? kSmallMaxRows : kStreamWholeRows)) return false;
  int plan[3] = {0, 0, 0};
  me_gemm_bf16_stream_plan(m, n, k, gated ? 1 : 0, 1, compute_units(), plan);
  const long long cus = compute_units(), rounds = (plan[2] + cus - 1) / cus;
  return (long long)plan[2] * 16 >= rounds * cus * 15;
}

int compute_units() {
  static int units = 0;
  if (!units) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      units = n;
    else
      units = 256;
  }
  return units;
}

std::mutex g_refused_mutex;
std::set<std::tuple<int, int, int>> g_refused;  // (N, K, output type) the GEMM library has no algorithm for

// A plain bfloat16 product of many rows: the GEMM library, as the reference hands every projection to one;
// sizes it has no algorithm for go to the kernels of this folder.
void library_product(const void* x, const void* w, void* out, int m, int n, int k, int out_dtype, hipStream_t stream) {
  const auto shape = std::make_tuple(n, k, out_dtype);
  bool refused;
  {
    std::lock_guard<std::mutex> hold(g_refused_mutex);
    refused = g_refused.count(shape) != 0;
  }
  if (!refused) {
    if (me_gemm_bf16_library(x, w, out, m, n, k, out_dtype, stream) == 0) return;
    std::lock_guard<std::mutex> hold(g_refused_mutex);
    g_refused.insert(shape);
  }
  if (k % 64 == 0 && m > kSmallMaxRows && (((uintptr_t)x | (uintptr_t)w) & 15) == 0) {  // the tiled matrix-core kernel of this folder
    ok(me_gemm_bf16_tiled(x, w, out, m, n, k, 0, out_dtype, 0, stream));
    return;
  }
  if (k % 8 == 0) {  // slices of 64 rows through the small matrix-core kernel
    const size_t out_elem = out_dtype == kF32 ? 4 : 2;
    for (int lo = 0; lo < m; lo += kSmallMaxRows) {
      const int rows = std::min(kSmallMaxRows, m - lo);
      ok(me_gemm_bf16_small((const char*)x + (size_t)lo * k * 2, nullptr, nullptr, nullptr, 0.f, nullptr, w,
                            (char*)out + (size_t)lo * n * out_elem, rows, n, k, 0, 0, out_dtype, 1, stream));
    }
    return;
  }
  ok(me_gemm_plain(x, w, out, m, n, k, kBF16, out_dtype, stream));
}

// (keys per split, number of splits) of a decode launch: enough waves to fill the chip, splits of at least 64
// keys, boundaries at multiples of 64.
void decode_splits(int items, int kv_units, int max_ctx, int& split_keys, int& num_splits) {
  const int units = std::max(1, items * kv_units);
  const int splits = std::max(1, std::min((kDecodeWaves + units - 1) / units, std::max(max_ctx, 64) / 64));
  split_keys = (max_ctx + splits - 1) / splits;
  split_keys = (split_keys + 63) / 64 * 64;
  num_splits = (max_ctx + split_keys - 1) / split_keys;
}

struct SplitPlan {
  int split_keys, num_splits, full_splits;
  const int* live;
};

// The grid of a launch that a graph replays with fewer live items than it holds is laid out for the fewest it
// will ever see; the kernel reads the count of live items and takes as many of the grid's splits as they need.
SplitPlan split_plan(int items, int kv_units, int max_ctx, int least_live, const int* live_count) {
  int keys, full;
  decode_splits(items, kv_units, max_ctx, keys, full);
  if (!live_count || least_live >= items) return {keys, full, full, nullptr};
  int splits;
  decode_splits(std::max(1, least_live), kv_units, max_ctx, keys, splits);
  return {keys, splits, std::min(full, splits), live_count};
}

class Run {
 public:
  Run(const Program& prog, const std::vector<Value>& values, const StepView& s, Arena& arena, int32_t* fed_tokens,
      hipStream_t stream)
      : prog_(prog), s_(s), arena_(arena), fed_tokens_(fed_tokens), stream_(stream), dtype_(prog.dtype()),
        elem_(prog.dtype() == kF32 ? 4 : 2), t_(s.lay.tokens), h_(prog.hidden()) {
    x_ = (float*)arena_.take((size_t)t_ * h_ * 4);
    spare_ = (float*)arena_.take((size_t)t_ * h_ * 4);
    normed_ = arena_.take((size_t)t_ * h_ * elem_);
    for (const Value& v : values) bufs_.push_back(arena_.take((size_t)t_ * v.cols * v.elem));
  }

  RunResult go() {
    for (const Op& op : prog_.ops()) {
      const size_t mark = arena_.used;
      released_to_ = (size_t)-1;
      step(op);
      // the logits, the drawn tokens and partial sums that wait for the next norm outlive their operation;
      // an operation that used up waiting partial sums gives their memory back too
      if (op.kind != kOpHead && op.kind != kOpSample && op.kind != kOpLinearDelta)
        arena_.used = released_to_ != (size_t)-1 ? released_to_ : mark;
    }
    return result_;
  }

 private:
  const int32_t* idx(int offset) const { return s_.dev + offset; }

  void step(const Op& op) {
    switch (op.kind) {
      case kOpEmbed: {
        const int table_dtype = dtype_;
        if (s_.fed && fed_tokens_)
          ok(me_embed_fed(x_, op.p[0], idx(s_.lay.token_ids), idx(s_.lay.token_source), fed_tokens_, t_, h_, prog_.vocab(),
                          op.f[0], table_dtype, stream_));
        else
          ok(me_embed(x_, op.p[0], idx(s_.lay.token_ids), t_, h_, prog_.vocab(), op.f[0], table_dtype, stream_));
        pending_ = Pending();
        break;
      }
      case kOpNormLinear:
        norm_linear(op);
        break;
      case kOpNorm:
        add_norm((const float*)op.p[0], op.f[0], bufs_[op.out]);
        break;
      case kOpLinear:
        product(bufs_[op.in], op.p[1], (int)op.i[0], (int)op.i[1], (int)op.i[2], dtype_, bufs_[op.out]);
        break;
      case kOpLinearDelta:
        linear_delta(op);
        break;
      case kOpDelta:
        pending_ = Pending();
        pending_.delta = bufs_[op.in];
        break;
      case kOpAttention:
        attention(op);
        break;
      case kOpHead:
        head(op);
        break;
      case kOpSample:
        sample();
        break;
      default:
        throw Error(kBadValue, "unknown operation in a step program");
    }
  }

  // x += pending; out = rmsnorm(x) * w, as a kernel of its own.
  void add_norm(const float* w, float eps, void* out) {
    ok(me_add_rmsnorm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, w, out, nullptr, t_, h_, eps, 1,
                      dtype_, stream_));
    pending_ = Pending();
    release_parts();
  }

  void release_parts() {
    if (parts_mark_ != (size_t)-1 && !pending_.parts) {
      arena_.used = released_to_ = parts_mark_;
      parts_mark_ = (size_t)-1;
    }
  }

  void norm_linear(const Op& op) {
    const float* w_norm = (const float*)op.p[0];
    const int rows_of_w = (int)op.i[0], k = (int)op.i[1];
    const int gated = (int)op.i[2];  // 0, or the code of the gate's activation
    if (k != h_) throw Error(kBadValue, "a product behind a norm reads the hidden size");
    const int n = gated ? rows_of_w / 2 : rows_of_w;
    // Decode-sized steps: the residual add and the norm are the product's prologue; the sum goes to the second
    // residual buffer, since other blocks of the kernel still read the first.
    // A row or two: the weight-streaming kernel adds and norms the rows itself while its first weights are on their
    // way, whatever the delta is (one row: 857 -> 967 tokens/s, two: 1,605 -> 1,700; from four rows on every block's
    // reads of the partial sums cost more than the launch they save: 2,749 -> 2,668).
    if (dtype_ == kBF16 && t_ <= kNormStreamRows && me_gemm_bf16_stream_norm_fits(t_, k) && streams(t_, rows_of_w, k)) {
      const bool adds = pending_.any();
      ok(me_gemm_bf16_stream_norm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, w_norm, op.f[0],
                                  adds ? spare_ : nullptr, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, compute_units(), stream_));
      if (adds) std::swap(x_, spare_);
      pending_ = Pending();
      release_parts();
      return;
    }
    // Up to 16 rows with nothing, or a tensor, to add (the first layer's norm; parts of other kinds): the small kernel's
    // prologue.
    if (dtype_ == kBF16 && t_ <= kSmallFastRows && k % 8 == 0 && !pending_.parts && !weight_bound(t_, rows_of_w, k)) {
      ok(me_gemm_bf16_small(nullptr, x_, pending_.delta, w_norm, op.f[0], pending_.delta ? spare_ : nullptr, op.p[1],
                            bufs_[op.out], t_, n, k, 1, gated, dtype_, 1, stream_));
      if (pending_.delta) std::swap(x_, spare_);
      pending_ = Pending();
      return;
    }
    add_norm(w_norm, op.f[0], normed_);
    product(normed_, op.p[1], rows_of_w, k, gated, dtype_, bufs_[op.out]);
  }

  // out = x . W^T (gated, the code of an activation: act(gate) * up with W = [gate rows; up rows]).
  void product(const void* x, const void* w, int rows_of_w, int k, int gated, int out_dtype, void* out) {
    const int m = t_rows_;
    const int n = gated ? rows_of_w / 2 : rows_of_w;
    if (dtype_ == kF32) {  // a true 32-bit product, additions in ascending k whatever the rows
      if (!gated) {
        ok(me_gemm_f32((const float*)x, (const float*)w, (float*)out, m, n, k, stream_));
        return;
      }
      float* both = (float*)arena_.take((size_t)m * rows_of_w * 4);
      ok(me_gemm_f32((const float*)x, (const float*)w, both, m, rows_of_w, k, stream_));
      ok(me_swiglu(both, out, m, n, gated, kF32, stream_));
      return;
    }
    const bool heavy = weight_bound(m, rows_of_w, k);
    if (heavy && m <= kSmallFastRows && (out_dtype == kBF16 || !gated)) {  // up to 16 rows it is ahead of the library too
      ok(me_gemm_bf16_stream(x, w, out, m, n, k, gated, out_dtype, 1, compute_units(), stream_));
      return;
    }
    if (heavy && (out_dtype == kBF16 || !gated) && stream_serves_mid_rows(m, n, k, gated != 0)) {
      ok(me_gemm_bf16_stream(x, w, out, m, n, k, gated, out_dtype, 1, compute_units(), stream_));
      return;
    }
    if (!heavy && m > kSmallFastRows && streams(m, rows_of_w, k) && (out_dtype == kBF16 || !gated)) {
      ok(me_gemm_bf16_stream(x, w, out, m, n, k, gated, out_dtype, 1, compute_units(), stream_));
      return;
    }
    if (!heavy && small_serves(m, k)) {
      ok(me_gemm_bf16_small(x, nullptr, nullptr, nullptr, 0.f, nullptr, w, out, m, n, k, 0, gated, out_dtype, 1, stream_));
      return;
    }
    if (gated && m <= kStreamGroupRows && k % 8 == 0 && (int64_t)rows_of_w * k < kStreamMinElements && out_dtype == kBF16) {
      // 65 to 256 rows of a small gated weight: the weight-streaming kernel, its blocks once per group of 64 rows (2 x 3,072 x
      // 1,024: 10.7-13.1 us against 15.5-19.1 with the library and a SwiGLU kernel, 16 with the tiled kernel; the plain
      // products of that size are no faster than the library's: 9.2 against 8.8-9.2, 7.8 against 7.6-8.3)
      ok(me_gemm_bf16_stream(x, w, out, m, n, k, gated, out_dtype, 1, compute_units(), stream_));
      return;
    }
    if (gated) {
      if (m >= kTiledMinRows && k % 64 == 0 && k <= kTiledMaxK && out_dtype == kBF16) {  // ahead of the library product + SwiGLU kernel
        ok(me_gemm_bf16_tiled(x, w, out, m, n, k, gated, out_dtype, 0, stream_));
        return;
      }
      void* both = arena_.take((size_t)m * rows_of_w * 2);
      library_product(x, w, both, m, rows_of_w, k, kBF16, stream_);
      ok(me_swiglu(both, out, m, n, gated, kBF16, stream_));
      return;
    }
    library_product(x, w, out, m, n, k, out_dtype, stream_);
  }

  // A product whose result only ever is the pending delta of the residual stream.
  void linear_delta(const Op& op) {
    const int n = (int)op.i[0], k = (int)op.i[1];
    if (n != h_) throw Error(kBadValue, "a delta of the residual stream has the hidden size");
    const void* x = bufs_[op.in];
    pending_ = Pending();
    if (dtype_ == kBF16 && streams(t_, n, k)) {
      // float32 partial sums over runs of k (one run for short k): the next add-and-norm adds them up, and the delta is
      // never rounded to bfloat16 on its way into the float32 residual stream
      const int splits = me_gemm_bf16_stream_splits(t_, n, k, compute_units());
      parts_mark_ = arena_.used;
      float* parts = (float*)arena_.take((size_t)splits * t_ * n * 4);
      ok(me_gemm_bf16_stream(x, op.p[1], parts, t_, n, k, 0, kF32, splits, compute_units(), stream_));
      pending_.parts = parts;
      pending_.num_parts = splits;
      pending_.stride = (long long)t_ * n;
      return;
    }
    if (dtype_ == kBF16) {
      // more rows: the library's product with a float32 result, which stands as one partial sum: the delta is never
      // rounded to bfloat16 on its way into the float32 residual stream
      parts_mark_ = arena_.used;
      float* sum = (float*)arena_.take((size_t)t_ * n * 4);
      library_product(x, op.p[1], sum, t_, n, k, kF32, stream_);
      pending_.parts = sum;
      pending_.num_parts = 1;
      pending_.stride = (long long)t_ * n;
      return;
    }
    const size_t mark = arena_.used;
    product(x, op.p[1], n, k, 0, dtype_, bufs_[op.out]);
    arena_.used = mark;
    pending_.delta = bufs_[op.out];
  }

  void attention(const Op& op) {
    const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], rd = (int)op.i[3], bs = (int)op.i[4];
    const int window = (int)op.i[5], g = (int)op.i[7];
    const bool owns = op.i[6] != 0;
    const float eps = op.f[0], scale = op.f[1];
    const float* q_w = (const float*)op.p[0];
    const float* k_w = owns ? (const float*)op.p[1] : nullptr;
    const float* rope = (const float*)op.p[2];
    void *kc = (void*)op.p[3], *vc = (void*)op.p[4];
    if (g < 0 || g >= (int)s_.lay.widths.size()) throw Error(kBadValue, "an attention layer names a cache group the step lacks");
    const int32_t* table = idx(s_.lay.tables[g]);
    const int width = s_.lay.widths[g], items = s_.lay.items, group = nh / nkv;
    if (rope && op.i[8] < s_.max_ctx)
      throw Error(kBadValue, "the rotary table covers " + std::to_string(op.i[8]) + " positions, the step may reach " +
                                 std::to_string(s_.max_ctx));
    void* out = bufs_[op.out];
    const void* qkv = bufs_[op.in];
    const bool mfma = dtype_ == kBF16 && me_attention_mfma_supported(d, bs) && group <= 16;
    auto partials = [&](const SplitPlan& sp, float*& part_o, float*& part_ml) {
      part_o = (float*)arena_.take((size_t)items * nh * sp.num_splits * d * 4);
      part_ml = (float*)arena_.take((size_t)items * nh * sp.num_splits * 2 * 4);
    };
    const int chunks = (group + 15) / 16;
    if (s_.decode_only && (long long)width * bs < s_.max_ctx && mfma)
      throw Error(kBadValue, "the block table cannot hold the step's longest context");
    if (dtype_ == kBF16 && s_.decode_only && me_attention_decode_fused_supported(d, bs, rd, group)) {
      // one new token per item: norm, rotary, page write and attention in one launch
      const SplitPlan sp = split_plan(items, nkv * chunks, s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float *part_o, *part_ml;
      partials(sp, part_o, part_ml);
      ok(me_attention_decode_fused_bf16(qkv, q_w, k_w, rope, rd, eps, owns ? 1 : 0, kc, vc, idx(s_.lay.item_ctx), table, width, out,
                                        part_o, part_ml, items, nh, nkv, d, bs, window, scale, sp.split_keys, sp.num_splits,
                                        s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves, stream_));
      return;
    }
    void* q = arena_.take((size_t)t_ * nh * d * elem_);
    int segments = 0, seg_items = 0;
    if (owns && t_ >= 64) {  // many tokens: the values are written a page segment (a transposed tile) at a time
      seg_items = items;
      for (int i = 0; i < items; ++i) segments += (s_.starts[i] + s_.qlens[i] - 1) / 16 - s_.starts[i] / 16 + 1;
    }
    ok(me_qk_norm_rope_scatter(qkv, q_w, k_w, rope, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, q, kc, vc, t_, nh,
                               nkv, d, rd, bs, eps, owns ? 1 : 0, dtype_, segments ? idx(s_.lay.item_start) : nullptr, seg_items,
                               segments, stream_));
    if (mfma && s_.decode_only) {
      const SplitPlan sp = split_plan(items, nkv * chunks, s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float *part_o, *part_ml;
      partials(sp, part_o, part_ml);
      ok(me_attention_decode_bf16(q, kc, vc, idx(s_.lay.item_ctx), table, width, out, part_o, part_ml, items, nh, nkv, d, bs, window,
                                  scale, sp.split_keys, sp.num_splits, s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves,
                                  stream_));
      return;
    }
    if (mfma) {
      auto it = s_.plans.find({nh, nkv, d, window});
      if (it == s_.plans.end()) throw Error(kBroken, "the step has no work list for a prefill attention layer");
      const StepView::Plan& p = it->second;
      float *part_o = nullptr, *part_ml = nullptr;
      if (p.max_chunks > 1) {
        part_o = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * d * 4);
        part_ml = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * 2 * 4);
      }
      ok(me_attention_prefill_bf16(q, kc, vc, items, table, width, out, idx(p.work), idx(p.bundle_first), p.bundles, part_o, part_ml,
                                   p.token_chunks >= 0 ? idx(p.token_chunks) : nullptr, p.max_chunks, t_, nh, nkv, d, bs, window,
                                   scale, p.columns, stream_));
      return;
    }
    ok(me_attention_general(q, kc, vc, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, out, t_, nh, nkv, d, bs, window,
                            scale, dtype_, items, stream_));
  }

  // Rows are selected before the final norm, as the reference does (model.py:186); logits are float32.
  void head(const Op& op) {
    const int rows = s_.lay.rows, vocab = prog_.vocab();
    result_.rows = rows;
    if (rows == 0) {
      pending_ = Pending();
      return;
    }
    void* picked = arena_.take((size_t)rows * h_ * elem_);
    ok(me_add_rmsnorm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, (const float*)op.p[0], picked,
                      idx(s_.lay.want_rows), rows, h_, op.f[0], 0, dtype_, stream_));
    pending_ = Pending();
    float* logits = (float*)arena_.take((size_t)rows * vocab * 4);
    if (dtype_ == kF32)
      ok(me_gemm_f32((const float*)picked, (const float*)op.p[1], logits, rows, vocab, h_, stream_));
    else if (rows > 2 && rows <= kHeadStreamRows && weight_bound(rows, vocab, h_))  // ahead of the small kernel and the library
      ok(me_gemm_bf16_stream(picked, op.p[1], logits, rows, vocab, h_, 0, kF32, 1, compute_units(), stream_));
    else if (rows <= kSmallFastRows && h_ % 8 == 0)
      ok(me_gemm_bf16_small(picked, nullptr, nullptr, nullptr, 0.f, nullptr, op.p[1], logits, rows, vocab, h_, 0, 0, kF32, 1, stream_));
    else
      library_product(picked, op.p[1], logits, rows, vocab, h_, kF32, stream_);
    if (op.f[1] != 1.f) ok(me_scale_f32(logits, op.f[1], (long long)rows * vocab, stream_));
    result_.logits = logits;
  }

  void sample() {
    const int rows = s_.lay.rows;
    if (rows == 0 || !result_.logits) return;
    int32_t* drawn = fed_tokens_ ? fed_tokens_ : (int32_t*)arena_.take((size_t)rows * 4);
    void* ws = arena_.take((size_t)rows * me_sample_chunks(prog_.vocab()) * 8);
    ok(me_sample(result_.logits, rows, prog_.vocab(), (const float*)idx(s_.lay.temperatures),
                 (const uint64_t*)idx(s_.lay.sample_keys), drawn, ws, stream_));
    result_.drawn = drawn;
  }

  const Program& prog_;
  const StepView& s_;
  Arena& arena_;
  int32_t* fed_tokens_;
  hipStream_t stream_;
  const int dtype_, elem_, t_, h_;
  const int& t_rows_ = t_;
  float *x_, *spare_;
  void* normed_;
  std::vector<void*> bufs_;
  Pending pending_;
  size_t parts_mark_ = (size_t)-1, released_to_ = (size_t)-1;
  RunResult result_;
};

}  // namespace

RunResult Program::run(const StepView& s, char* arena, size_t arena_bytes, int32_t* fed_tokens, hipStream_t stream) const {
  Arena a{arena, arena_bytes};
  Run run(*this, values_, s, a, fed_tokens, stream);
  return run.go();
}

std::vector<std::vector<int>> Program::prefill_geometries() const {
  std::vector<std::vector<int>> out;
  if (dtype_ != kBF16) return out;
  for (const Op& op : ops_) {
    if (op.kind != kOpAttention) continue;
    const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], bs = (int)op.i[4], window = (int)op.i[5];
    if (!me_attention_mfma_supported(d, bs) || nh / nkv > 16) continue;
    std::vector<int> key = {nh, nkv, d, window};
    if (std::find(out.begin(), out.end(), key) == out.end()) out.push_back(key);
  }
  return out;
}

size_t Program::arena_need(int64_t tokens, int64_t items, int64_t rows, int64_t max_ctx) const {
  const size_t elem = dtype_ == kF32 ? 4 : 2;
  const size_t pad = 256;
  size_t fixed = 2 * ((size_t)tokens * hidden_ * 4 + pad) + (size_t)tokens * hidden_ * elem + pad;
  for (const Value& v : values_) fixed += (size_t)tokens * v.cols * v.elem + pad;
  size_t scratch = 0;
  for (const Op& op : ops_) {
    size_t need = 0;
    if (op.kind == kOpNormLinear || op.kind == kOpLinear) need = (size_t)tokens * op.i[0] * 4 + pad;
    if (op.kind == kOpLinearDelta)  // up to 16 partial sums of up to 64 rows, or one float32 result of all rows
      need = std::max<size_t>((size_t)16 * std::min<int64_t>(tokens, kSmallMaxRows), (size_t)tokens) * op.i[0] * 4 + pad;
    if (op.kind == kOpAttention) {
      const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2];
      const int chunks = (nh / nkv + 15) / 16;
      size_t most = 0;  // items x splits at its largest over the batch sizes a launch may hold
      for (int64_t b = 1; b <= items; ++b) {
        int keys, splits;
        decode_splits((int)std::max<int64_t>(1, (b + 1) / 2), nkv * chunks, (int)max_ctx, keys, splits);
        most = std::max(most, (size_t)b * splits);
      }
      const size_t decode = most * nh * (d + 2) * 4 + 2 * pad;
      const size_t prefill = (size_t)(256ll << 20) + (size_t)(256ll << 20) * 2 / d + (size_t)tokens * nh * 8 + 2 * pad;
      need = (size_t)tokens * nh * d * elem + pad + std::max(decode, tokens > items ? prefill : (size_t)0);
    }
    scratch = std::max(scratch, need);
  }
  const size_t tail = (size_t)rows * hidden_ * elem + (size_t)rows * vocab_ * 4 + (size_t)rows * 4 +
                      (size_t)rows * me_sample_chunks(vocab_) * 8 + 4 * pad;
  // partial sums of the last delta wait beside the head's buffers
  return fixed + 2 * scratch + tail + std::max<size_t>((size_t)16 * kSmallMaxRows, (size_t)tokens) * hidden_ * 4 + (1 << 16);
}

}  // namespace me
