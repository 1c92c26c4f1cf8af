// Running a step program: the choice of kernel per operation and step size, and the launches.
#include "program.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <mutex>
#include <set>
#include <tuple>

#include "../kernels.h"
#include "choice.h"

int me_fail(const char* fmt, ...);

namespace me {

namespace {

constexpr int kF32 = 0, kBF16 = 1;
constexpr int kDecodeWaves = 1024;  // waves that a decode attention launch aims at (four per compute unit of 256)

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
  // A delta that has added itself to the stream and left the norm behind it half done: bf16(x * w) in the buffer of
  // normed rows and the rows' sums of squares in `ss_blocks` partial sums, for the product behind the norm `carried_w`.
  const float* ss = nullptr;
  int ss_blocks = 0;
  const void* carried_w = nullptr;
  bool any() const { return delta || parts; }
  bool carried() const { return ss != nullptr; }
};

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

// x += a . w^T through the library; false (and nothing done) for sizes it has no algorithm for.
bool library_adds(const void* a, const void* w, float* x, int m, int n, int k, hipStream_t stream) {
  const auto shape = std::make_tuple(n, k, kF32);
  {
    std::lock_guard<std::mutex> hold(g_refused_mutex);
    if (g_refused.count(shape)) return false;
  }
  if (me_gemm_bf16_library_add(a, w, x, m, n, k, stream) == 0) return true;
  std::lock_guard<std::mutex> hold(g_refused_mutex);
  g_refused.insert(shape);
  return false;
}

// (keys per split, number of splits) of a decode launch: enough waves to fill the chip, splits of at least 64
// keys, whole tiles of 16 (rounded to 64 keys, 3 items at a context of 4,096 had 32 splits of 128 keys where 43 of 96
// fit: a step of 3 / 5 / 9 items 1.348 -> 1.293 / 1.501 -> 1.452 / 1.818 -> 1.772 ms, other counts level).
void decode_splits(int items, int kv_units, int max_ctx, int& split_keys, int& num_splits) {
  const int units = std::max(1, items * kv_units);
  const int splits = std::max(1, std::min((kDecodeWaves + units - 1) / units, std::max(max_ctx, 64) / 64));
  split_keys = (max_ctx + splits - 1) / splits;
  split_keys = (split_keys + 15) / 16 * 16;
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
      : prog_(prog), values_(values), s_(s), arena_(arena), fed_tokens_(fed_tokens), stream_(stream), dtype_(prog.dtype()),
        elem_(prog.dtype() == kF32 ? 4 : 2), t_(s.lay.tokens), h_(prog.hidden()) {
    x_ = (float*)arena_.take((size_t)t_ * h_ * 4);
    spare_ = (float*)arena_.take((size_t)t_ * h_ * 4);
    normed_ = arena_.take((size_t)t_ * h_ * elem_);
    for (const Value& v : values) bufs_.push_back(arena_.take((size_t)t_ * v.cols * v.elem));
  }

  RunResult go() {
    const std::vector<Op>& ops = prog_.ops();
    for (size_t at = 0; at < ops.size(); ++at) {
      const Op& op = ops[at];
      next_ = at + 1 < ops.size() ? &ops[at + 1] : nullptr;
      const size_t mark = arena_.used;
      released_to_ = (size_t)-1;
      if (pending_.carried() && op.kind != kOpNormLinear)
        throw Error(kBroken, "a norm was left to a product that does not follow");
      step(op);
      // the logits, the drawn tokens and partial sums that wait for the next norm outlive their operation;
      // an operation that used up waiting partial sums gives their memory back too
      if (op.kind != kOpHead && op.kind != kOpHeadRows && op.kind != kOpSample && op.kind != kOpLinearDelta)
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
      case kOpAdd:
        if (pending_.any())
          ok(me_residual_add(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, t_, h_, dtype_, stream_));
        pending_ = Pending();
        release_parts();
        break;
      case kOpCall:
        call(op);
        break;
      case kOpHeadRows:
        head_rows(op);
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
    if (parts_mark_ != (size_t)-1 && !pending_.parts && !pending_.ss) {
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
    if (pending_.carried()) {  // the add is done and the norm half done: this product multiplies its rows by the rest
      if (op.p[0] != pending_.carried_w) throw Error(kBroken, "a norm was left to the product behind another norm");
      const ProductChoice c = choose_product(dtype_, kRolePlain, t_, rows_of_w, k, gated, dtype_, compute_units(), true);
      if (c.kernel == kProductSmall && !c.gate_after)
        ok(me_gemm_bf16_small_scaled(normed_, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, pending_.ss, pending_.ss_blocks, k,
                                     op.f[0], stream_));
      else if (c.kernel == kProductStream && !c.gate_after)
        ok(me_gemm_bf16_stream_scaled(normed_, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, compute_units(), pending_.ss,
                                      pending_.ss_blocks, k, op.f[0], stream_));
      else
        throw Error(kBroken, "a norm was left to a product whose kernel does not scale its rows");
      pending_ = Pending();
      release_parts();
      return;
    }
    const int pending = pending_.parts ? kPendingParts : pending_.delta ? kPendingTensor : kPendingNone;
    // Where the add and the norm ride on the product the sum goes to the second residual buffer, since other blocks
    // of the kernel still read the first.
    switch (choose_norm_fusion(dtype_, t_, rows_of_w, k, pending, compute_units(), true)) {
      case kNormInStream: {
        const bool adds = pending_.any();
        ok(me_gemm_bf16_stream_norm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, w_norm, op.f[0],
                                    adds ? spare_ : nullptr, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, compute_units(),
                                    stream_));
        if (adds) std::swap(x_, spare_);
        pending_ = Pending();
        release_parts();
        return;
      }
      case kNormInSmall:
        ok(me_gemm_bf16_small(nullptr, x_, pending_.delta, w_norm, op.f[0], pending_.delta ? spare_ : nullptr, op.p[1],
                              bufs_[op.out], t_, n, k, 1, gated, dtype_, 1, stream_));
        if (pending_.delta) std::swap(x_, spare_);
        pending_ = Pending();
        return;
      default:
        add_norm(w_norm, op.f[0], normed_);
        product(normed_, op.p[1], rows_of_w, k, gated, dtype_, bufs_[op.out]);
    }
  }

  // out = x . W^T (gated, the code of an activation: act(gate) * up with W = [gate rows; up rows]), by the kernel
  // that choose_product names.
  void product(const void* x, const void* w, int rows_of_w, int k, int gated, int out_dtype, void* out, int role = kRolePlain,
               int rows = -1) {
    const int m = rows < 0 ? t_ : rows;
    const int n = gated ? rows_of_w / 2 : rows_of_w;
    const ProductChoice c = choose_product(dtype_, role, m, rows_of_w, k, gated, out_dtype, compute_units(), true);
    void* dst = out;
    const int cols = c.gate_after ? rows_of_w : n;
    const int inner_dtype = c.gate_after ? dtype_ : out_dtype;
    if (c.gate_after) dst = arena_.take((size_t)m * rows_of_w * elem_);
    const int epilogue = c.gate_after ? 0 : gated;
    switch (c.kernel) {
      case kProductF32:
        ok(me_gemm_f32((const float*)x, (const float*)w, (float*)dst, m, cols, k, stream_));
        break;
      case kProductSmall:
        ok(me_gemm_bf16_small(x, nullptr, nullptr, nullptr, 0.f, nullptr, w, dst, m, cols, k, 0, epilogue, inner_dtype, 1, stream_));
        break;
      case kProductStream:
        ok(me_gemm_bf16_stream(x, w, dst, m, cols, k, epilogue, c.partial_sums ? kF32 : inner_dtype, c.runs, compute_units(),
                               stream_));
        break;
      case kProductTiled:
        ok(me_gemm_bf16_tiled(x, w, dst, m, cols, k, epilogue, inner_dtype, 0, stream_));
        break;
      default:
        library_product(x, w, dst, m, cols, k, c.partial_sums ? kF32 : inner_dtype, stream_);
    }
    if (c.gate_after) ok(me_swiglu(dst, out, m, n, gated, dtype_, stream_));
  }

  // A product whose result only ever is the pending delta of the residual stream.
  void linear_delta(const Op& op) {
    const int n = (int)op.i[0], k = (int)op.i[1];
    if (n != h_) throw Error(kBadValue, "a delta of the residual stream has the hidden size");
    const void* x = bufs_[op.in];
    pending_ = Pending();
    if (attn_parts_.o) {  // decode attention left its splits to this product
      const AttnParts a = attn_parts_;
      attn_parts_ = AttnParts();
      if (a.value != op.in || k != a.nh * a.d) throw Error(kBroken, "attention left its splits to a product that does not follow");
      const int runs = me_attention_out_product_runs(a.nh);
      parts_mark_ = a.mark;
      float* parts = (float*)arena_.take((size_t)runs * t_ * n * 4);
      ok(me_attention_out_product_bf16(a.o, a.ml, a.splits, op.p[1], parts, t_, a.nh, a.d, n, stream_));
      pending_.parts = parts;
      pending_.num_parts = runs;
      pending_.stride = (long long)t_ * n;
      return;
    }
    if (next_ && next_->kind == kOpNormLinear && next_->i[1] == h_ &&
        choose_carried_norm(dtype_, t_, n, k, (int)next_->i[0], (int)next_->i[2], compute_units(), true)) {
      // x += product in the product's epilogue, which also starts the norm behind it (choice.cpp)
      const int blocks = me_gemm_bf16_stream_carry_blocks(t_, n, k, compute_units());
      parts_mark_ = arena_.used;
      float* ss = (float*)arena_.take((size_t)t_ * blocks * 4);
      ok(me_gemm_bf16_stream_carry(x, op.p[1], x_, normed_, ss, (const float*)next_->p[0], t_, n, k, compute_units(), stream_));
      pending_.ss = ss;
      pending_.ss_blocks = blocks;
      pending_.carried_w = next_->p[0];
      return;
    }
    const ProductChoice c = choose_product(dtype_, kRoleDeltaInto, t_, n, k, 0, dtype_, compute_units(), true);
    if (c.adds_into) {  // x += product, in the library's epilogue: nothing stays pending
      if (library_adds(x, op.p[1], x_, t_, n, k, stream_)) return;
      // (a size the library has no algorithm for: the product as one partial sum, through this folder's kernels)
      parts_mark_ = arena_.used;
      float* sum = (float*)arena_.take((size_t)t_ * n * 4);
      library_product(x, op.p[1], sum, t_, n, k, kF32, stream_);
      pending_.parts = sum;
      pending_.num_parts = 1;
      pending_.stride = (long long)t_ * n;
      return;
    }
    if (c.partial_sums) {  // float32 sums over runs of k (or one whole sum) that wait for the next add-and-norm
      parts_mark_ = arena_.used;
      float* parts = (float*)arena_.take((size_t)c.runs * t_ * n * 4);
      product(x, op.p[1], n, k, 0, kF32, parts, kRoleDelta);
      pending_.parts = parts;
      pending_.num_parts = c.runs;
      pending_.stride = (long long)t_ * n;
      return;
    }
    const size_t mark = arena_.used;
    product(x, op.p[1], n, k, 0, dtype_, bufs_[op.out], kRoleDelta);
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
    const size_t mark = arena_.used;
    auto partials = [&](const SplitPlan& sp, float*& part_o, float*& part_ml) {
      part_o = (float*)arena_.take((size_t)items * nh * sp.num_splits * d * 4);
      part_ml = (float*)arena_.take((size_t)items * nh * sp.num_splits * 2 * 4);
    };
    // A decode step of very few items leaves the splits' partial results to the output projection behind it: no kernel
    // of its own adds them up.
    auto leaves_to_product = [&](const SplitPlan& sp, float* part_o, float* part_ml) {
      if (!(next_ && next_->kind == kOpLinearDelta && next_->in == op.out && next_->i[0] == h_ && next_->i[1] == (int64_t)nh * d &&
            items == t_ && choose_split_sum_in_product(dtype_, items, h_, true) &&
            me_attention_decode_leaves_parts(items, nh, nkv, d, sp.num_splits) &&
            me_attention_out_product_supported(items, nh, d, h_, sp.num_splits)))
        return false;
      attn_parts_.o = part_o;
      attn_parts_.ml = part_ml;
      attn_parts_.splits = sp.num_splits;
      attn_parts_.nh = nh;
      attn_parts_.d = d;
      attn_parts_.value = op.out;
      attn_parts_.mark = mark;
      released_to_ = arena_.used;  // the partial results outlive this operation
      return true;
    };
    const int chunks = (group + 15) / 16;
    if (s_.decode_only && (long long)width * bs < s_.max_ctx && mfma)
      throw Error(kBadValue, "the block table cannot hold the step's longest context");
    if (dtype_ == kBF16 && s_.decode_only && me_attention_decode_fused_supported(d, bs, rd, group)) {
      // one new token per item: norm, rotary, page write and attention in one launch
      const SplitPlan sp = split_plan(items, nkv * chunks, s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float *part_o, *part_ml;
      partials(sp, part_o, part_ml);
      if (leaves_to_product(sp, part_o, part_ml)) out = nullptr;
      ok(me_attention_decode_fused_bf16(qkv, q_w, k_w, rope, rd, eps, owns ? 1 : 0, kc, vc, idx(s_.lay.item_ctx), table, width, out,
                                        part_o, part_ml, items, nh, nkv, d, bs, window, scale, sp.split_keys, sp.num_splits,
                                        s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves, idx(s_.lay.live_items) + 1, stream_));
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
      if (leaves_to_product(sp, part_o, part_ml)) out = nullptr;
      ok(me_attention_decode_bf16(q, kc, vc, idx(s_.lay.item_ctx), table, width, out, part_o, part_ml, items, nh, nkv, d, bs, window,
                                  scale, sp.split_keys, sp.num_splits, s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves,
                                  idx(s_.lay.live_items) + 1, stream_));
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
    const int rows = s_.lay.rows;
    result_.rows = rows;
    if (rows == 0) {
      pending_ = Pending();
      return;
    }
    void* picked = arena_.take((size_t)rows * h_ * elem_);
    ok(me_add_rmsnorm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, (const float*)op.p[0], picked,
                      idx(s_.lay.want_rows), rows, h_, op.f[0], 0, dtype_, stream_));
    pending_ = Pending();
    logits_of(picked, op);
  }

  // The head behind a final norm that a part computed itself: the value's first rows are the normed wanted rows.
  void head_rows(const Op& op) {
    result_.rows = s_.lay.rows;
    if (s_.lay.rows == 0) return;
    logits_of(bufs_[op.in], op);
  }

  void logits_of(const void* picked, const Op& op) {
    const int rows = s_.lay.rows, vocab = prog_.vocab();
    float* logits = (float*)arena_.take((size_t)rows * vocab * 4);
    product(picked, op.p[1], vocab, h_, 0, kF32, logits, kRoleHead, rows);
    if (op.f[1] != 1.f) ok(me_scale_f32(logits, op.f[1], (long long)rows * vocab, stream_));
    result_.logits = logits;
  }

  // A part that brings its own code: it reads and writes values of the step and launches on the step's stream.
  void call(const Op& op) {
    CallFrame f{};
    f.context = (void*)op.p[1];
    f.in = op.in >= 0 ? bufs_[op.in] : nullptr;
    f.out = op.out >= 0 ? bufs_[op.out] : nullptr;
    f.x = x_;
    f.in_cols = op.in >= 0 ? values_[op.in].cols : 0;
    f.out_cols = op.out >= 0 ? values_[op.out].cols : 0;
    f.in_elem = op.in >= 0 ? values_[op.in].elem : 0;
    f.out_elem = op.out >= 0 ? values_[op.out].elem : 0;
    f.tokens = t_;
    f.rows = s_.lay.rows;
    f.stream = stream_;
    if (!op.p[0]) throw Error(kBadValue, "a called part needs its function");
    if (((CallFn)op.p[0])(&f) != 0) throw Error(kBadState, "a part's own code failed in a step");
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
  const std::vector<Value>& values_;
  const StepView& s_;
  Arena& arena_;
  int32_t* fed_tokens_;
  hipStream_t stream_;
  const int dtype_, elem_, t_, h_;
  float *x_, *spare_;
  void* normed_;
  std::vector<void*> bufs_;
  Pending pending_;
  struct AttnParts {  // what a decode attention left for the output projection behind it
    float *o = nullptr, *ml = nullptr;
    int splits = 0, nh = 0, d = 0, value = -1;
    size_t mark = 0;
  } attn_parts_;
  const Op* next_ = nullptr;  // the operation behind the one being run
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
      need = std::max<size_t>((size_t)kMaxRuns * std::min<int64_t>(tokens, kSmallMaxRows), (size_t)tokens) * op.i[0] * 4 + pad;
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
  return fixed + 2 * scratch + tail + std::max<size_t>((size_t)kMaxRuns * kSmallMaxRows, (size_t)tokens) * hidden_ * 4 + (1 << 16);
}

}  // namespace me

// A plain bfloat16 product through the GEMM library, with this folder's kernels where the library has no algorithm:
// what the step program calls for a product that choose_product leaves to the library, for callers outside it.
extern "C" int me_gemm_bf16_any(const void* x, const void* w, void* out, int m, int n, int k, int out_dtype, hipStream_t stream) {
  try {
    me::library_product(x, w, out, m, n, k, out_dtype, stream);
    return 0;
  } catch (const std::exception& e) {
    return me_fail("%s", e.what());
  }
}
