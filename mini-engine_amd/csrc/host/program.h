// The native step program: a model's forward pass as a list of operations that C++ runs from one
// call, so that a step costs the host one call, not one per kernel. The Python parts write their
// operations into it once, when the model is built (each part knows what it computes, none knows the
// model it is in); which kernel serves an operation is decided per step from the step's size.
//
// State that the operations share: the residual stream x (float32 [tokens, hidden]) in one of two
// buffers, and a pending delta (a part's output that the next norm adds to x while it norms): nothing,
// a buffer in the compute dtype, partial sums over runs of k that the add sums up, or, where the delta's
// product has added itself to x already, the first half of the norm behind it (the rows times the norm's
// weight, and their sums of squares) for the product after the norm to finish.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <map>
#include <string>
#include <vector>

#include "core.h"
#include "prefill_plan.h"

namespace me {

enum OpKind {
  kOpEmbed = 0,       // p0 table, f0 the multiplier on the looked-up rows; -> x
  kOpNormLinear = 1,  // p0 norm weight, f0 eps, p1 W [rows, K], i0 rows of W, i1 K, i2 gated; pending + x -> out
  kOpNorm = 2,        // p0 norm weight, f0 eps; pending + x -> out [tokens, hidden]
  kOpLinear = 3,      // in, p1 W, i0 rows of W, i1 K, i2 gated -> out
  kOpLinearDelta = 4, // in, p1 W, i0 rows of W (= hidden), i1 K -> pending
  kOpDelta = 5,       // in -> pending
  kOpAttention = 6,   // in qkv, p0 q-norm weight, p1 k-norm weight, p2 rotary table, p3 key pages, p4 value pages;
                      // i0 heads, i1 kv heads, i2 head size, i3 rotary size, i4 page size, i5 window, i6 writes pages,
                      // i7 cache group, i8 positions the table covers; f0 eps, f1 scale -> out [tokens, heads * head size]
  kOpHead = 7,        // p0 final norm weight, f0 eps, p1 head W [vocab, hidden], f1 the scale on the logits -> logits of the
                      // wanted rows
  kOpSample = 8,      // logits -> one token per wanted row
  kOpAdd = 9,         // pending + x -> x, as a kernel of its own (before a norm that is no RMS norm)
  kOpCall = 10,       // a part that brings its own code: p0 a function `int (const CallFrame*)`, p1 its context;
                      // in (or -1), out (or -1): the values it reads and writes. It launches on the step's stream.
  kOpHeadRows = 11,   // in: a value whose first rows are the normed wanted rows; p1 head W, f1 the scale on the logits
};

// What a called part is handed (kOpCall). Pointers are device memory of this step: they change from step to step.
struct CallFrame {
  void* context;
  const void* in;   // [tokens, in_cols] or null
  void* out;        // [tokens, out_cols] or null
  float* x;         // the residual stream, float32 [tokens, hidden]
  int64_t in_cols, out_cols;
  int32_t in_elem, out_elem;  // bytes per element
  int32_t tokens, rows;
  hipStream_t stream;
};
typedef int (*CallFn)(const CallFrame*);

struct Op {
  int kind = 0, in = -1, out = -1;
  const void* p[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  int64_t i[10] = {0};
  float f[2] = {0.f, 0.f};
};

struct Value {
  int64_t cols;
  int elem;  // bytes per element
};

// What a run needs to know of its step.
struct StepView {
  const int32_t* dev = nullptr;  // the packed index buffer on the device
  StepLayout lay;
  const int* starts = nullptr;  // host: first position and token count of every item
  const int* qlens = nullptr;
  int max_ctx = 1;
  bool decode_only = true;
  int least_live = 0;  // the fewest live items a replay of this launch will hold (= items for an eager step)
  bool fed = false;  // token ids may come from the tokens the step before drew (the token_source section says which)
  // prefill plans behind the indices, by attention geometry (heads, kv heads, head size, window)
  struct Plan {
    int work = 0, bundle_first = 0, token_chunks = -1, bundles = 0, max_chunks = 1, columns = 0;
  };
  std::map<std::vector<int>, Plan> plans;
};

struct RunResult {
  float* logits = nullptr;
  int32_t* drawn = nullptr;
  int rows = 0;
};

class Program {
 public:
  Program(int dtype, int hidden, int vocab) : dtype_(dtype), hidden_(hidden), vocab_(vocab) {}
  int add_value(int64_t cols, int elem) {
    values_.push_back({cols, elem});
    return (int)values_.size() - 1;
  }
  void add_op(const Op& op) { ops_.push_back(op); }
  int dtype() const { return dtype_; }
  int hidden() const { return hidden_; }
  int vocab() const { return vocab_; }
  const std::vector<Op>& ops() const { return ops_; }
  // Bytes of arena that a step of these sizes may need.
  size_t arena_need(int64_t tokens, int64_t items, int64_t rows, int64_t max_ctx) const;
  RunResult run(const StepView& s, char* arena, size_t arena_bytes, int32_t* fed_tokens, hipStream_t stream) const;
  // Distinct attention geometries that take the matrix-core prefill kernel (their steps need a work list).
  std::vector<std::vector<int>> prefill_geometries() const;

 private:
  int dtype_, hidden_, vocab_;
  std::vector<Value> values_;
  std::vector<Op> ops_;
};

}  // namespace me
