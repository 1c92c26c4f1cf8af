// The native runner: owns a model's step program and the memory its steps use, and runs a step of the
// host core from one call: check, pack the indices (and the prefill attention's work lists) into pinned
// memory, one upload, every kernel of the model, the draw of the next tokens. Memory is handed in by
// the caller (one arena for activations and workspaces, two pinned staging buffers, the index buffer on
// the device): nothing is allocated while steps run, so a run can be captured into a graph.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <list>

#include "../kernels.h"
#include "program.h"

int me_fail(const char* fmt, ...);

namespace {

struct CachedPlan {
  std::vector<int> key;
  me::WorkList list;
  int columns = 0;
};

struct Runner {
  me::Program prog;
  char* arena = nullptr;
  size_t arena_bytes = 0;
  int32_t* staging[2] = {nullptr, nullptr};
  hipEvent_t copied[2] = {nullptr, nullptr};
  bool in_flight[2] = {false, false};
  size_t staging_ints = 0;
  int parity = 0;
  int32_t* dev_index = nullptr;
  size_t dev_index_ints = 0;
  int spare_page = 0, spare_slot = 0;
  int compute_units = 0;
  std::vector<std::vector<int>> geometries;
  std::list<CachedPlan> plans;  // the last work lists made, newest first: the steps of a serving loop repeat
  std::vector<int> starts, qlens;
  Runner(int dtype, int hidden, int vocab) : prog(dtype, hidden, vocab) {}
  ~Runner() {
    for (hipEvent_t e : copied)
      if (e) hipEventDestroy(e);
  }
};

thread_local int g_kind = 0;

#define ME_RUN_GUARD(...)                 \
  try {                                   \
    g_kind = 0;                           \
    __VA_ARGS__                           \
  } catch (const me::Error& e) {          \
    g_kind = e.kind;                      \
    me_fail("%s", e.what());              \
    return -1;                            \
  } catch (const std::exception& e) {     \
    g_kind = me::kBroken;                 \
    me_fail("%s", e.what());              \
    return -1;                            \
  }

void hip_ok(hipError_t e, const char* what) {
  if (e != hipSuccess) throw me::Error(me::kBadState, std::string(what) + ": " + hipGetErrorString(e));
}

// The work list of one attention geometry for the current step, from the cache or made now.
const CachedPlan& plan_for(Runner& r, const std::vector<int>& geometry) {
  const int nh = geometry[0], nkv = geometry[1], d = geometry[2], window = geometry[3];
  std::vector<int> key = geometry;
  key.insert(key.end(), r.starts.begin(), r.starts.end());
  key.push_back(-1);
  key.insert(key.end(), r.qlens.begin(), r.qlens.end());
  for (auto it = r.plans.begin(); it != r.plans.end(); ++it)
    if (it->key == key) {
      r.plans.splice(r.plans.begin(), r.plans, it);
      return r.plans.front();
    }
  CachedPlan fresh;
  fresh.key = key;
  const int items = (int)r.starts.size(), group = nh / nkv;
  const bool wide = me::wide_blocks_pay(r.starts.data(), r.qlens.data(), items,
                                        std::max(1, me_attention_prefill_columns(1) / group), window, nkv, r.compute_units);
  fresh.columns = me_attention_prefill_columns(wide ? 1 : 0);
  me::build_work_list(r.starts.data(), r.qlens.data(), items, fresh.columns / group, window, nkv, r.compute_units,
                      (long long)nh * d * 4, fresh.list);
  r.plans.push_front(std::move(fresh));
  if (r.plans.size() > 64) r.plans.pop_back();
  return r.plans.front();
}

void report(const me::RunResult& res, int64_t* out) {
  out[0] = (int64_t)(intptr_t)res.logits;
  out[1] = res.rows;
  out[2] = (int64_t)(intptr_t)res.drawn;
  out[3] = 0;
}

}  // namespace

extern "C" {

int me_runner_error_kind() { return g_kind; }

void* me_runner_new(int dtype, int hidden, int vocab) {
  if ((dtype != 0 && dtype != 1) || hidden < 1 || vocab < 1) {
    me_fail("me_runner_new: dtype=%d hidden=%d vocab=%d", dtype, hidden, vocab);
    return nullptr;
  }
  return new Runner(dtype, hidden, vocab);
}

void me_runner_delete(void* runner) { delete (Runner*)runner; }

int me_runner_value(void* runner, int64_t cols, int elem) {
  ME_RUN_GUARD(if (cols < 1 || (elem != 2 && elem != 4)) throw me::Error(me::kBadValue, "a value needs columns and 2- or 4-byte elements");
               return ((Runner*)runner)->prog.add_value(cols, elem);)
}

// ptrs: 6 pointers, ints: 10, floats: 2 (see OpKind in program.h for what each operation reads).
int me_runner_op(void* runner, int kind, int in, int out, const void* const* ptrs, const int64_t* ints, const float* floats) {
  ME_RUN_GUARD(me::Op op; op.kind = kind; op.in = in; op.out = out;
               for (int i = 0; i < 6; ++i) op.p[i] = ptrs[i];
               for (int i = 0; i < 10; ++i) op.i[i] = ints[i];
               op.f[0] = floats[0]; op.f[1] = floats[1];
               Runner* r = (Runner*)runner; r->prog.add_op(op); r->geometries = r->prog.prefill_geometries();
               return (int)r->prog.ops().size();)
}

int64_t me_runner_arena_need(void* runner, int64_t tokens, int64_t items, int64_t rows, int64_t max_ctx) {
  ME_RUN_GUARD(return (int64_t)((Runner*)runner)->prog.arena_need(tokens, items, rows, max_ctx);)
}

// Ints that the staging and index buffers need for a step of these sizes: the packed indices plus the work
// lists of the prefill attention (one per attention geometry of the program).
int64_t me_runner_index_need(void* runner, int tokens, int items, int rows, const int32_t* widths, int num_groups) {
  ME_RUN_GUARD(Runner* r = (Runner*)runner;
               const me::StepLayout l = me::StepLayout::make(tokens, items, rows, std::vector<int>(widths, widths + num_groups));
               // tiles: at most one per 1 token-run of an item plus one per item; cut pieces: at most as many again
               // plus two per compute unit; 8 ints per entry, one per bundle, one per token
               const int64_t entries = 2 * ((int64_t)tokens / 4 + items) + 2048;
               return (int64_t)l.total + (int64_t)r->geometries.size() * (entries * 9 + tokens) + 64;)
}

// The memory of eager steps; may be given anew (larger) between steps, once the device has finished the last.
int me_runner_memory(void* runner, void* arena, int64_t arena_bytes, int32_t* staging0, int32_t* staging1, int64_t staging_ints,
                     int32_t* dev_index, int64_t dev_index_ints, int spare_page, int spare_slot) {
  ME_RUN_GUARD(Runner* r = (Runner*)runner;
               if (!arena || arena_bytes < 1 || !staging0 || !staging1 || !dev_index)
                 throw me::Error(me::kBadValue, "the runner needs an arena, two staging buffers and an index buffer");
               r->arena = (char*)arena; r->arena_bytes = (size_t)arena_bytes; r->staging[0] = staging0; r->staging[1] = staging1;
               r->staging_ints = (size_t)staging_ints; r->dev_index = dev_index; r->dev_index_ints = (size_t)dev_index_ints;
               r->spare_page = spare_page; r->spare_slot = spare_slot; r->in_flight[0] = r->in_flight[1] = false;
               int dev = 0; hip_ok(hipGetDevice(&dev), "hipGetDevice");
               hip_ok(hipDeviceGetAttribute(&r->compute_units, hipDeviceAttributeMultiprocessorCount, dev), "compute unit count");
               for (int i = 0; i < 2; ++i)
                 if (!r->copied[i]) hip_ok(hipEventCreateWithFlags(&r->copied[i], hipEventDisableTiming), "hipEventCreate");
               return 0;)
}

// Run the step that the core holds, eagerly: out[0] logits (device, float32 [rows, vocab]), out[1] rows,
// out[2] the tokens drawn for the rows (device int32), if the program draws, out[3] the query columns of the
// prefill attention's blocks (0: the step ran no such kernel).
int me_runner_step(void* runner, void* core_box, hipStream_t stream, int64_t* out) {
  ME_RUN_GUARD(
      Runner* r = (Runner*)runner; me::Core& c = *me::core_in_box(core_box);
      if (!r->arena) throw me::Error(me::kBadState, "the runner has no memory yet");
      c.check_step(r->prog.vocab(), true);
      me::StepView s;
      s.lay = c.layout(nullptr, 0);
      r->starts.clear(); r->qlens.clear();
      int longest = 0, ctx = 0;
      for (const me::StepItem& it : c.step()) {
        r->starts.push_back(it.start); r->qlens.push_back(it.count);
        longest = std::max(longest, it.count); ctx = std::max(ctx, it.start + it.count);
      }
      s.starts = r->starts.data(); s.qlens = r->qlens.data(); s.max_ctx = ctx; s.decode_only = longest == 1;
      s.least_live = s.lay.items;
      const int slot = r->parity; r->parity ^= 1;
      if (r->in_flight[slot]) { hip_ok(hipEventSynchronize(r->copied[slot]), "waiting for a staging buffer"); r->in_flight[slot] = false; }
      int32_t* host = r->staging[slot];
      size_t total = (size_t)s.lay.total;
      if (total > r->staging_ints || total > r->dev_index_ints) throw me::Error(me::kBadState, "the step's indices do not fit the runner's buffers");
      c.pack(host, s.lay, r->spare_page, r->spare_slot);
      if (!s.decode_only)
        for (const std::vector<int>& geometry : r->geometries) {
          const CachedPlan& p = plan_for(*r, geometry);
          const size_t need = p.list.work.size() + p.list.bundle_first.size() + (p.list.max_chunks > 1 ? p.list.token_chunks.size() : 0);
          if (total + need > r->staging_ints || total + need > r->dev_index_ints)
            throw me::Error(me::kBadState, "the step's attention work list does not fit the runner's buffers");
          me::StepView::Plan v;
          v.work = (int)total; std::copy(p.list.work.begin(), p.list.work.end(), host + total); total += p.list.work.size();
          v.bundle_first = (int)total; std::copy(p.list.bundle_first.begin(), p.list.bundle_first.end(), host + total);
          total += p.list.bundle_first.size();
          if (p.list.max_chunks > 1) { v.token_chunks = (int)total;
            std::copy(p.list.token_chunks.begin(), p.list.token_chunks.end(), host + total); total += p.list.token_chunks.size(); }
          v.bundles = (int)p.list.bundle_first.size(); v.max_chunks = p.list.max_chunks; v.columns = p.columns;
          s.plans[geometry] = v;
        }
      hip_ok(hipMemcpyAsync(r->dev_index, host, total * 4, hipMemcpyHostToDevice, stream), "uploading the step's indices");
      hip_ok(hipEventRecord(r->copied[slot], stream), "hipEventRecord"); r->in_flight[slot] = true;
      s.dev = r->dev_index;
      report(r->prog.run(s, r->arena, r->arena_bytes, nullptr, stream), out);
      if (!s.plans.empty()) out[3] = s.plans.begin()->second.columns;
      return 0;)
}

// Run a decode step whose indices already are on the device, in a buffer of `bucket` one-token items laid
// out with `widths` (what a graph is captured on and replayed from), with workspaces from an arena of the
// caller's (the one a graph was captured on stays the graph's). `drawn`: where the tokens drawn for the
// rows go (null: into the arena); with `fed`, token ids come from there too, where the buffer's
// token_source section says so: the tokens the step before drew.
int me_runner_static(void* runner, void* arena, int64_t arena_bytes, const int32_t* dev_index, int bucket,
                     const int32_t* widths, int num_groups, int max_ctx, int least_live, int32_t* drawn, int fed,
                     hipStream_t stream, int64_t* out) {
  ME_RUN_GUARD(
      Runner* r = (Runner*)runner;
      if (!arena || arena_bytes < 1 || !dev_index) throw me::Error(me::kBadValue, "a static step needs an arena and an index buffer");
      if (bucket < 1 || max_ctx < 1) throw me::Error(me::kBadValue, "a static step needs items and a context length");
      if (fed && !drawn) throw me::Error(me::kBadValue, "fed token ids need the buffer the step before drew into");
      me::StepView s;
      s.lay = me::StepLayout::make(bucket, bucket, bucket, std::vector<int>(widths, widths + num_groups));
      std::vector<int> starts(bucket, 0), qlens(bucket, 1);
      s.starts = starts.data(); s.qlens = qlens.data(); s.max_ctx = max_ctx; s.decode_only = true;
      s.least_live = std::max(1, std::min(least_live, bucket));
      s.dev = dev_index; s.fed = fed != 0;
      report(r->prog.run(s, (char*)arena, (size_t)arena_bytes, drawn, stream), out);
      return 0;)
}

}  // extern "C"
