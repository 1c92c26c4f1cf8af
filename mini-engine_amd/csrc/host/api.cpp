// The C face of the host core, called from Python through ctypes. Every function returns a value
// >= 0 on success and -1 on failure, with the failure's kind in me_host_error_kind() and its text in
// me_last_error(). Requests are named by the handles me_core_request returns.
#include "core.h"

#include <algorithm>
#include <unordered_map>

int me_fail(const char* fmt, ...);

namespace {

struct CoreBox {
  me::Core core;
  std::unordered_map<int, std::vector<me::RowMemo>> memos;  // per graph bucket: what its rows hold
  explicit CoreBox(const me::CoreConfig& c) : core(c) {}
};

thread_local int g_kind = 0;

int failed(const me::Error& e) {
  g_kind = e.kind;
  me_fail("%s", e.what());
  return -1;
}
int failed(const std::exception& e) {
  g_kind = me::kBroken;
  me_fail("%s", e.what());
  return -1;
}

#define ME_GUARD(...)             \
  try {                           \
    g_kind = 0;                   \
    __VA_ARGS__                   \
  } catch (const me::Error& e) {  \
    return failed(e);             \
  } catch (const std::exception& e) { \
    return failed(e);             \
  }

me::Core& core_of(void* box) { return ((CoreBox*)box)->core; }

std::vector<std::vector<int32_t>> unflatten(const me::Core& c, const int32_t* hits, int blocks) {
  std::vector<std::vector<int32_t>> per_group(c.num_groups());
  for (int g = 0; g < c.num_groups(); ++g) per_group[g].assign(hits + (size_t)g * blocks, hits + (size_t)(g + 1) * blocks);
  return per_group;
}

}  // namespace

me::Core* me::core_in_box(void* box) { return &((CoreBox*)box)->core; }

extern "C" {

int me_host_error_kind() { return g_kind; }

// settings: block_size, prefix_caching, num_state_slots, has_state, max_num_seqs, max_num_batched_tokens,
// max_model_len; groups: (window, num_pages) per cache group.
void* me_core_new(const int32_t* settings, const int32_t* groups, int num_groups, const int32_t* eos, int num_eos,
                  uint64_t seed) {
  try {
    g_kind = 0;
    me::CoreConfig c;
    c.block_size = settings[0];
    c.prefix_caching = settings[1] != 0;
    c.num_state_slots = settings[2];
    c.has_state = settings[3] != 0;
    c.max_num_seqs = settings[4];
    c.max_num_batched_tokens = settings[5];
    c.max_model_len = settings[6];
    for (int g = 0; g < num_groups; ++g) c.groups.push_back({groups[2 * g], groups[2 * g + 1]});
    c.eos_ids.assign(eos, eos + num_eos);
    c.seed = seed;
    return new CoreBox(c);
  } catch (const me::Error& e) {
    failed(e);
  } catch (const std::exception& e) {
    failed(e);
  }
  return nullptr;
}

void me_core_delete(void* box) { delete (CoreBox*)box; }

int me_core_set_limits(void* box, int max_num_seqs, int max_num_batched_tokens, int max_model_len, const int32_t* eos,
                       int num_eos) {
  ME_GUARD(if (max_num_seqs < 1 || max_num_batched_tokens < 1 || max_model_len < 1)
               throw me::Error(me::kBadValue, "limits must be positive");
           core_of(box).set_limits(max_num_seqs, max_num_batched_tokens, max_model_len, std::vector<int32_t>(eos, eos + num_eos));
           return 0;)
}

// ------------------------------------------------------------------------------------ requests
int64_t me_core_request(void* box, const int32_t* tokens, int count, int max_tokens, float temperature, int ignore_eos) {
  ME_GUARD(return core_of(box).create(tokens, count, max_tokens, temperature, ignore_eos != 0)->handle;)
}

int me_core_release(void* box, int64_t handle) { ME_GUARD(core_of(box).unhold(handle); return 0;) }

// out: phase, tokens, prompt tokens, computed, cached at admission, preemptions, state slot, table epoch,
// digests in its chain
int me_core_request_info(void* box, int64_t handle, int64_t* out) {
  ME_GUARD(const me::Request* r = core_of(box).get(handle); out[0] = r->phase; out[1] = r->size(); out[2] = r->num_prompt;
           out[3] = r->num_computed; out[4] = r->num_cached; out[5] = r->num_preemptions; out[6] = r->state_slot;
           out[7] = r->table_epoch; out[8] = (int64_t)r->chain.size(); return 0;)
}

int me_core_request_tokens(void* box, int64_t handle, int from, int count, int32_t* out) {
  ME_GUARD(const me::Request* r = core_of(box).get(handle);
           if (from < 0 || count < 0 || from + count > r->size()) throw me::Error(me::kBadValue, "token range out of bounds");
           std::copy(r->tokens.begin() + from, r->tokens.begin() + from + count, out); return count;)
}

int me_core_request_table(void* box, int64_t handle, int group, int32_t* out, int cap) {
  ME_GUARD(const me::Request* r = core_of(box).get(handle);
           if (group < 0 || group >= (int)r->tables.size()) return 0;
           const auto& t = r->tables[group]; if (out) std::copy(t.begin(), t.begin() + std::min<size_t>(cap, t.size()), out);
           return (int)t.size();)
}

int me_core_request_extend(void* box, int64_t handle, const int32_t* tokens, int count) {
  ME_GUARD(me::Request* r = core_of(box).get(handle); r->tokens.insert(r->tokens.end(), tokens, tokens + count);
           return r->size();)
}

// what: 0 num_computed, 1 num_prompt (a trace's requests have no prompt apart from what steps bring)
int me_core_request_set(void* box, int64_t handle, int what, int64_t value) {
  ME_GUARD(me::Request* r = core_of(box).get(handle);
           if (value < 0 || value > r->size()) throw me::Error(me::kBadValue, "value beyond the request's tokens");
           if (what == 0) r->num_computed = (int)value; else if (what == 1) r->num_prompt = (int)value;
           else throw me::Error(me::kBadValue, "unknown field"); return 0;)
}

int me_core_request_truncate(void* box, int64_t handle, int count) {
  ME_GUARD(me::Request* r = core_of(box).get(handle);
           if (count < r->num_computed || count > r->size()) throw me::Error(me::kBadValue, "cannot truncate there");
           r->tokens.resize(count); return count;)
}

// --------------------------------------------------------------------------------------- pages
int me_chain_digest(const uint8_t* parent, int parent_len, const int32_t* tokens, int count, uint8_t* out16) {
  ME_GUARD(const me::Digest d = me::chain_digest(parent, (size_t)parent_len, tokens, count); memcpy(out16, d.bytes, 16);
           return 0;)
}

// Hit pages go to out[g * blocks + i]; returns the number of hit blocks (cap: blocks out can hold per group).
int me_core_match(void* box, const int32_t* tokens, int count, int32_t* out, int cap) {
  ME_GUARD(std::vector<std::vector<int32_t>> hits; me::Core& c = core_of(box); const int blocks = c.match(tokens, count, hits);
           if (blocks > cap) throw me::Error(me::kBadValue, "the buffer for hit pages is too small");
           for (int g = 0; g < c.num_groups(); ++g) std::copy(hits[g].begin(), hits[g].end(), out + (size_t)g * blocks);
           return blocks;)
}

// 1: grown, 0: no room (nothing changed)
int me_core_grow(void* box, int64_t handle, int num_tokens, const int32_t* hits, int hit_blocks) {
  ME_GUARD(me::Core& c = core_of(box); me::Request* r = c.get(handle);
           if (hit_blocks > 0) { auto per_group = unflatten(c, hits, hit_blocks); return c.grow(r, num_tokens, &per_group) ? 1 : 0; }
           return c.grow(r, num_tokens) ? 1 : 0;)
}

int me_core_drop(void* box, int64_t handle) { ME_GUARD(me::Core& c = core_of(box); c.drop(c.get(handle)); return 0;) }
int me_core_drop_passed(void* box, int64_t handle) { ME_GUARD(me::Core& c = core_of(box); return c.drop_passed(c.get(handle));) }
int me_core_note_computed(void* box, int64_t handle) { ME_GUARD(me::Core& c = core_of(box); c.note_computed(c.get(handle)); return 0;) }
int me_core_forget_digests(void* box) { ME_GUARD(core_of(box).forget_digests(); return 0;) }
int me_core_can_ever_hold(void* box, int tokens) { ME_GUARD(return core_of(box).can_ever_hold(tokens) ? 1 : 0;) }

// out: groups, caching on, least free pages over the groups, evictions, state slots (0: none), free slots
int me_core_pages_info(void* box, int64_t* out) {
  ME_GUARD(me::Core& c = core_of(box); out[0] = c.num_groups(); out[1] = c.caching(); out[2] = c.num_free_pages();
           out[3] = c.evictions(); out[4] = c.slots() ? c.slots()->count() : 0; out[5] = c.slots() ? c.slots()->num_free() : 0;
           return 0;)
}

// A pool as arrays (for tests and diagnostics): holders[p], has_digest[p], digests[16 p], free_order[..]; returns
// the number of free pages. Any pointer may be null.
int me_core_pool(void* box, int group, int32_t* holders, uint8_t* has_digest, uint8_t* digests, int32_t* free_order,
                 int64_t* info) {
  ME_GUARD(me::Core& c = core_of(box);
           if (group < 0 || group >= c.num_groups()) throw me::Error(me::kBadValue, "no such cache group");
           me::PagePool& p = c.pool(group);
           for (int i = 0; i < p.num_pages(); ++i) {
             if (holders) holders[i] = p.holders(i);
             if (has_digest) has_digest[i] = p.has_digest(i);
             if (digests && p.has_digest(i)) memcpy(digests + 16 * (size_t)i, p.digest(i).bytes, 16);
           }
           const std::vector<int32_t> order = p.free_order();
           if (free_order) std::copy(order.begin(), order.end(), free_order);
           if (info) { info[0] = p.num_pages(); info[1] = p.num_free(); info[2] = p.evictions(); }
           return (int)order.size();)
}

int me_core_find_digest(void* box, int group, const uint8_t* digest16) {
  ME_GUARD(me::Digest d; memcpy(d.bytes, digest16, 16); const int page = core_of(box).pool(group).find(d);
           return page < 0 ? -2 : page;)
}

int me_core_release_page(void* box, int group, int page) {
  ME_GUARD(me::Core& c = core_of(box);
           if (group < 0 || group >= c.num_groups() || page < 0 || page >= c.pool(group).num_pages())
             throw me::Error(me::kBadValue, "no such page");
           c.pool(group).release(page); return 0;)
}

int me_core_slots(void* box, uint8_t* taken, int cap) {
  ME_GUARD(me::StateSlots* s = core_of(box).slots(); if (!s) return 0;
           for (int i = 0; i < s->count() && i < cap; ++i) taken[i] = s->taken(i); return s->count();)
}

// ----------------------------------------------------------------------------------- scheduler
int me_core_enqueue(void* box, int64_t handle) { ME_GUARD(me::Core& c = core_of(box); c.enqueue(c.get(handle)); return 0;) }
int me_core_plan(void* box) { ME_GUARD(return core_of(box).plan();) }

int me_core_settle(void* box, const int32_t* next_tokens, int count, int64_t* finished, int cap) {
  ME_GUARD(std::vector<int64_t> done; const int n = core_of(box).settle(next_tokens, count, done);
           for (int i = 0; i < n && i < cap; ++i) finished[i] = done[i]; return n;)
}

// Handles of the waiting queue (front first), then of the running list (admission order).
int me_core_queues(void* box, int64_t* waiting, int cap_waiting, int64_t* running, int cap_running, int32_t* counts) {
  ME_GUARD(me::Core& c = core_of(box); int i = 0;
           for (me::Request* r : c.waiting()) { if (i < cap_waiting) waiting[i] = r->handle; ++i; }
           counts[0] = i; i = 0;
           for (me::Request* r : c.running()) { if (i < cap_running) running[i] = r->handle; ++i; }
           counts[1] = i; return 0;)
}

// out: preemptions, tokens served by the prefix cache, evictions, unfinished (0/1)
int me_core_counters(void* box, int64_t* out) {
  ME_GUARD(me::Core& c = core_of(box); out[0] = c.preemptions; out[1] = c.cached_tokens; out[2] = c.evictions();
           out[3] = c.unfinished(); out[4] = c.generated; return 0;)
}

// ---------------------------------------------------------------------------------------- step
int me_core_step_clear(void* box) { ME_GUARD(core_of(box).step().clear(); return 0;) }

int me_core_step_add(void* box, int64_t handle, int start, int count, const int32_t* want, int num_want) {
  ME_GUARD(me::Core& c = core_of(box); me::StepItem it{c.get(handle), start, count, {}}; it.want.assign(want, want + num_want);
           c.step().push_back(std::move(it)); return (int)c.step().size();)
}

// Per item: handle, start, count, number of wanted places, state slot (-1: none). Returns the number of items.
int me_core_step_items(void* box, int64_t* handles, int32_t* starts, int32_t* counts, int32_t* wants, int32_t* slots, int cap) {
  ME_GUARD(auto& s = core_of(box).step(); int i = 0;
           for (const me::StepItem& it : s) { if (i < cap) { handles[i] = it.request->handle; starts[i] = it.start;
               counts[i] = it.count; wants[i] = (int)it.want.size(); slots[i] = it.request->state_slot; } ++i; }
           return i;)
}

// out: tokens, items, wanted rows, longest item, longest context, 1 if every item is one token, 1 if every item
// wants exactly its last token, 1 if some row is sampled with a temperature
int me_core_step_summary(void* box, int32_t* out) {
  ME_GUARD(auto& s = core_of(box).step(); int t = 0, r = 0, longest = 0, ctx = 0, decode = 1, last_only = 1, warm = 0;
           for (const me::StepItem& it : s) { t += it.count; r += (int)it.want.size(); longest = std::max(longest, it.count);
             ctx = std::max(ctx, it.start + it.count); decode &= it.count == 1;
             last_only &= it.want.size() == 1 && it.want[0] == it.count - 1;
             warm |= it.request->temperature > 0.f; }
           out[0] = t; out[1] = (int)s.size(); out[2] = r; out[3] = longest; out[4] = ctx; out[5] = decode; out[6] = last_only;
           out[7] = warm; return (int)s.size();)
}

int me_core_step_check(void* box, int vocab_size, int scan_pages) {
  ME_GUARD(core_of(box).check_step(vocab_size, scan_pages != 0); return 0;)
}

// out: tokens, items, rows, total, then the offsets of token_ids, positions, token_item, want_rows, item_start,
// item_ctx, state_slots, live_items, temperatures, sample_keys, token_source, then per group its width and its
// table's offset.
static void write_layout(const me::StepLayout& l, int32_t* out) {
  const int head[] = {l.tokens, l.items, l.rows, l.total, l.token_ids, l.positions, l.token_item, l.want_rows, l.item_start,
                      l.item_ctx, l.state_slots, l.live_items, l.temperatures, l.sample_keys, l.token_source};
  std::copy(head, head + 15, out);
  for (size_t g = 0; g < l.widths.size(); ++g) {
    out[15 + 2 * g] = l.widths[g];
    out[16 + 2 * g] = l.tables[g];
  }
}

int me_step_layout(int tokens, int items, int rows, const int32_t* widths, int num_groups, int32_t* out) {
  ME_GUARD(write_layout(me::StepLayout::make(tokens, items, rows, std::vector<int>(widths, widths + num_groups)), out);
           return 0;)
}

int me_core_step_layout(void* box, const int32_t* widths, int pad_items, int32_t* out) {
  ME_GUARD(me::Core& c = core_of(box); std::vector<int> w; if (widths) w.assign(widths, widths + c.num_groups());
           write_layout(c.layout(widths ? &w : nullptr, pad_items), out); return 0;)
}

int me_core_step_pack(void* box, int32_t* dst, int cap, const int32_t* widths, int pad_items, int spare_page, int spare_slot) {
  ME_GUARD(me::Core& c = core_of(box); std::vector<int> w; if (widths) w.assign(widths, widths + c.num_groups());
           const me::StepLayout l = c.layout(widths ? &w : nullptr, pad_items);
           if (l.total > cap) throw me::Error(me::kBadValue, "the step does not fit its buffer");
           c.pack(dst, l, spare_page, spare_slot); return l.total;)
}

// The buffer of a step that holds nothing but `items` padding items (what a graph is captured on).
int me_core_pack_padding(void* box, int32_t* dst, int cap, const int32_t* widths, int items, int spare_page, int spare_slot) {
  ME_GUARD(me::Core& c = core_of(box); std::vector<int> w(widths, widths + c.num_groups());
           const me::StepLayout l = me::StepLayout::make(items, items, items, w);
           if (l.total > cap) throw me::Error(me::kBadValue, "the step does not fit its buffer");
           std::vector<me::StepItem> held; held.swap(c.step());
           try { c.pack(dst, l, spare_page, spare_slot); } catch (...) { held.swap(c.step()); throw; }
           held.swap(c.step()); return l.total;)
}

// Settle the planned step from the tokens drawn for its wanted rows, in the order of the rows: an item
// with a wanted place takes the next of them, any other item none.
int me_core_settle_rows(void* box, const int32_t* drawn, int count, int64_t* finished, int cap) {
  ME_GUARD(me::Core& c = core_of(box); std::vector<int32_t> next; int at = 0;
           for (const me::StepItem& it : c.step()) {
             if (it.want.size() > 1) throw me::Error(me::kBadValue, "a scheduled item wants at most its last place");
             if (it.want.empty()) { next.push_back(-1); continue; }
             if (at >= count) throw me::Error(me::kBadValue, "fewer tokens were drawn than the step has wanted rows");
             next.push_back(drawn[at++]); }
           if (at != count) throw me::Error(me::kBadValue, "more tokens were drawn than the step has wanted rows");
           std::vector<int64_t> done; const int n = c.settle(next.data(), (int)next.size(), done);
           for (int i = 0; i < n && i < cap; ++i) finished[i] = done[i]; return n;)
}

// One step ahead (Core::plan_ahead, Core::settle_in_flight).
int me_core_plan_ahead(void* box) { ME_GUARD(return core_of(box).plan_ahead();) }

int me_core_settle_in_flight(void* box, const int32_t* drawn, int count, int64_t* finished, int cap) {
  ME_GUARD(std::vector<int64_t> done; const int n = core_of(box).settle_in_flight(drawn, count, done);
           for (int i = 0; i < n && i < cap; ++i) finished[i] = done[i]; return n;)
}

int me_core_step_refill(void* box, int bucket, int32_t* dst, const int32_t* widths, int spare_page, int spare_slot) {
  ME_GUARD(CoreBox* b = (CoreBox*)box; me::Core& c = b->core; std::vector<int> w(widths, widths + c.num_groups());
           const me::StepLayout l = me::StepLayout::make(bucket, bucket, bucket, w);
           c.refill(dst, l, b->memos[bucket], spare_page, spare_slot); return l.total;)
}

int me_core_forget_rows(void* box, int bucket) { ME_GUARD(((CoreBox*)box)->memos.erase(bucket); return 0;) }

}  // extern "C"
