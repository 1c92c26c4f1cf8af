// Page pools, prefix digests, state slots, and the core's page operations.
#include "blake2b.h"
#include "core.h"

#include <algorithm>

namespace me {

Digest chain_digest(const uint8_t* parent, size_t parent_len, const int32_t* tokens, int count) {
  Blake2b h(16);
  if (parent_len) h.update(parent, parent_len);
  for (int i = 0; i < count; ++i) {
    const uint32_t t = (uint32_t)tokens[i];
    const uint8_t le[4] = {(uint8_t)t, (uint8_t)(t >> 8), (uint8_t)(t >> 16), (uint8_t)(t >> 24)};
    h.update(le, 4);
  }
  Digest d;
  h.finish(d.bytes);
  return d;
}

// ---------------------------------------------------------------------------------- PagePool
PagePool::PagePool(int num_pages)
    : holders_(num_pages, 0), has_digest_(num_pages, 0), digest_(num_pages), next_(num_pages + 1), prev_(num_pages + 1),
      listed_(num_pages, 0) {
  const int head = num_pages;
  next_[head] = prev_[head] = head;
  for (int p = 0; p < num_pages; ++p) link_back(p);  // a fresh pool hands out pages in ascending order
}

void PagePool::link_back(int page) {
  const int head = num_pages(), last = prev_[head];
  next_[last] = page;
  prev_[page] = last;
  next_[page] = head;
  prev_[head] = page;
  listed_[page] = 1;
  ++free_count_;
}

void PagePool::link_front(int page) {
  const int head = num_pages(), first = next_[head];
  next_[head] = page;
  prev_[page] = head;
  next_[page] = first;
  prev_[first] = page;
  listed_[page] = 1;
  ++free_count_;
}

void PagePool::unlink(int page) {
  next_[prev_[page]] = next_[page];
  prev_[next_[page]] = prev_[page];
  listed_[page] = 0;
  --free_count_;
}

int PagePool::find(const Digest& d) const {
  auto it = by_digest_.find(d);
  return it == by_digest_.end() ? -1 : it->second;
}

// The front of the free order becomes a page for new content. If it still carried a digest, that
// prefix is gone from the cache now: this is the eviction (reference block_manager.py:144-152).
int PagePool::take() {
  const int head = num_pages();
  const int page = next_[head];
  if (page == head) throw Error(kBroken, "a page was taken from an empty pool");
  unlink(page);
  if (has_digest_[page]) {
    by_digest_.erase(digest_[page]);
    has_digest_[page] = 0;
    ++evictions_;
  }
  holders_[page] = 1;
  return page;
}

void PagePool::retain(int page) {
  if (holders_[page] == 0) unlink(page);
  ++holders_[page];
}

// A page nobody holds any more waits at the back of the free order when its content can still serve
// a prefix hit, and at the front when it cannot (reference block_manager.py:107-118).
void PagePool::release(int page) {
  if (holders_[page] <= 0) throw Error(kBroken, "double free of page " + std::to_string(page));
  if (--holders_[page] == 0) {
    if (has_digest_[page])
      link_back(page);
    else
      link_front(page);
  }
}

// A page takes a digest only when it has none and no other page serves that prefix already: of two
// equal prompts computed side by side the second keeps a private copy (block_manager.py:120-134).
bool PagePool::publish(int page, const Digest& d) {
  if (has_digest_[page] || by_digest_.count(d)) return false;
  has_digest_[page] = 1;
  digest_[page] = d;
  by_digest_.emplace(d, page);
  return true;
}

void PagePool::forget_digests() {
  for (auto& kv : by_digest_) has_digest_[kv.second] = 0;
  by_digest_.clear();
}

std::vector<int32_t> PagePool::free_order() const {
  std::vector<int32_t> out;
  const int head = num_pages();
  for (int p = next_[head]; p != head; p = next_[p]) out.push_back(p);
  return out;
}

// --------------------------------------------------------------------------------- StateSlots
StateSlots::StateSlots(int count) : taken_(count, 0) {
  for (int s = count - 1; s >= 0; --s) spare_.push_back(s);  // slot 0 goes out first
}

int StateSlots::take() {
  if (spare_.empty()) return -1;
  const int s = spare_.back();
  spare_.pop_back();
  taken_[s] = 1;
  return s;
}

void StateSlots::give_back(int slot) {
  if (slot < 0 || slot >= count() || !taken_[slot]) throw Error(kBroken, "state slot freed twice");
  taken_[slot] = 0;
  spare_.push_back(slot);
}

// --------------------------------------------------------------------------- the core's pages
Core::Core(const CoreConfig& config) : config_(config) {
  if (config_.block_size < 1) throw Error(kBadValue, "block_size must be positive");
  if (config_.groups.empty()) throw Error(kBadValue, "at least one cache group is needed");
  bool all_kept = true;
  for (const GroupConfig& g : config_.groups) {
    if (g.num_pages < 1) throw Error(kBadValue, "num_blocks must be positive");
    if (g.window < 0) throw Error(kBadValue, "a window must be >= 0");
    pools_.emplace_back(g.num_pages);
    all_kept = all_kept && g.window == 0;
  }
  if (config_.num_state_slots > 0) slots_.reset(new StateSlots(config_.num_state_slots));
  // a cached prefix can only stand for computed tokens when every group still has all of its keys
  // and no layer has carried state over them
  caching_ = config_.prefix_caching && all_kept && !config_.has_state;
}

int Core::num_free_pages() const {
  int least = pools_[0].num_free();
  for (const PagePool& p : pools_) least = std::min(least, p.num_free());
  return least;
}

long Core::evictions() const {
  long n = 0;
  for (const PagePool& p : pools_) n += p.evictions();
  return n;
}

// Whether a request of this many tokens could hold what a step of it needs, all pools empty. A group
// that keeps every key needs all of the request's pages; a window group needs the window and the
// longest portion a step may bring, plus a page for the portion's ragged start.
bool Core::can_ever_hold(int tokens) const {
  const int all = blocks_for(tokens);
  for (size_t g = 0; g < pools_.size(); ++g) {
    int need = all;
    const int w = config_.groups[g].window;
    if (w > 0) need = std::min(all, blocks_for(w + std::min(config_.max_num_batched_tokens, tokens)) + 1);
    if (need > pools_[g].num_pages()) return false;
  }
  return true;
}

// The longest run of cached full blocks at the head of `tokens` that every group still has. The last
// token is never served from the cache, so that one token at least is computed and gives logits
// (reference block_manager.py:62-79).
int Core::match(const int32_t* tokens, int count, std::vector<std::vector<int32_t>>& hits) const {
  hits.assign(pools_.size(), {});
  if (!caching_) return 0;
  const int bs = config_.block_size;
  Digest parent{};
  int found = 0;
  for (int i = 0; i < (count - 1) / bs; ++i) {
    const Digest d = chain_digest(parent.bytes, i ? 16 : 0, tokens + (size_t)i * bs, bs);
    std::vector<int> pages(pools_.size());
    bool everywhere = true;
    for (size_t g = 0; g < pools_.size(); ++g) {
      pages[g] = pools_[g].find(d);
      everywhere = everywhere && pages[g] >= 0;
    }
    if (!everywhere) break;
    for (size_t g = 0; g < pools_.size(); ++g) hits[g].push_back(pages[g]);
    parent = d;
    ++found;
  }
  return found;
}

// Make every table of `r` cover `num_tokens` tokens and give it a state slot if it has none: all of
// it or nothing. Pages found in the prefix cache (`hits`, only for empty tables) are shared; a hit
// page that was waiting in the free order takes a free place as a new page does
// (reference block_manager.py:83-105).
bool Core::grow(Request* r, int num_tokens, const std::vector<std::vector<int32_t>>* hits) {
  const size_t groups = pools_.size();
  if (r->tables.size() < groups) r->tables.resize(groups);
  const int need = blocks_for(num_tokens);
  const bool wants_slot = slots_ && r->state_slot < 0;
  bool any_hit = false;
  if (hits) {
    if (hits->size() != groups) throw Error(kBadValue, "cached pages must be given per cache group");
    for (const auto& h : *hits) any_hit = any_hit || !h.empty();
  }
  if (any_hit)
    for (const auto& t : r->tables)
      if (!t.empty()) throw Error(kBadValue, "cached blocks can only seed an empty block table");

  std::vector<int> fresh(groups, 0);
  for (size_t g = 0; g < groups; ++g) {
    const int hit_count = any_hit ? (int)(*hits)[g].size() : 0;
    fresh[g] = std::max(0, need - (int)r->tables[g].size() - hit_count);
    int revived = 0;
    if (any_hit)
      for (int page : (*hits)[g]) {
        if (page < 0 || page >= pools_[g].num_pages()) throw Error(kBadValue, "a cached page id is out of range");
        revived += pools_[g].holders(page) == 0;
      }
    if (fresh[g] + revived > pools_[g].num_free()) return false;
  }
  if (wants_slot && slots_->num_free() == 0) return false;

  for (size_t g = 0; g < groups; ++g) {
    std::vector<int32_t>& table = r->tables[g];
    if (any_hit)
      for (int page : (*hits)[g]) {
        pools_[g].retain(page);
        table.push_back(page);
      }
    for (int i = 0; i < fresh[g]; ++i) table.push_back(pools_[g].take());
  }
  if (wants_slot) r->state_slot = slots_->take();
  return true;
}

// Give back everything `r` holds. Pages go back last page first, so that of pages freed together a
// request's tail is taken again before its head, which other prompts are likelier to share.
void Core::drop(Request* r) {
  for (size_t g = 0; g < r->tables.size() && g < pools_.size(); ++g) {
    std::vector<int32_t>& table = r->tables[g];
    for (size_t i = table.size(); i-- > 0;)
      if (table[i] >= 0) pools_[g].release(table[i]);
    table.clear();
  }
  ++r->table_epoch;
  r->chain.clear();
  if (slots_ && r->state_slot >= 0) slots_->give_back(r->state_slot);
  r->state_slot = -1;
}

// Pages of window groups that no later query of `r` can see go back at once: a query at position
// p >= num_computed sees the keys from p - window + 1 on.
int Core::drop_passed(Request* r) {
  int freed = 0;
  for (size_t g = 0; g < r->tables.size() && g < pools_.size(); ++g) {
    const int w = config_.groups[g].window;
    if (w <= 0) continue;
    const int first_needed = std::max(0, r->num_computed - w + 1);
    std::vector<int32_t>& table = r->tables[g];
    const int whole = std::min((int)table.size(), first_needed / config_.block_size);
    for (int i = 0; i < whole; ++i)
      if (table[i] >= 0) {
        pools_[g].release(table[i]);
        table[i] = -1;
        ++r->table_epoch;
        ++freed;
      }
  }
  return freed;
}

// Blocks of `r` that have become full and computed since the last call get their chained digest
// (over prompt and generated tokens alike) and are offered to the prefix cache.
void Core::note_computed(Request* r) {
  if (!caching_) return;
  const int bs = config_.block_size;
  for (int i = (int)r->chain.size(); i < r->num_computed / bs; ++i) {
    const Digest d = chain_digest(i ? r->chain.back().bytes : nullptr, i ? 16 : 0, r->tokens.data() + (size_t)i * bs, bs);
    r->chain.push_back(d);
    for (size_t g = 0; g < pools_.size(); ++g)
      if (i < (int)r->tables[g].size() && r->tables[g][i] >= 0) pools_[g].publish(r->tables[g][i], d);
  }
}

void Core::forget_digests() {
  for (PagePool& p : pools_) p.forget_digests();
}

}  // namespace me
