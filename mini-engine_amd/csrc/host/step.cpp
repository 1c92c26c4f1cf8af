// A step's indices: checks that make every index a kernel will form a valid one, and the packing of
// the items into one int32 buffer that is uploaded with one copy.
//
// Sections of the buffer, in order (T tokens, B items, R wanted rows, G groups of width W_g):
//   token_ids[T] positions[T] token_item[T] want_rows[R] item_start[B+1] item_ctx[B] state_slots[B]
//   live_items[2] (the live items; bit 0 of the second word: the items share pages) temperatures[R] (float bits) sample_keys[R] (64 bits each, 8-byte aligned)
//   token_source[T] (-1: the token's id is token_ids[t]; r >= 0: it is the r-th token the step before drew,
//   which is still on the device)
//   block_table_0[B, W_0] ... block_table_{G-1}[B, W_{G-1}]
// Instead of a padded mask the kernels get, per token, its absolute position and the index of its
// item, and per item and cache group a row of the block table.
#include "core.h"

#include <algorithm>

namespace me {

StepLayout StepLayout::make(int tokens, int items, int rows, const std::vector<int>& widths) {
  StepLayout l;
  l.tokens = tokens;
  l.items = items;
  l.rows = rows;
  l.widths = widths;
  int at = 0;
  auto section = [&](int& where, int count) {
    where = at;
    at += count;
  };
  section(l.token_ids, tokens);
  section(l.positions, tokens);
  section(l.token_item, tokens);
  section(l.want_rows, rows);
  section(l.item_start, items + 1);
  section(l.item_ctx, items);
  section(l.state_slots, items);
  section(l.live_items, 2);
  section(l.temperatures, rows);
  at += at & 1;  // the keys are read as 64-bit values
  section(l.sample_keys, 2 * rows);
  section(l.token_source, tokens);
  for (int w : widths) {
    l.tables.push_back(at);
    at += items * w;
  }
  l.total = at;
  return l;
}

static uint64_t mix64(uint64_t z) {  // splitmix64's finaliser, as the sampling kernel mixes its noise
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

// The key of a request's next draw: a function of the engine's seed, the request's number within
// this engine and the index of the output token, so a request's samples do not depend on what shares
// its batches, and a second engine with the same seed draws the same.
uint64_t Core::draw_key(const Request* r) const {
  return mix64(mix64(mix64(config_.seed) ^ (uint64_t)r->serial) ^ (uint64_t)r->num_output());
}

void Core::check_step(int vocab_size, bool scan_pages) const {
  if (step_.empty()) throw Error(kBadValue, "a step needs at least one item");
  const int bs = config_.block_size;
  // A request named twice would advance twice when the step is settled, and its second item would read keys that the
  // first writes in the same launch.
  const uint64_t stamp = ++check_stamp_;
  for (const StepItem& it : step_) {
    if (it.request->seen_in_check == stamp)
      throw Error(kBadValue, "request " + std::to_string(it.request->handle) + " appears twice in one step");
    it.request->seen_in_check = stamp;
  }
  for (const StepItem& it : step_) {
    const Request* r = it.request;
    if (it.count < 1) throw Error(kBadValue, "an item needs at least one token");
    if (it.start < 0) throw Error(kBadValue, "item starts at negative position " + std::to_string(it.start));
    // Positions between the computed ones and the item's first would hold whatever the page's owner before left there,
    // and every later token would see them under the causal mask.
    if (it.start > r->num_computed)
      throw Error(kBadValue, "item starts at position " + std::to_string(it.start) + " but only " +
                                 std::to_string(r->num_computed) + " tokens of its request are computed: a step may not leave a gap");
    if (it.start + it.count > r->size()) throw Error(kBadValue, "an item reaches beyond its request's tokens");
    if (it.start + it.count > config_.max_model_len)
      throw Error(kBadValue, "item reaches position " + std::to_string(it.start + it.count) + ", beyond the limit of " +
                                 std::to_string(config_.max_model_len));
    for (int i = it.start; i < it.start + it.count; ++i)
      if (r->tokens[i] < 0 || r->tokens[i] >= vocab_size)
        throw Error(kBadValue, "token id " + std::to_string(r->tokens[i]) + " is outside the vocabulary of " +
                                   std::to_string(vocab_size));
    for (int w : it.want)
      if (w < 0 || w >= it.count)
        throw Error(kBadValue, "wanted place " + std::to_string(w) + " is outside the item's " + std::to_string(it.count) +
                                   " tokens");
    const int need = blocks_for(it.start + it.count);
    for (size_t g = 0; g < pools_.size(); ++g) {
      const std::vector<int32_t>* table = g < r->tables.size() ? &r->tables[g] : nullptr;
      const int have = table ? (int)table->size() : 0;
      if (have < need)
        throw Error(kBadValue, "block table of group " + std::to_string(g) + " has " + std::to_string(have) + " pages, " +
                                   std::to_string(need) + " are needed");
      if (!scan_pages) continue;
      const int w = config_.groups[g].window;
      const int first_key = w > 0 ? std::max(0, it.start - w + 1) : 0;
      for (int i = first_key / bs; i < need; ++i)
        if ((*table)[i] < 0)
          throw Error(kBadValue, "group " + std::to_string(g) + ": a page the step reads or writes was already given back");
    }
  }
}

// Layout of the current step. Without `widths` every table is as wide as the step's longest;
// `pad_items` one-token items that write to the spare page follow the step's own.
StepLayout Core::layout(const std::vector<int>* widths, int pad_items) const {
  int tokens = pad_items, rows = pad_items;
  std::vector<int> w(pools_.size(), 1);
  for (const StepItem& it : step_) {
    tokens += it.count;
    rows += (int)it.want.size();
    for (size_t g = 0; g < pools_.size() && g < it.request->tables.size(); ++g)
      w[g] = std::max(w[g], (int)it.request->tables[g].size());
  }
  return StepLayout::make(tokens, (int)step_.size() + pad_items, rows, widths ? *widths : w);
}

// What the kernels of a step may want to know of it beside its indices. Bit 0: a quarter or more of the keys that the
// step's items read lie in pages that came out of the prefix cache, pages that other items read too: decode attention
// then loads keys and values so that they stay in the caches (ordinary loads), not as data that passes through once.
int Core::step_flags() const {
  long long cached = 0, keys = 0;
  for (const StepItem& it : step_) {
    const int ctx = it.start + it.count;
    keys += ctx;
    cached += std::min(it.request->num_cached, ctx);
  }
  return cached > 0 && 4 * cached >= keys ? 1 : 0;
}

void Core::pack(int32_t* dst, const StepLayout& lay, int spare_page, int spare_slot) const {
  std::fill(dst, dst + lay.total, 0);
  std::fill_n(dst + lay.token_source, lay.tokens, -1);
  const int live = (int)step_.size();
  int cursor = 0, row = 0;
  for (int i = 0; i < lay.items; ++i) {
    dst[lay.item_start + i] = cursor;
    if (i >= live) {  // padding: a one-token item at position 0 of the spare page
      dst[lay.token_item + cursor] = i;
      dst[lay.want_rows + row++] = cursor;
      dst[lay.item_ctx + i] = 1;
      dst[lay.state_slots + i] = spare_slot;
      for (size_t g = 0; g < lay.widths.size(); ++g)
        std::fill_n(dst + lay.tables[g] + (size_t)i * lay.widths[g], lay.widths[g], spare_page);
      ++cursor;
      continue;
    }
    const StepItem& it = step_[i];
    const Request* r = it.request;
    for (int j = 0; j < it.count; ++j) {
      dst[lay.token_ids + cursor + j] = r->tokens[it.start + j];
      dst[lay.positions + cursor + j] = it.start + j;
      dst[lay.token_item + cursor + j] = i;
      if (r->pending && it.start + j + 1 == r->size()) dst[lay.token_source + cursor + j] = r->fed_row;
    }
    for (int w : it.want) {
      // a wanted place that is the request's last token is where the next token is drawn from
      if (it.start + w + 1 == r->size()) {
        memcpy(dst + lay.temperatures + row, &r->temperature, 4);
        const uint64_t key = draw_key(r);
        memcpy(dst + lay.sample_keys + 2 * row, &key, 8);
      }
      dst[lay.want_rows + row++] = cursor + w;
    }
    dst[lay.item_ctx + i] = it.start + it.count;
    dst[lay.state_slots + i] = r->state_slot >= 0 ? r->state_slot : spare_slot;
    for (size_t g = 0; g < lay.widths.size(); ++g) {
      int32_t* out = dst + lay.tables[g] + (size_t)i * lay.widths[g];
      std::fill_n(out, lay.widths[g], spare_page);
      if (g < r->tables.size()) {
        if ((int)r->tables[g].size() > lay.widths[g]) throw Error(kBadValue, "a block table is wider than the step's buffer");
        std::copy(r->tables[g].begin(), r->tables[g].end(), out);
      }
    }
    cursor += it.count;
  }
  dst[lay.item_start + lay.items] = cursor;
  dst[lay.live_items] = live;
  dst[lay.live_items + 1] = step_flags();
}

// The indices of a decode-only step written into a buffer that still holds those of the last step
// replayed from it (the pinned source of a captured graph's index buffer). Token, position, length,
// slot and sampling inputs of every row are written anew. A row of a block table is only extended by
// the pages its request has gained when the row held the same request's table last time and nothing
// but appended pages has changed it since (table_epoch); tables of window groups, whose entries
// change as pages are given back, are written whole. The pages a row gains are checked as they are
// written. Rows beyond the step's items point at the spare page and slot.
void Core::refill(int32_t* dst, const StepLayout& lay, std::vector<RowMemo>& rows, int spare_page, int spare_slot) const {
  const int live = (int)step_.size(), bucket = lay.items;
  const int bs = config_.block_size;
  if (live > bucket || lay.tokens != bucket || lay.rows != bucket) throw Error(kBadValue, "the step does not fit the bucket");
  rows.resize(bucket);
  for (int i = 0; i < bucket; ++i) {
    const bool is_live = i < live;
    const StepItem* it = is_live ? &step_[i] : nullptr;
    if (is_live && (it->count != 1 || it->want.size() != 1)) throw Error(kBadValue, "a replayed step decodes one token per item");
    const Request* r = is_live ? it->request : nullptr;
    dst[lay.token_ids + i] = is_live ? r->tokens[it->start] : 0;
    dst[lay.positions + i] = is_live ? it->start : 0;
    dst[lay.item_ctx + i] = is_live ? it->start + 1 : 1;
    dst[lay.token_source + i] = is_live && r->pending && it->start + 1 == r->size() ? r->fed_row : -1;
    dst[lay.state_slots + i] = is_live && r->state_slot >= 0 ? r->state_slot : spare_slot;
    float temperature = 0.f;
    uint64_t key = 0;
    if (is_live && it->start + 1 == r->size()) {
      temperature = r->temperature;
      key = draw_key(r);
    }
    memcpy(dst + lay.temperatures + i, &temperature, 4);
    memcpy(dst + lay.sample_keys + 2 * i, &key, 8);
    RowMemo& memo = rows[i];
    if (!is_live) {
      if (memo.handle != -1 || memo.written.empty()) {  // also a row whose last refill threw half-way (-2)
        for (size_t g = 0; g < lay.widths.size(); ++g)
          std::fill_n(dst + lay.tables[g] + (size_t)i * lay.widths[g], lay.widths[g], spare_page);
        memo.handle = -1;
        memo.written.assign(lay.widths.size(), 0);
      }
      continue;
    }
    const bool same = memo.handle == r->handle && memo.epoch == r->table_epoch && memo.written.size() == lay.widths.size();
    std::vector<int> written = same ? memo.written : std::vector<int>(lay.widths.size(), 0);
    memo.handle = -2;  // until the row is complete, should a check below throw
    const int need = it->start / bs + 1;
    for (size_t g = 0; g < lay.widths.size(); ++g) {
      const std::vector<int32_t>& table = r->tables[g];
      const int width = lay.widths[g], window = config_.groups[g].window;
      if ((int)table.size() > width) throw Error(kBadValue, "a block table is wider than the graph's buffer");
      int32_t* out = dst + lay.tables[g] + (size_t)i * width;
      int have = same && window == 0 ? written[g] : -1;
      if (have < 0) {
        std::fill_n(out, width, spare_page);
        have = 0;
      }
      const int first_key = window > 0 ? std::max(0, it->start - window + 1) : 0;
      for (int p = std::max(have, first_key / bs); p < need; ++p)
        if (table[p] < 0)
          throw Error(kBadValue, "group " + std::to_string(g) + ": a page the step reads or writes was already given back");
      if (have < (int)table.size()) {
        std::copy(table.begin() + have, table.end(), out + have);
        written[g] = (int)table.size();
      }
    }
    memo.handle = r->handle;
    memo.epoch = r->table_epoch;
    memo.written = written;
  }
  dst[lay.live_items] = live;
  dst[lay.live_items + 1] = step_flags();
}

}  // namespace me
