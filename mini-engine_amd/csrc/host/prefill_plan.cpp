// The work list of a step's prefill attention: which tile of query tokens meets which range of keys,
// and which block runs which entries. It depends on the step's items and on the attention's geometry
// (heads, window), not on the layer, so a step builds it once for all layers of a kind.
#include "prefill_plan.h"

#include <algorithm>
#include <functional>
#include <queue>

namespace me {

namespace {

constexpr int kPieceOverhead = 2;  // what starting another piece of work costs a block, in key tiles (3 us against 1.5)
constexpr int kCutOverhead = 8;    // what cutting any tile costs a step, in key tiles: partial results written and the kernel that
                                   // adds them up (one prompt of 65 to 384 tokens: a step 8% longer with cut tiles than without,
                                   // 512: 3%, 768: the same, 1,024: 2% shorter, 2,048: 5% shorter)
constexpr long long kPartialBytesMax = 256ll << 20;  // most memory the partial results of cut tiles may take

struct Tile {
  int item, first_token, tokens, first_pos, first_key, last_pos, key_tiles;
};
struct Piece {
  int length, tile, chunk, first_tile;  // chunk -1: the tile in one piece
};

// Pieces of tiles cut into ranges of at most `cap` key tiles: full ranges first, the remainder last (small
// remainders fill the gaps beside long pieces).
std::vector<Piece> cut(const std::vector<Tile>& tiles, int cap) {
  std::vector<Piece> pieces;
  for (int i = 0; i < (int)tiles.size(); ++i) {
    const int n = tiles[i].key_tiles;
    if (n <= cap) {
      pieces.push_back({n, i, -1, 0});
      continue;
    }
    int j = 0;
    for (int t0 = 0; t0 < n; t0 += cap, ++j) pieces.push_back({std::min(cap, n - t0), i, j, t0});
  }
  return pieces;
}

// Longest piece first into the least loaded bin; returns the longest bin's load.
long long pack(std::vector<Piece> pieces, int bins, std::vector<std::vector<Piece>>& loads) {
  std::stable_sort(pieces.begin(), pieces.end(), [](const Piece& a, const Piece& b) { return a.length > b.length; });
  typedef std::pair<long long, int> Bin;  // (load, index): the smallest load first, the lowest index among equals
  std::priority_queue<Bin, std::vector<Bin>, std::greater<Bin>> heap;
  for (int b = 0; b < bins; ++b) heap.push({0, b});
  loads.assign(bins, {});
  long long span = 0;
  for (const Piece& p : pieces) {
    Bin bin = heap.top();
    heap.pop();
    loads[bin.second].push_back(p);
    bin.first += p.length + kPieceOverhead;
    span = std::max(span, bin.first);
    heap.push(bin);
  }
  return span;
}

}  // namespace

// Blocks of twice as many query columns read each key and value tile once for twice the work, but a step
// has half as many of them. They are taken when every compute unit still gets a whole one, or when the
// step has so many key tiles to walk that tiles are cut into key ranges anyway (measured on 256 compute
// units: from 4,096 tokens of whole prompts on, or a 2,048-token portion behind 2,048 tokens, 8-24%
// faster; three prompts of 1,024 tokens, a third slower); not when the wide blocks would be a third
// emptier than the narrow ones (many items of few tokens).
static double g_wide_min_blocks = 1.0, g_wide_min_key_tiles = 20.0;  // per compute unit

bool wide_blocks_pay(const int* starts, const int* qlens, int items, int tpb, int window, int nkv, int slots) {
  const int half = std::max(1, tpb / 2);
  long long wide_fill = 0, narrow_fill = 0;
  for (int i = 0; i < items; ++i) {
    wide_fill += (long long)((qlens[i] + tpb - 1) / tpb) * tpb;
    narrow_fill += (long long)((qlens[i] + half - 1) / half) * half;
  }
  if (3 * wide_fill > 4 * narrow_fill) return false;
  long long blocks = 0, key_tiles = 0;
  for (int i = 0; i < items; ++i)
    for (int t0 = 0; t0 < qlens[i]; t0 += tpb) {
      const int last = starts[i] + std::min(t0 + tpb, qlens[i]) - 1;
      const int first = window > 0 ? std::max(0, starts[i] + t0 - window + 1) : 0;
      ++blocks;
      key_tiles += last / 64 - first / 64 + 1;
    }
  return blocks * nkv >= g_wide_min_blocks * slots || key_tiles * nkv >= g_wide_min_key_tiles * slots;
}

// A tile of `tpb` query tokens of an item meets the keys from its window's first (rounded down to a
// multiple of 64) to its last token's position: n key tiles of 64. A bundle of entries is run by one
// block per kv head. With more tiles than compute units per kv head the bundles are the tiles, longest
// first (the hardware starts blocks in that order and evens them out). With at most that many (a prompt of
// up to a few thousand tokens, whose causal tiles differ in length by a factor of their number; a short
// portion over a long context) the tiles are cut into ranges of at most `cap` key tiles, whose partial
// results a second kernel adds up, and the pieces are packed into one bundle per compute unit; `cap` is
// the candidate with the shortest longest bundle, where cutting at all counts as kCutOverhead key tiles.
void build_work_list(const int* starts, const int* qlens, int items, int tpb, int window, int nkv, int slots,
                     long long partial_row_bytes, WorkList& out) {
  std::vector<Tile> tiles;
  int offset = 0;
  for (int i = 0; i < items; ++i) {
    for (int t0 = 0; t0 < qlens[i]; t0 += tpb) {
      const int count = std::min(tpb, qlens[i] - t0);
      const int p_first = starts[i] + t0, p_last = p_first + count - 1;
      const int k0 = window > 0 ? (std::max(p_first - window + 1, 0) / 64) * 64 : 0;
      tiles.push_back({i, offset + t0, count, p_first, k0, p_last, (p_last - k0) / 64 + 1});
    }
    offset += qlens[i];
  }
  const int bins = std::max(1, slots / std::max(1, nkv));
  int longest = 0;
  long long total = 0;
  for (const Tile& t : tiles) {
    longest = std::max(longest, t.key_tiles);
    total += t.key_tiles;
  }
  std::vector<std::vector<Piece>> bundles;
  if ((int)tiles.size() > bins) {
    std::vector<Piece> whole = cut(tiles, longest);
    std::stable_sort(whole.begin(), whole.end(), [](const Piece& a, const Piece& b) { return a.length > b.length; });
    for (const Piece& p : whole) bundles.push_back({p});
  } else {
    long long chunk_limit = 1ll << 30;
    if (partial_row_bytes > 0) chunk_limit = std::max(1ll, kPartialBytesMax / (partial_row_bytes * std::max(1, offset)));
    std::vector<int> caps = {longest, (int)((total + bins - 1) / bins), (int)((total + 2ll * bins - 1) / (2ll * bins)),
                             (longest + 1) / 2, (longest + 2) / 3};
    std::sort(caps.begin(), caps.end());
    caps.erase(std::unique(caps.begin(), caps.end()), caps.end());
    bool have = false;
    double best_score = 0;
    int best_cap = 0;
    std::vector<std::vector<Piece>> best;
    for (int cap : caps) {
      if (cap < 1 || (longest + cap - 1) / cap > chunk_limit) continue;
      std::vector<Piece> pieces = cut(tiles, cap);
      std::vector<std::vector<Piece>> loads;
      const double score = (double)pack(pieces, bins, loads) + (cap < longest ? kCutOverhead : 0) + 0.01 * (double)pieces.size();
      if (!have || score < best_score || (score == best_score && cap < best_cap)) {
        have = true;
        best_score = score;
        best_cap = cap;
        best.swap(loads);
      }
    }
    for (auto& b : best)
      if (!b.empty()) bundles.push_back(std::move(b));
    auto load = [](const std::vector<Piece>& b) {
      long long s = 0;
      for (const Piece& p : b) s += p.length;
      return s;
    };
    std::stable_sort(bundles.begin(), bundles.end(),
                     [&](const std::vector<Piece>& a, const std::vector<Piece>& b) { return load(a) > load(b); });
  }
  out.token_chunks.assign(offset, 1);
  std::vector<int> chunks_of(tiles.size(), 1);
  for (const auto& bundle : bundles)
    for (const Piece& p : bundle) chunks_of[p.tile] = std::max(chunks_of[p.tile], p.chunk + 1);
  out.work.clear();
  out.bundle_first.clear();
  for (const auto& bundle : bundles) {
    out.bundle_first.push_back((int)out.work.size() / 8);
    for (const Piece& p : bundle) {
      const Tile& t = tiles[p.tile];
      const int row[8] = {t.item, t.first_token, t.tokens, t.first_pos, t.first_key + 64 * p.first_tile,
                          std::min(t.last_pos, t.first_key + 64 * (p.first_tile + p.length) - 1), p.chunk, 0};
      out.work.insert(out.work.end(), row, row + 8);
    }
    out.work.back() = 1;  // the bundle ends with this entry
  }
  out.max_chunks = 1;
  for (size_t i = 0; i < tiles.size(); ++i) {
    out.max_chunks = std::max(out.max_chunks, chunks_of[i]);
    if (chunks_of[i] > 1)
      std::fill(out.token_chunks.begin() + tiles[i].first_token, out.token_chunks.begin() + tiles[i].first_token + tiles[i].tokens,
                chunks_of[i]);
  }
}

}  // namespace me

extern "C" {

// For Python callers and tests: the work list as flat arrays. work takes 8 ints per entry, bundle_first one per
// bundle, token_chunks one per token; counts: entries, bundles, max chunks. Returns 0, or -1 when a buffer is
// too small (counts then say what is needed).
int me_prefill_work_list(const int32_t* starts, const int32_t* qlens, int items, int tpb, int window, int nkv, int slots,
                         long long partial_row_bytes, int32_t* work, int cap_entries, int32_t* bundle_first, int cap_bundles,
                         int32_t* token_chunks, int cap_tokens, int32_t* counts) {
  me::WorkList list;
  me::build_work_list(starts, qlens, items, tpb, window, nkv, slots, partial_row_bytes, list);
  counts[0] = (int)list.work.size() / 8;
  counts[1] = (int)list.bundle_first.size();
  counts[2] = list.max_chunks;
  if (counts[0] > cap_entries || counts[1] > cap_bundles || (int)list.token_chunks.size() > cap_tokens) return -1;
  std::copy(list.work.begin(), list.work.end(), work);
  std::copy(list.bundle_first.begin(), list.bundle_first.end(), bundle_first);
  std::copy(list.token_chunks.begin(), list.token_chunks.end(), token_chunks);
  return 0;
}

// The two limits of wide_blocks_pay (blocks and key tiles per compute unit), for measurements and tests that
// want one block width whatever the step: sets both, gives the old ones back through `old` (2 doubles).
void me_prefill_wide_limits(double min_blocks, double min_key_tiles, double* old) {
  if (old) {
    old[0] = me::g_wide_min_blocks;
    old[1] = me::g_wide_min_key_tiles;
  }
  me::g_wide_min_blocks = min_blocks;
  me::g_wide_min_key_tiles = min_key_tiles;
}

int me_prefill_wide_blocks_pay(const int32_t* starts, const int32_t* qlens, int items, int tpb, int window, int nkv, int slots) {
  return me::wide_blocks_pay(starts, qlens, items, tpb, window, nkv, slots) ? 1 : 0;
}

}  // extern "C"
