// The host side of the engine that holds no tensors: requests, page pools with prefix digests and an
// eviction order, slots for fixed-size per-request state, the continuous-batching scheduler, and the
// packing of a step's indices into the one int32 buffer the kernels read.
//
// Behaviour follows the reference's src/mini_engine/block_manager.py, scheduler.py and sequence.py
// (cited where a rule is taken from them); the structure is this engine's own: pages are arrays
// indexed by page id with an intrusive list for the eviction order, requests are owned by the core
// and named by integer handles, and a step is a list the scheduler or a trace fills before it is
// checked and packed.
#pragma once

#include <stdint.h>
#include <string.h>

#include <deque>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace me {

// Errors cross the C boundary as a code and a message; the Python side raises by code.
enum ErrorKind { kOk = 0, kBadValue = 1, kBadState = 2, kBroken = 3 };
struct Error : std::runtime_error {
  ErrorKind kind;
  Error(ErrorKind k, const std::string& what) : std::runtime_error(what), kind(k) {}
};

// ------------------------------------------------------------------------------------- digests
struct Digest {
  uint8_t bytes[16];
  bool operator==(const Digest& o) const { return memcmp(bytes, o.bytes, 16) == 0; }
};
struct DigestHasher {
  size_t operator()(const Digest& d) const {
    uint64_t x;
    memcpy(&x, d.bytes, 8);
    return (size_t)x;
  }
};
// blake2b-128 over the parent's digest (nothing for the first block) followed by every token id as
// four little-endian bytes: equal digests mean equal whole prefixes (reference block_manager.py:26-35).
Digest chain_digest(const uint8_t* parent, size_t parent_len, const int32_t* tokens, int count);

// --------------------------------------------------------------------------------------- pages
// The pages of one cache group. A page has a count of holders; pages without holders stand in the
// free order, from which new pages are taken at the front. A page may carry the digest of the
// token prefix whose keys it holds; it keeps digest and content while it waits in the free order
// and loses both only when it is taken for new content.
class PagePool {
 public:
  explicit PagePool(int num_pages);
  int num_pages() const { return (int)holders_.size(); }
  int num_free() const { return free_count_; }
  int holders(int page) const { return holders_[page]; }
  bool has_digest(int page) const { return has_digest_[page] != 0; }
  const Digest& digest(int page) const { return digest_[page]; }
  long evictions() const { return evictions_; }
  int find(const Digest& d) const;
  int take();
  void retain(int page);
  void release(int page);
  bool publish(int page, const Digest& d);
  void forget_digests();
  std::vector<int32_t> free_order() const;

 private:
  void link_back(int page);
  void link_front(int page);
  void unlink(int page);
  std::vector<int32_t> holders_;
  std::vector<uint8_t> has_digest_;
  std::vector<Digest> digest_;
  std::unordered_map<Digest, int32_t, DigestHasher> by_digest_;
  // the free order as a list threaded through two arrays; index num_pages is the list's head cell
  std::vector<int32_t> next_, prev_;
  std::vector<uint8_t> listed_;
  int free_count_ = 0;
  long evictions_ = 0;
};

class StateSlots {
 public:
  explicit StateSlots(int count);
  int count() const { return (int)taken_.size(); }
  int num_free() const { return (int)spare_.size(); }
  bool taken(int slot) const { return taken_[slot] != 0; }
  int take();  // -1 when none is left
  void give_back(int slot);

 private:
  std::vector<int32_t> spare_;
  std::vector<uint8_t> taken_;
};

// ------------------------------------------------------------------------------------ requests
enum RequestPhase { kWaiting = 0, kRunning = 1, kFinished = 2 };

struct Request {
  int64_t handle = -1;
  int64_t serial = -1;  // order of creation within this core: what sampling keys are made from
  std::vector<int32_t> tokens;  // prompt, then what was generated
  int num_prompt = 0;
  int num_computed = 0;  // tokens [0, num_computed) have keys and values in the pages of `tables`
  int phase = kWaiting;
  std::vector<std::vector<int32_t>> tables;  // one per cache group; -1: a page a window has passed
  std::vector<Digest> chain;                 // digests of the full blocks computed so far
  uint32_t table_epoch = 0;  // counts changes of `tables` other than appended pages
  int state_slot = -1;
  int num_cached = 0;       // tokens found in the prefix cache at the last admission
  int num_preemptions = 0;
  int max_tokens = 64;
  float temperature = 0.f;
  bool ignore_eos = false;
  bool held = true;  // a Python object still names this request
  // While a step is in flight whose draw for this request the host has not read yet: the last of `tokens` is a
  // stand-in for that draw, which a step planned ahead feeds from row `fed_row` of the draws on the device.
  bool pending = false;
  int fed_row = -1;
  mutable uint64_t seen_in_check = 0;  // the last check of a step that met this request (finds one named twice)

  int size() const { return (int)tokens.size(); }
  int uncomputed() const { return size() - num_computed; }
  int num_output() const { return size() - num_prompt; }
};

struct GroupConfig {
  int window = 0;  // 0: every key stays needed; w: a query sees the last w keys
  int num_pages = 0;
};

struct CoreConfig {
  int block_size = 16;
  std::vector<GroupConfig> groups;
  bool prefix_caching = true;
  int num_state_slots = 0;
  bool has_state = false;  // some layer keeps per-request state: no prefix hits then
  int max_num_seqs = 16;
  int max_num_batched_tokens = 2048;
  int max_model_len = 4096;
  std::vector<int32_t> eos_ids;
  uint64_t seed = 0;
};

// ------------------------------------------------------------------------------------ one step
struct StepItem {
  Request* request;
  int start;   // position of the first token of this step
  int count;   // how many of the request's tokens it runs
  std::vector<int32_t> want;  // places among them whose logits are wanted
};

// Offsets (in int32 units) of the sections of a packed step buffer.
struct StepLayout {
  int tokens = 0, items = 0, rows = 0;
  std::vector<int> widths;
  int token_ids = 0, positions = 0, token_item = 0, want_rows = 0, item_start = 0, item_ctx = 0, state_slots = 0,
      live_items = 0, temperatures = 0, sample_keys = 0, token_source = 0;
  std::vector<int> tables;
  int total = 0;
  static StepLayout make(int tokens, int items, int rows, const std::vector<int>& widths);
};

// What the refill of a replayed graph's buffer remembers of a row: whose table it holds and how far.
struct RowMemo {
  int64_t handle = -1;
  uint32_t epoch = 0;
  std::vector<int> written;
};

class Core {
 public:
  explicit Core(const CoreConfig& config);
  const CoreConfig& config() const { return config_; }
  void set_limits(int max_num_seqs, int max_num_batched_tokens, int max_model_len, const std::vector<int32_t>& eos) {
    config_.max_num_seqs = max_num_seqs;
    config_.max_num_batched_tokens = max_num_batched_tokens;
    config_.max_model_len = max_model_len;
    config_.eos_ids = eos;
  }

  // requests
  Request* create(const int32_t* tokens, int count, int max_tokens, float temperature, bool ignore_eos);
  Request* get(int64_t handle) const;
  void unhold(int64_t handle);

  // pages (the reference's block manager, over several groups)
  int num_groups() const { return (int)pools_.size(); }
  PagePool& pool(int g) { return pools_[g]; }
  StateSlots* slots() { return slots_.get(); }
  bool caching() const { return caching_; }
  int blocks_for(int tokens) const { return (tokens + config_.block_size - 1) / config_.block_size; }
  int num_free_pages() const;
  long evictions() const;
  bool can_ever_hold(int tokens) const;
  int match(const int32_t* tokens, int count, std::vector<std::vector<int32_t>>& hits) const;
  bool grow(Request* r, int num_tokens, const std::vector<std::vector<int32_t>>* hits = nullptr);
  void drop(Request* r);
  int drop_passed(Request* r);
  void note_computed(Request* r);
  void forget_digests();

  // scheduler
  void enqueue(Request* r);
  bool unfinished() const { return !waiting_.empty() || !running_.empty() || !in_flight_.empty(); }
  int plan();  // fills step() from the queues; returns the number of items
  int settle(const int32_t* next_tokens, int count, std::vector<int64_t>& finished);
  // One step ahead: see scheduler.cpp.
  int plan_ahead();
  int settle_in_flight(const int32_t* drawn, int count, std::vector<int64_t>& finished);
  bool has_in_flight() const { return !in_flight_.empty(); }
  const std::deque<Request*>& waiting() const { return waiting_; }
  const std::vector<Request*>& running() const { return running_; }
  long preemptions = 0, cached_tokens = 0, generated = 0;  // generated: tokens appended to requests by draws

  // the step under construction / last planned
  std::vector<StepItem>& step() { return step_; }
  void check_step(int vocab_size, bool scan_pages) const;
  StepLayout layout(const std::vector<int>* widths, int pad_items) const;
  int step_flags() const;
  void pack(int32_t* dst, const StepLayout& lay, int spare_page, int spare_slot) const;
  void refill(int32_t* dst, const StepLayout& lay, std::vector<RowMemo>& rows, int spare_page, int spare_slot) const;
  uint64_t draw_key(const Request* r) const;

 private:
  void evict(Request* r);
  bool done(const Request* r, int32_t token) const;
  CoreConfig config_;
  std::vector<PagePool> pools_;
  std::unique_ptr<StateSlots> slots_;
  bool caching_ = false;
  std::unordered_map<int64_t, std::unique_ptr<Request>> requests_;
  int64_t next_handle_ = 0;
  std::deque<Request*> waiting_;
  std::vector<Request*> running_;
  std::vector<StepItem> step_;
  mutable uint64_t check_stamp_ = 0;
  std::vector<StepItem> in_flight_;  // the step launched before step_ whose draws are not settled yet
  void reap(Request* r);
  void finish(Request* r, std::vector<int64_t>& finished);
};

// The core inside the box that the C functions of api.cpp hand out.
Core* core_in_box(void* box);

}  // namespace me
