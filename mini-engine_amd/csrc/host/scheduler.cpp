// Requests and the continuous-batching scheduler of the core.
//
// Each step has a budget of tokens that decoded tokens and portions of prompts share. Requests that
// are already running come first, in the order they were admitted; then waiting requests are
// admitted first come first served (reference scheduler.py:65-103). A whole prompt, a portion of
// one, a decoded token and the recomputation after a preemption are all "the next n tokens from
// num_computed on".
#include "core.h"

#include <algorithm>

namespace me {

Request* Core::create(const int32_t* tokens, int count, int max_tokens, float temperature, bool ignore_eos) {
  if (count < 1) throw Error(kBadValue, "prompt must contain at least one token");
  if (max_tokens < 1) throw Error(kBadValue, "max_tokens must be >= 1");
  if (!(temperature >= 0.f)) throw Error(kBadValue, "temperature must be >= 0");
  std::unique_ptr<Request> r(new Request);
  r->handle = r->serial = next_handle_++;
  r->tokens.assign(tokens, tokens + count);
  r->num_prompt = count;
  r->tables.resize(pools_.size());
  r->max_tokens = max_tokens;
  r->temperature = temperature;
  r->ignore_eos = ignore_eos;
  Request* raw = r.get();
  requests_.emplace(raw->handle, std::move(r));
  return raw;
}

Request* Core::get(int64_t handle) const {
  auto it = requests_.find(handle);
  if (it == requests_.end()) throw Error(kBadValue, "no request with handle " + std::to_string(handle));
  return it->second.get();
}

// A request's record lives while a Python object names it or a queue holds it.
void Core::reap(Request* r) {
  if (r->held) return;
  if (r->phase == kRunning) return;
  if (std::find(waiting_.begin(), waiting_.end(), r) != waiting_.end()) return;
  for (const StepItem& it : step_)
    if (it.request == r) return;
  for (const StepItem& it : in_flight_)
    if (it.request == r) return;
  drop(r);
  requests_.erase(r->handle);
}

void Core::unhold(int64_t handle) {
  auto it = requests_.find(handle);
  if (it == requests_.end()) return;
  it->second->held = false;
  reap(it->second.get());
}

// A request that could never run to its end is refused when it is added, not starved later
// (reference scheduler.py:54-60).
void Core::enqueue(Request* r) {
  const int longest = r->size() + r->max_tokens;
  if (longest > config_.max_model_len)
    throw Error(kBadValue, "prompt + max_tokens = " + std::to_string(longest) + " exceeds max_model_len");
  if (!can_ever_hold(longest))
    throw Error(kBadValue, "request needs more than the " + std::to_string(pools_[0].num_pages()) + " KV blocks available");
  r->phase = kWaiting;
  waiting_.push_back(r);
}

// Recompute preemption: the request gives back its pages and its slot, keeps its tokens (generated
// ones too) and goes to the head of the waiting queue; when it is admitted again the prefix cache
// usually still has most of its blocks (reference scheduler.py:150-159).
void Core::evict(Request* r) {
  running_.erase(std::find(running_.begin(), running_.end(), r));
  drop(r);
  r->phase = kWaiting;
  r->num_computed = 0;
  ++r->num_preemptions;
  ++preemptions;
  waiting_.push_front(r);
}

int Core::plan() {
  if (!in_flight_.empty()) throw Error(kBadState, "a step is in flight: settle it before the next one is planned from the queues");
  step_.clear();
  int budget = config_.max_num_batched_tokens;
  bool memory_was_tight = false;

  // Running requests. One that cannot get its pages makes the request admitted last give up
  // everything, again and again until it fits or is the last itself; then it waits for the next step.
  // The request admitted last stands behind every request this loop has reached, so nothing that is
  // already part of the step is ever evicted.
  size_t at = 0;
  while (at < running_.size() && budget > 0) {
    Request* r = running_[at];
    const int n = std::min(r->uncomputed(), budget);
    bool fits = grow(r, r->num_computed + n);
    while (!fits) {
      Request* last = running_.back();
      evict(last);
      memory_was_tight = true;
      if (last == r) break;
      fits = grow(r, r->num_computed + n);
    }
    if (!fits) break;  // r was the last one and is waiting now
    StepItem item{r, r->num_computed, n, {}};
    if (r->num_computed + n == r->size()) item.want.push_back(n - 1);
    step_.push_back(std::move(item));
    budget -= n;
    ++at;
  }

  // Waiting requests, in order, each with what the prefix cache has of it; none in a step that had to
  // evict, and none past one that does not fit (no queue jumping). Pages are taken for the portion
  // of this step only.
  std::vector<std::vector<int32_t>> hits;
  while (!memory_was_tight && !waiting_.empty() && budget > 0 && (int)running_.size() < config_.max_num_seqs) {
    Request* r = waiting_.front();
    const int hit_tokens = match(r->tokens.data(), r->size(), hits) * config_.block_size;
    const int n = std::min(r->size() - hit_tokens, budget);
    if (!grow(r, hit_tokens + n, &hits)) break;
    waiting_.pop_front();
    r->phase = kRunning;
    r->num_computed = r->num_cached = hit_tokens;
    cached_tokens += hit_tokens;
    running_.push_back(r);
    StepItem item{r, hit_tokens, n, {}};
    if (hit_tokens + n == r->size()) item.want.push_back(n - 1);
    step_.push_back(std::move(item));
    budget -= n;
  }
  return (int)step_.size();
}

bool Core::done(const Request* r, int32_t token) const {
  if (!r->ignore_eos && std::find(config_.eos_ids.begin(), config_.eos_ids.end(), token) != config_.eos_ids.end())
    return true;  // the end token stays in the output
  return r->num_output() >= r->max_tokens;
}

void Core::finish(Request* r, std::vector<int64_t>& finished) {
  r->phase = kFinished;
  drop(r);
  running_.erase(std::find(running_.begin(), running_.end(), r));
  finished.push_back(r->handle);
}

// After the model ran the planned step: next_tokens[i] is the token sampled for item i, or negative
// for a portion that did not reach its request's last token (reference scheduler.py:107-123). An item
// of a step planned ahead whose request ended with the draw before it is passed over: its token was
// computed for nothing.
int Core::settle(const int32_t* next_tokens, int count, std::vector<int64_t>& finished) {
  if (count != (int)step_.size()) throw Error(kBadValue, "one token (or none) per scheduled sequence is needed");
  if (!in_flight_.empty()) throw Error(kBadState, "the step before this one is still in flight: settle it first");
  finished.clear();
  std::vector<StepItem> items;
  items.swap(step_);
  for (int i = 0; i < count; ++i) {
    Request* r = items[i].request;
    if (r->phase == kFinished) continue;
    r->num_computed += items[i].count;
    note_computed(r);
    drop_passed(r);
    if (next_tokens[i] < 0) continue;
    r->tokens.push_back(next_tokens[i]);
    ++generated;
    if (done(r, next_tokens[i])) finish(r, finished);
  }
  for (const StepItem& it : items) reap(it.request);
  return (int)finished.size();
}

// One step ahead. The planned step has been launched and its draws are still on the device. When it decodes
// one token for every running request and no waiting request could be admitted, the step after it is known
// but for the token ids: every request that cannot end by its count of tokens decodes the token it is about
// to draw. plan_ahead() makes the launched step the one in flight (its requests advance as settle() would
// advance them, with a stand-in for the unknown token) and plans that next step, whose token ids the device
// takes from the draws of the step in flight (`fed_row`). Returns its number of items, or 0 when nothing was
// changed: the caller then settles and plans as usual. The pages every request needs are taken first, so
// nothing is evicted on the way. A request that ends with the draw in flight (an end token) has run one token
// too many in the step planned ahead; settle() passes it over.
int Core::plan_ahead() {
  if (!in_flight_.empty()) throw Error(kBadState, "a step is in flight already");
  if (step_.empty() || step_.size() != running_.size()) return 0;
  if (!waiting_.empty() && (int)running_.size() < config_.max_num_seqs) return 0;
  std::vector<int> goes_on;
  for (size_t i = 0; i < step_.size(); ++i) {
    const StepItem& it = step_[i];
    const Request* r = it.request;
    if (it.count != 1 || it.want.size() != 1 || it.want[0] != 0 || it.start + 1 != r->size() || r->pending ||
        r->phase != kRunning)
      return 0;
    if (r->num_output() + 1 < r->max_tokens && r->size() + 1 <= config_.max_model_len) goes_on.push_back((int)i);
  }
  if (goes_on.empty()) return 0;
  for (int i : goes_on)
    if (!grow(step_[i].request, step_[i].request->size() + 1)) return 0;
  in_flight_.swap(step_);
  for (StepItem& it : in_flight_) {
    Request* r = it.request;
    r->num_computed += 1;
    note_computed(r);
    drop_passed(r);
  }
  for (int i : goes_on) {
    Request* r = in_flight_[i].request;
    r->tokens.push_back(0);
    r->pending = true;
    r->fed_row = i;
    step_.push_back(StepItem{r, r->size() - 1, 1, {0}});
  }
  return (int)step_.size();
}

// The draws of the step in flight, one per item in the order of its rows: stand-ins become tokens, requests
// end as in settle(). The step planned ahead stays planned.
int Core::settle_in_flight(const int32_t* drawn, int count, std::vector<int64_t>& finished) {
  if (count != (int)in_flight_.size()) throw Error(kBadValue, "one token per item of the step in flight is needed");
  finished.clear();
  std::vector<StepItem> items;
  items.swap(in_flight_);
  for (int i = 0; i < count; ++i) {
    Request* r = items[i].request;
    if (r->pending) {
      r->tokens.back() = drawn[i];
      r->pending = false;
      r->fed_row = -1;
    } else {
      r->tokens.push_back(drawn[i]);
    }
    ++generated;
    if (done(r, drawn[i])) finish(r, finished);
  }
  for (const StepItem& it : items) reap(it.request);
  return (int)finished.size();
}

}  // namespace me
