#include "scheduler.h"

#include <algorithm>
#include <stdexcept>

namespace mgpt {

Scheduler::Scheduler(CacheManager* cache, const SchedulerConfig& cfg) : cache_(cache), cfg_(cfg) {
  if (!cache) throw std::invalid_argument("scheduler needs a cache manager");
  if (cfg.max_batch_size <= 0 || cfg.max_num_batched_tokens <= 0 || cfg.prefill_chunk < 0 ||
      cfg.max_positions <= 0)
    throw std::invalid_argument("bad scheduler configuration");
  if (cfg.max_batch_size > cache->max_requests())
    throw std::invalid_argument("max_batch_size exceeds the cache manager's request slots");
  if (cfg.max_num_batched_tokens < cfg.max_batch_size)
    throw std::invalid_argument("max_num_batched_tokens must cover one decode token per running request");
}

Request* Scheduler::get(int id) {
  if (id < 0 || id >= (int)requests_.size()) return nullptr;
  return requests_[id].get();
}

const Request* Scheduler::request(int id) const {
  if (id < 0 || id >= (int)requests_.size()) return nullptr;
  return requests_[id].get();
}

int Scheduler::add_request(const int* prompt, int n_prompt, int max_tokens, int eot,
                           float temperature, int top_k, float top_p, uint64_t seed, bool has_seed) {
  if (n_prompt <= 0 || !prompt) return ERR_EMPTY_PROMPT;
  if (max_tokens <= 0 || top_k < 0 || !(top_p > 0.0f && top_p <= 1.0f)) return ERR_BAD_PARAMS;
  // src/minigpt_infer/engine/engine.py:73-88
  if (n_prompt + max_tokens > cfg_.max_positions) return ERR_TOO_LONG;
  // the last sampled token is never fed back, so prompt + max_tokens - 1 tokens are cached at most
  for (int g = 0; g < cache_->num_groups(); ++g)
    if (cache_->pages_needed(g, n_prompt + max_tokens - 1) > cache_->group(g).num_pages)
      return ERR_NEVER_FITS;
  auto r = std::make_unique<Request>();
  // the id of a forgotten request is used again, so that a scheduler that serves for a long time
  // holds as many records as it has live requests
  if (!free_ids_.empty()) {
    r->id = free_ids_.back();
    free_ids_.pop_back();
  } else {
    r->id = (int)requests_.size();
    requests_.emplace_back();
  }
  r->prompt.assign(prompt, prompt + n_prompt);
  r->max_tokens = max_tokens;
  r->eot = eot;
  r->temperature = temperature;
  r->top_k = top_k;
  r->top_p = top_p;
  r->seed = has_seed ? seed : num_added_;     // a stream of its own per arrival
  ++num_added_;
  const int id = r->id;
  requests_[id] = std::move(r);
  waiting_.push_back(id);
  return id;
}

void Scheduler::preempt(Request& r) {
  // src/minigpt_infer/engine/scheduler.py:84-90: outputs are kept, the cache is not
  cache_->free_slot(r.slot);
  r.slot = -1;
  r.num_computed = 0;
  r.status = WAITING;
  running_.erase(std::find(running_.begin(), running_.end(), r.id));
  waiting_.push_front(r.id);
  ++num_preemptions;
  preempted_this_step_ = true;
}

void Scheduler::finish(Request& r, FinishReason why) {
  // src/minigpt_infer/engine/scheduler.py:92-99: pages go back in the same step
  r.status = FINISHED;
  r.finish_reason = why;
  if (r.slot >= 0) {
    cache_->free_slot(r.slot);
    r.slot = -1;
  }
  auto it = std::find(running_.begin(), running_.end(), r.id);
  if (it != running_.end()) running_.erase(it);
}

bool Scheduler::cancel(int id) {
  // src/minigpt_infer/engine/scheduler.py:101-117
  Request* r = get(id);
  if (!r || r->status == FINISHED) return false;
  if (r->status == WAITING) {
    auto it = std::find(waiting_.begin(), waiting_.end(), id);
    if (it != waiting_.end()) waiting_.erase(it);
  }
  finish(*r, FINISH_CANCELLED);  // a planned entry of it is skipped by commit
  return true;
}

void Scheduler::ensure_capacity_for_decode() {
  // src/minigpt_infer/engine/scheduler.py:58-82
  const std::vector<int> snapshot = running_;
  for (int id : snapshot) {
    Request& r = *get(id);
    if (r.status != RUNNING) continue;  // preempted earlier in this pass
    if (r.num_tokens() - r.num_computed != 1) continue;  // still in its prompt: pages are held
    while (!cache_->reserve(r.slot, r.num_computed + 1)) {
      // Evict the newest running request.  The reference never evicts the one that asks
      // (scheduler.py:78-82 picks the newest other one), which lets a newcomer push out an older
      // request; by default the asker itself goes when it is the newest, and spare_asker brings the
      // reference's rule back (the asker then goes only when it is the last one running).
      int vid = running_.back();
      if (cfg_.spare_asker && vid == id && running_.size() > 1) vid = running_[running_.size() - 2];
      Request& victim = *get(vid);
      const bool self = victim.id == id;
      preempt(victim);
      if (self) break;
    }
  }
}

void Scheduler::schedule_decodes(int& budget) {
  for (int id : running_) {
    if (budget <= 0) break;
    Request& r = *get(id);
    if (r.num_tokens() - r.num_computed != 1) continue;
    entries_.push_back({id, r.num_computed, 1, true});
    --budget;
    ++num_decode_tokens;
  }
}

void Scheduler::schedule_prompts(int& budget, bool allow_admission) {
  auto portion = [&](const Request& r) {
    int q = r.num_tokens() - r.num_computed;
    if (cfg_.prefill_chunk > 0) q = std::min(q, cfg_.prefill_chunk);
    return std::min(q, budget);
  };
  // unfinished prompts of running requests first, in admission order
  for (int id : running_) {
    if (budget <= 0) return;
    Request& r = *get(id);
    const int remaining = r.num_tokens() - r.num_computed;
    if (remaining <= 1) continue;
    const int q = portion(r);
    entries_.push_back({id, r.num_computed, q, q == remaining});
    budget -= q;
    num_prompt_tokens += q;
  }
  if (!allow_admission) return;
  // then new requests from the head of the queue; the head blocks those behind it
  // (src/minigpt_infer/engine/scheduler.py:40-50)
  while (!waiting_.empty() && (int)running_.size() < cfg_.max_batch_size && budget > 0) {
    Request& r = *get(waiting_.front());
    if (cache_->num_free_slots() == 0 || !cache_->can_allocate(r.num_tokens())) break;
    r.slot = cache_->acquire_slot();
    cache_->reserve(r.slot, r.num_tokens());  // the whole context, so a prompt never stalls half-way
    r.status = RUNNING;
    r.num_computed = 0;
    waiting_.pop_front();
    running_.push_back(r.id);
    const int q = portion(r);
    entries_.push_back({r.id, 0, q, q == r.num_tokens()});
    budget -= q;
    num_prompt_tokens += q;
  }
}

const std::vector<StepEntry>& Scheduler::schedule() {
  if (pending_ > 0) throw std::runtime_error("schedule(): a planned burst has not been handed in yet");
  entries_.clear();
  preempted_this_step_ = false;
  int budget = cfg_.max_num_batched_tokens;
  if (cfg_.mixed) {
    ensure_capacity_for_decode();
    schedule_decodes(budget);
    // a request that was just evicted is not admitted again in the same step
    schedule_prompts(budget, !preempted_this_step_);
  } else {
    schedule_prompts(budget, true);
    if (entries_.empty()) {
      ensure_capacity_for_decode();
      schedule_decodes(budget);
    }
  }
  if (!entries_.empty()) ++num_steps;
  return entries_;
}

const std::vector<StepOutput>& Scheduler::commit(const int* tokens, int n_tokens) {
  outputs_.clear();
  int k = 0;
  const std::vector<StepEntry> entries = entries_;  // finish() edits running_, not this copy
  for (const StepEntry& e : entries) {
    Request& r = *get(e.id);
    if (r.status != RUNNING) {  // cancelled between schedule and commit
      if (e.sample) ++k;
      continue;
    }
    // the counter advances by what was written, never by the sampled token
    // (src/minigpt_infer/engine/engine.py:133-141)
    r.num_computed += e.q_len;
    cache_->release_passed(r.slot, r.num_computed);
    if (!e.sample) continue;
    if (k >= n_tokens) throw std::runtime_error("commit: fewer tokens than sampled entries");
    const int token = tokens[k++];
    r.output.push_back(token);
    // src/minigpt_infer/engine/engine.py:186-194
    FinishReason why = NOT_FINISHED;
    if (r.eot >= 0 && token == r.eot) why = FINISH_EOT;
    else if ((int)r.output.size() >= r.max_tokens) why = FINISH_LENGTH;
    if (why != NOT_FINISHED) finish(r, why);
    outputs_.push_back({r.id, token, why != NOT_FINISHED, (int)why});
  }
  entries_.clear();
  return outputs_;
}

int Scheduler::plan_burst(int max_k) {
  if (max_k < 2 || running_.empty() || !waiting_.empty()) return 0;
  if (pending_ > 0) {
    // planning ahead of a burst that is not handed in yet: only while its requests are still the
    // running ones, in their order (nobody has met an end token in the stretches handed in so far)
    if (entries_.size() != running_.size()) return 0;
    for (size_t i = 0; i < running_.size(); ++i)
      if (entries_[i].id != running_[i]) return 0;
  }
  int k = max_k;
  for (int id : running_) {
    const Request& r = *get(id);
    if (r.num_tokens() - r.num_computed != 1) return 0;  // still in its prompt
    k = std::min(k, r.max_tokens - (int)r.output.size() - pending_);
  }
  if (k < 2) return 0;
  // pages for k more tokens each, or no burst at all
  for (int g = 0; g < cache_->num_groups(); ++g) {
    long need = 0;
    for (int id : running_) {
      const Request& r = *get(id);
      need += std::max(0, cache_->pages_needed(g, r.num_computed + pending_ + k) - cache_->table_len(r.slot, g));
    }
    if (need > cache_->num_free_pages(g)) return 0;
  }
  entries_.clear();
  for (int id : running_) {
    Request& r = *get(id);
    cache_->reserve(r.slot, r.num_computed + pending_ + k);
    entries_.push_back({id, r.num_computed + pending_, 1, true});
  }
  num_decode_tokens += (long)k * (long)entries_.size();
  num_steps += k;
  pending_ += k;
  return k;
}

const std::vector<StepOutput>& Scheduler::commit_burst(const int* tokens, int k, bool last) {
  outputs_.clear();
  const std::vector<StepEntry> entries = entries_;
  const int n = (int)entries.size();
  for (int j = 0; j < k; ++j) {
    for (int i = 0; i < n; ++i) {
      Request& r = *get(entries[i].id);
      if (r.status != RUNNING) continue;  // ended earlier in this burst
      r.num_computed += 1;
      cache_->release_passed(r.slot, r.num_computed);
      const int token = tokens[(long)j * n + i];
      r.output.push_back(token);
      FinishReason why = NOT_FINISHED;
      if (r.eot >= 0 && token == r.eot) why = FINISH_EOT;
      else if ((int)r.output.size() >= r.max_tokens) why = FINISH_LENGTH;
      if (why != NOT_FINISHED) finish(r, why);
      outputs_.push_back({r.id, token, why != NOT_FINISHED, (int)why});
    }
  }
  pending_ = std::max(0, pending_ - k);
  if (last && pending_ == 0) entries_.clear();
  return outputs_;
}

void Scheduler::forget_finished() {
  // not while a burst's tokens are still to come: its entries name requests that may have ended
  if (pending_ > 0) return;
  for (auto& r : requests_)
    if (r && r->status == FINISHED) {
      free_ids_.push_back(r->id);
      r.reset();
    }
}

}  // namespace mgpt
