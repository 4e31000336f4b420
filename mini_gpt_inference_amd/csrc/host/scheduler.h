// Continuous-batching scheduler: admits requests, cuts prompts into portions
// under a token budget, decodes, finishes and frees.
//
// Queues, first-come admission with head-of-line blocking, newest-first
// preempt-by-recompute and free-on-finish follow the reference
// (src/minigpt_infer/engine/scheduler.py:23-117).  Prompt portions and steps
// that mix prompt work with decoding are not in the reference
// (scheduler.py:9-12); with mixed = false and prefill_chunk = 0 the policy is
// the reference's: a step that has prompt work runs prompts only.
//
// One rule covers prompts, portions, recompute and decoding: a request's context
// is prompt + outputs; a step feeds context[num_computed : num_computed + q]
// with 1 <= q <= remaining; only when num_computed reaches the context's length
// is a logit row produced and one token sampled (src/minigpt_infer/engine/engine.py:243-244,
// 281-282; src/minigpt_infer/engine/request.py:59-63).
#pragma once

#include <cstdint>
#include <deque>
#include <memory>
#include <vector>

#include "cache_manager.h"

namespace mgpt {

enum RequestStatus { WAITING = 0, RUNNING = 1, FINISHED = 2 };
enum FinishReason { NOT_FINISHED = 0, FINISH_EOT = 1, FINISH_LENGTH = 2, FINISH_CANCELLED = 3 };

struct SchedulerConfig {
  int max_batch_size;          // most requests running at once
  int max_num_batched_tokens;  // token budget of one step
  int prefill_chunk;           // largest prompt portion per request and step; 0 = no limit
  bool mixed;                  // prompt portions beside decode tokens in one step
  int max_positions;           // prompt + max_tokens may not exceed it (engine.py:83-88)
  bool spare_asker = false;    // when pages run out: true = evict the newest running request other than
                               // the one that asks (scheduler.py:66-82); false = the newest, the asker too
};

struct Request {
  int id = -1;
  std::vector<int> prompt;
  std::vector<int> output;
  int max_tokens = 0;
  int eot = -1;  // -1: none
  float temperature = 1.0f;
  int top_k = 0;       // 0: off
  float top_p = 1.0f;  // 1: off
  uint64_t seed = 0;
  int num_computed = 0;  // tokens whose keys and values are in the cache
  int slot = -1;
  RequestStatus status = WAITING;
  FinishReason finish_reason = NOT_FINISHED;
  int num_tokens() const { return (int)(prompt.size() + output.size()); }
  int token_at(int i) const { return i < (int)prompt.size() ? prompt[i] : output[i - prompt.size()]; }
};

struct StepEntry {
  int id;       // request id
  int ctx;      // tokens already cached = position of the first new token
  int q_len;    // tokens fed in this step
  bool sample;  // the context is complete after this step: a logit row and one new token
};

struct StepOutput {
  int id;
  int token;
  int finished;  // 0/1
  int reason;    // FinishReason
};

class Scheduler {
 public:
  // add_request errors
  static constexpr int ERR_EMPTY_PROMPT = -1;
  static constexpr int ERR_TOO_LONG = -2;      // prompt + max_tokens > max_positions
  static constexpr int ERR_NEVER_FITS = -3;    // more pages than the whole pool holds
  static constexpr int ERR_BAD_PARAMS = -4;

  Scheduler(CacheManager* cache, const SchedulerConfig& cfg);

  int add_request(const int* prompt, int n_prompt, int max_tokens, int eot, float temperature,
                  int top_k, float top_p, uint64_t seed, bool has_seed);
  bool has_work() const { return !waiting_.empty() || !running_.empty(); }
  bool cancel(int id);

  // Decides the next step.  The entries stay valid until the next call.
  const std::vector<StepEntry>& schedule();
  // Takes the tokens sampled for the entries with sample = true, in entry order.
  const std::vector<StepOutput>& commit(const int* tokens, int n_tokens);

  // A burst: up to max_k decode steps of the running requests planned at once, so that the device
  // can run them back to back while it feeds each step's tokens to the next by itself.  Only when
  // every running request is decoding, nobody waits, and pages for all k tokens are free; k stops
  // at the first request's length limit, so nobody can end before a burst's last step except by its
  // end token.  Returns k >= 2 with entries() set to step 0, or 0 when a burst is not possible
  // (then nothing has changed).  Step j of a burst feeds position ctx + j.
  // A further burst may be planned before the last one's tokens are all handed in (the device then
  // never waits for the host between them): it starts where that one will end, and is refused (0) once
  // a request of that one has ended, since the device goes on computing for the same requests.
  int plan_burst(int max_k);
  // tokens[j * n_entries + i]: what entry i sampled in step j.  A request that meets its end token
  // in step j ends there; what the device computed for it afterwards is dropped.  A burst may be
  // handed in in several stretches of steps, in order (the device is then still at work on the later
  // ones: pages that a request's end frees are given to nobody before the next plan); `last` ends it.
  // The entries stay until every planned step has been handed in.
  const std::vector<StepOutput>& commit_burst(const int* tokens, int k, bool last = true);

  const Request* request(int id) const;
  const std::deque<int>& waiting() const { return waiting_; }
  const std::vector<int>& running() const { return running_; }
  const std::vector<StepEntry>& entries() const { return entries_; }

  long num_preemptions = 0;
  long num_steps = 0;
  long num_prompt_tokens = 0;  // scheduled as part of a portion of more than one token or an unfinished prompt
  long num_decode_tokens = 0;

  // drops the records of finished requests; their ids are given to later requests
  void forget_finished();
  int num_records() const { return (int)requests_.size() - (int)free_ids_.size(); }

 private:
  Request* get(int id);
  void preempt(Request& r);
  void finish(Request& r, FinishReason why);
  void ensure_capacity_for_decode();
  void schedule_decodes(int& budget);
  void schedule_prompts(int& budget, bool allow_admission);

  CacheManager* cache_;
  SchedulerConfig cfg_;
  std::vector<std::unique_ptr<Request>> requests_;  // index = id; null = forgotten
  std::vector<int> free_ids_;                        // ids of forgotten requests
  uint64_t num_added_ = 0;
  std::deque<int> waiting_;
  std::vector<int> running_;  // admission order
  std::vector<StepEntry> entries_;
  std::vector<StepOutput> outputs_;
  bool preempted_this_step_ = false;
  int pending_ = 0;  // steps of planned bursts whose tokens have not been handed in yet
};

}  // namespace mgpt
