// C interface of the host runtime (cache manager and scheduler), for ctypes.
// Every function catches C++ exceptions; the text of the last one is kept per thread.
#include <cstring>
#include <string>

#include "cache_manager.h"
#include "scheduler.h"

using mgpt::CacheManager;
using mgpt::GroupSpec;
using mgpt::Scheduler;
using mgpt::SchedulerConfig;

static thread_local std::string g_last_error;

#define GUARD_BEGIN try {
#define GUARD_END(fail)                  \
  }                                      \
  catch (const std::exception& e) {      \
    g_last_error = e.what();             \
    return fail;                         \
  }                                      \
  catch (...) {                          \
    g_last_error = "unknown C++ error";  \
    return fail;                         \
  }

extern "C" {

const char* mgpt_host_last_error() { return g_last_error.c_str(); }

// ---------------------------------------------------------------- cache manager
void* mgpt_cache_create(int n_groups, const int* page_sizes, const int* num_pages, const int* windows,
                        int max_requests) {
  GUARD_BEGIN
  std::vector<GroupSpec> groups;
  for (int g = 0; g < n_groups; ++g) groups.push_back({page_sizes[g], num_pages[g], windows[g]});
  return new CacheManager(groups, max_requests);
  GUARD_END(nullptr)
}

void mgpt_cache_destroy(void* cm) { delete static_cast<CacheManager*>(cm); }

int mgpt_cache_num_groups(void* cm) { return static_cast<CacheManager*>(cm)->num_groups(); }
int mgpt_cache_acquire_slot(void* cm) { return static_cast<CacheManager*>(cm)->acquire_slot(); }
int mgpt_cache_slot_live(void* cm, int slot) { return static_cast<CacheManager*>(cm)->slot_live(slot); }
int mgpt_cache_num_free_slots(void* cm) { return static_cast<CacheManager*>(cm)->num_free_slots(); }
int mgpt_cache_pages_needed(void* cm, int g, int n) { return static_cast<CacheManager*>(cm)->pages_needed(g, n); }
int mgpt_cache_can_allocate(void* cm, int n) { return static_cast<CacheManager*>(cm)->can_allocate(n); }
int mgpt_cache_reserve(void* cm, int slot, int n) { return static_cast<CacheManager*>(cm)->reserve(slot, n); }
int mgpt_cache_release_passed(void* cm, int slot, int n) {
  return static_cast<CacheManager*>(cm)->release_passed(slot, n);
}
int mgpt_cache_free_slot(void* cm, int slot) { return static_cast<CacheManager*>(cm)->free_slot(slot); }
int mgpt_cache_num_free_pages(void* cm, int g) { return static_cast<CacheManager*>(cm)->num_free_pages(g); }
int mgpt_cache_held_pages(void* cm, int slot, int g) {
  CacheManager* c = static_cast<CacheManager*>(cm);
  return c->slot_live(slot) ? c->held_pages(slot, g) : -1;
}
int mgpt_cache_table_len(void* cm, int slot, int g) {
  CacheManager* c = static_cast<CacheManager*>(cm);
  return c->slot_live(slot) ? c->table_len(slot, g) : -1;
}
int mgpt_cache_copy_table(void* cm, int slot, int g, int* out, int cap) {
  CacheManager* c = static_cast<CacheManager*>(cm);
  if (!c->slot_live(slot)) return -1;
  int n = c->table_len(slot, g);
  if (n > cap) return -2;
  std::memcpy(out, c->table(slot, g), sizeof(int) * n);
  return n;
}
int mgpt_cache_check(void* cm) { return static_cast<CacheManager*>(cm)->check(); }

int mgpt_cache_build_step(void* cm, int n_req, const int* slots, const int* ctx_lens, const int* q_lens,
                          int n_stride, int r_stride, int max_blocks, int* positions, int* q_req,
                          int* cu_q, int* seq_lens, int* slot_mapping, int* block_tables) {
  GUARD_BEGIN
  return static_cast<CacheManager*>(cm)->build_step(n_req, slots, ctx_lens, q_lens, n_stride, r_stride,
                                                    max_blocks, positions, q_req, cu_q, seq_lens,
                                                    slot_mapping, block_tables);
  GUARD_END(-100)
}

// ---------------------------------------------------------------- scheduler
void* mgpt_sched_create(void* cm, int max_batch_size, int max_num_batched_tokens, int prefill_chunk,
                        int mixed, int max_positions, int spare_asker) {
  GUARD_BEGIN
  SchedulerConfig cfg{max_batch_size, max_num_batched_tokens, prefill_chunk, mixed != 0, max_positions,
                      spare_asker != 0};
  return new Scheduler(static_cast<CacheManager*>(cm), cfg);
  GUARD_END(nullptr)
}

void mgpt_sched_destroy(void* s) { delete static_cast<Scheduler*>(s); }

int mgpt_sched_add(void* s, const int* prompt, int n_prompt, int max_tokens, int eot, float temperature,
                   int top_k, float top_p, unsigned long long seed, int has_seed) {
  GUARD_BEGIN
  return static_cast<Scheduler*>(s)->add_request(prompt, n_prompt, max_tokens, eot, temperature, top_k,
                                                 top_p, seed, has_seed != 0);
  GUARD_END(-100)
}

int mgpt_sched_has_work(void* s) { return static_cast<Scheduler*>(s)->has_work(); }
int mgpt_sched_cancel(void* s, int id) { return static_cast<Scheduler*>(s)->cancel(id); }

// Plans the next step; returns the number of entries and writes the totals:
// counts[0] = tokens, counts[1] = entries, counts[2] = entries that sample.
int mgpt_sched_schedule(void* s, int* counts) {
  GUARD_BEGIN
  const auto& e = static_cast<Scheduler*>(s)->schedule();
  int n = 0, m = 0;
  for (const auto& x : e) {
    n += x.q_len;
    m += x.sample;
  }
  counts[0] = n;
  counts[1] = (int)e.size();
  counts[2] = m;
  return (int)e.size();
  GUARD_END(-100)
}

int mgpt_sched_entries(void* s, int* ids, int* ctx, int* q_len, int* sample, int cap) {
  const auto& e = static_cast<Scheduler*>(s)->entries();
  if ((int)e.size() > cap) return -1;
  for (size_t i = 0; i < e.size(); ++i) {
    ids[i] = e[i].id;
    ctx[i] = e[i].ctx;
    q_len[i] = e[i].q_len;
    sample[i] = e[i].sample;
  }
  return (int)e.size();
}

// Fills the arrays of the planned step (step_offset = 0), or of step `step_offset` of a planned
// burst: every entry then feeds position ctx + step_offset, and its token, which only the device
// knows, is left 0 for the device to fill in.  Per-token arrays have n_stride entries, per-request
// arrays r_stride (cu_q one more), per-logit-row arrays m_stride; what lies beyond the real
// counts is padding that the kernels skip.  Returns 0, or a negative code.
int mgpt_sched_fill(void* sv, void* cm, int step_offset, int n_stride, int r_stride, int m_stride,
                    int max_blocks, int* token_ids, int* positions, int* q_req, int* cu_q, int* seq_lens,
                    int* slot_mapping, int* block_tables, int* state_slots, int* logit_rows,
                    float* temperature, int* top_k, float* top_p, unsigned long long* seeds,
                    int* out_index) {
  GUARD_BEGIN
  Scheduler* s = static_cast<Scheduler*>(sv);
  CacheManager* c = static_cast<CacheManager*>(cm);
  const auto& e = s->entries();
  const int R = (int)e.size();
  if (R > r_stride) return -3;
  std::vector<int> slots(R), ctx(R), ql(R);
  for (int i = 0; i < R; ++i) {
    const mgpt::Request* r = s->request(e[i].id);
    slots[i] = r->slot;
    ctx[i] = e[i].ctx + step_offset;
    ql[i] = e[i].q_len;
  }
  int n = c->build_step(R, slots.data(), ctx.data(), ql.data(), n_stride, r_stride, max_blocks, positions,
                        q_req, cu_q, seq_lens, slot_mapping, block_tables);
  if (n < 0) return n;
  int t = 0, m = 0;
  for (int i = 0; i < R; ++i) {
    const mgpt::Request* r = s->request(e[i].id);
    state_slots[i] = r->slot;
    // a burst planned ahead of one that is not handed in yet starts at a token only the device has
    for (int j = 0; j < e[i].q_len; ++j) {
      const int at = e[i].ctx + j;
      token_ids[t++] = (step_offset || at >= r->num_tokens()) ? 0 : r->token_at(at);
    }
    if (e[i].sample) {
      if (m >= m_stride) return -4;
      logit_rows[m] = t - 1;
      temperature[m] = r->temperature;
      top_k[m] = r->top_k;
      top_p[m] = r->top_p;
      seeds[m] = r->seed;
      out_index[m] = (int)r->output.size() + step_offset;
      ++m;
    }
  }
  for (int i = R; i < r_stride; ++i) state_slots[i] = -1;
  for (; t < n_stride; ++t) token_ids[t] = 0;
  for (; m < m_stride; ++m) {
    logit_rows[m] = 0;
    temperature[m] = 0.0f;
    top_k[m] = 0;
    top_p[m] = 1.0f;
    seeds[m] = 0;
    out_index[m] = 0;
  }
  return 0;
  GUARD_END(-100)
}

int mgpt_sched_commit(void* s, const int* tokens, int n_tokens, int* out_ids, int* out_tokens,
                      int* out_finished, int* out_reason, int cap) {
  GUARD_BEGIN
  const auto& o = static_cast<Scheduler*>(s)->commit(tokens, n_tokens);
  if ((int)o.size() > cap) return -1;
  for (size_t i = 0; i < o.size(); ++i) {
    out_ids[i] = o[i].id;
    out_tokens[i] = o[i].token;
    out_finished[i] = o[i].finished;
    out_reason[i] = o[i].reason;
  }
  return (int)o.size();
  GUARD_END(-100)
}

int mgpt_sched_plan_burst(void* s, int max_k) {
  GUARD_BEGIN
  return static_cast<Scheduler*>(s)->plan_burst(max_k);
  GUARD_END(-100)
}

int mgpt_sched_commit_burst(void* s, const int* tokens, int k, int last, int* out_ids, int* out_tokens,
                            int* out_finished, int* out_reason, int cap) {
  GUARD_BEGIN
  const auto& o = static_cast<Scheduler*>(s)->commit_burst(tokens, k, last != 0);
  if ((int)o.size() > cap) return -1;
  for (size_t i = 0; i < o.size(); ++i) {
    out_ids[i] = o[i].id;
    out_tokens[i] = o[i].token;
    out_finished[i] = o[i].finished;
    out_reason[i] = o[i].reason;
  }
  return (int)o.size();
  GUARD_END(-100)
}

// which: 0 preemptions, 1 steps, 2 prompt tokens, 3 decode tokens, 4 waiting, 5 running
long mgpt_sched_counter(void* sv, int which) {
  Scheduler* s = static_cast<Scheduler*>(sv);
  switch (which) {
    case 0: return s->num_preemptions;
    case 1: return s->num_steps;
    case 2: return s->num_prompt_tokens;
    case 3: return s->num_decode_tokens;
    case 4: return (long)s->waiting().size();
    case 5: return (long)s->running().size();
  }
  return -1;
}

// which: 0 waiting (front first), 1 running (admission order)
int mgpt_sched_queue(void* sv, int which, int* out, int cap) {
  Scheduler* s = static_cast<Scheduler*>(sv);
  int n = 0;
  if (which == 0) {
    for (int id : s->waiting()) {
      if (n >= cap) return -1;
      out[n++] = id;
    }
  } else {
    for (int id : s->running()) {
      if (n >= cap) return -1;
      out[n++] = id;
    }
  }
  return n;
}

// info: status, finish reason, num_computed, prompt length, output length, slot
int mgpt_sched_request_info(void* sv, int id, int* info) {
  const mgpt::Request* r = static_cast<Scheduler*>(sv)->request(id);
  if (!r) return -1;
  info[0] = r->status;
  info[1] = r->finish_reason;
  info[2] = r->num_computed;
  info[3] = (int)r->prompt.size();
  info[4] = (int)r->output.size();
  info[5] = r->slot;
  return 0;
}

int mgpt_sched_copy_output(void* sv, int id, int* out, int cap) {
  const mgpt::Request* r = static_cast<Scheduler*>(sv)->request(id);
  if (!r) return -1;
  if ((int)r->output.size() > cap) return -2;
  std::memcpy(out, r->output.data(), sizeof(int) * r->output.size());
  return (int)r->output.size();
}

void mgpt_sched_forget_finished(void* sv) { static_cast<Scheduler*>(sv)->forget_finished(); }

// request records that the scheduler holds now (waiting, running, and finished ones not yet forgotten)
int mgpt_sched_num_records(void* sv) { return static_cast<Scheduler*>(sv)->num_records(); }

}  // extern "C"
