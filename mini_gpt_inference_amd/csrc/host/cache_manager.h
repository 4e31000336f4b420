// Page bookkeeping for the key/value cache and the slots of per-request state.
//
// Follows the reference's BlockManager (src/minigpt_infer/cache/paged.py:32-94):
// a LIFO free list of page ids, tables that grow by whole pages, nothing is
// cleared when it is given back.  Beyond the reference: several groups of
// layers, each with a page pool of its own (all keys, or a window of them whose
// passed pages return early), and a fixed number of request slots that index
// both the tables and any fixed-size per-request state.
#pragma once

#include <cstdint>
#include <vector>

namespace mgpt {

struct GroupSpec {
  int page_size;  // tokens per page
  int num_pages;  // pages in this group's pool
  int window;     // 0: a query sees all earlier keys; w > 0: only the last w positions
};

class CacheManager {
 public:
  CacheManager(const std::vector<GroupSpec>& groups, int max_requests);

  int num_groups() const { return (int)groups_.size(); }
  int max_requests() const { return (int)slots_.size(); }
  const GroupSpec& group(int g) const { return groups_[g]; }

  // Request slots.  acquire returns -1 when none is free.
  int acquire_slot();
  bool slot_live(int slot) const;
  int num_free_slots() const { return (int)free_slots_.size(); }

  // Pages a sequence of n_tokens holds in group g (before any window release).
  int pages_needed(int g, int n_tokens) const;
  // Could a request that holds nothing get pages for n_tokens in every group?
  bool can_allocate(int n_tokens) const;
  // Grow the slot's tables so that positions [0, n_tokens) are covered in every
  // group (pages a window has already released stay released).  All or nothing:
  // returns false and changes nothing when some group has too few free pages.
  bool reserve(int slot, int n_tokens);
  // Give back the pages of window groups that no query at position >= n_computed can see.
  // Returns the number of pages released.
  int release_passed(int slot, int n_computed);
  // Give back every page of the slot and the slot itself.  False if the slot is not live.
  bool free_slot(int slot);

  int num_free_pages(int g) const { return (int)free_pages_[g].size(); }
  int table_len(int slot, int g) const { return (int)slots_[slot].tables[g].size(); }
  const int* table(int slot, int g) const { return slots_[slot].tables[g].data(); }
  int held_pages(int slot, int g) const;
  int covered_tokens(int slot) const { return slots_[slot].covered; }

  // Slot in the flat pool for the token at `position`, or -1 if its page is not held.
  long slot_of(int slot, int g, int position) const;

  // Fills the per-token and per-request arrays of one step.  For request i (its slot
  // slots[i], ctx_lens[i] tokens already cached, q_lens[i] new ones, in this order):
  //   positions[t], q_req[t] for each of its tokens, cu_q[i], seq_lens[i] = ctx + q,
  //   slot_mapping[g * n_stride + t], block_tables[(g * r_stride + i) * max_blocks + b]
  //   (-1 where no page is held).
  // Entries i >= n_req up to r_stride and tokens t >= N up to n_stride are filled as
  // padding: q_req -1, slot -1, position 0, seq_len 0.  Returns N, or -1 if a token's
  // page is not held, -2 if a table is longer than max_blocks, -3 on bad arguments.
  int build_step(int n_req, const int* slots, const int* ctx_lens, const int* q_lens, int n_stride,
                 int r_stride, int max_blocks, int* positions, int* q_req, int* cu_q, int* seq_lens,
                 int* slot_mapping, int* block_tables) const;

  // 0 if every page is either free or held by exactly one live slot, and every slot is
  // either free or live; otherwise a positive code naming what is wrong.
  int check() const;

 private:
  struct Slot {
    bool live = false;
    int covered = 0;                       // tokens the tables cover
    std::vector<std::vector<int>> tables;  // [group][page index] -> page id or -1
    std::vector<int> first_live;           // [group] first page index not released
  };
  std::vector<GroupSpec> groups_;
  std::vector<std::vector<int>> free_pages_;  // [group], LIFO
  std::vector<Slot> slots_;
  std::vector<int> free_slots_;  // LIFO
};

}  // namespace mgpt
