#include "cache_manager.h"

#include <algorithm>
#include <stdexcept>

namespace mgpt {

CacheManager::CacheManager(const std::vector<GroupSpec>& groups, int max_requests) : groups_(groups) {
  if (groups.empty()) throw std::invalid_argument("at least one cache group is needed");
  if (max_requests <= 0) throw std::invalid_argument("max_requests must be positive");
  for (const GroupSpec& g : groups_) {
    if (g.page_size <= 0 || g.num_pages <= 0 || g.window < 0)
      throw std::invalid_argument("bad cache group: page_size and num_pages > 0, window >= 0");
    // ids 0..n-1, taken from the end (src/minigpt_infer/cache/paged.py:39,63)
    std::vector<int> ids(g.num_pages);
    for (int i = 0; i < g.num_pages; ++i) ids[i] = i;
    free_pages_.push_back(std::move(ids));
  }
  slots_.resize(max_requests);
  for (Slot& s : slots_) {
    s.tables.resize(groups_.size());
    s.first_live.assign(groups_.size(), 0);
  }
  for (int i = max_requests - 1; i >= 0; --i) free_slots_.push_back(i);  // slot 0 goes out first
}

int CacheManager::acquire_slot() {
  if (free_slots_.empty()) return -1;
  int s = free_slots_.back();
  free_slots_.pop_back();
  Slot& slot = slots_[s];
  slot.live = true;
  slot.covered = 0;
  for (size_t g = 0; g < groups_.size(); ++g) {
    slot.tables[g].clear();
    slot.first_live[g] = 0;
  }
  return s;
}

bool CacheManager::slot_live(int slot) const {
  return slot >= 0 && slot < (int)slots_.size() && slots_[slot].live;
}

int CacheManager::pages_needed(int g, int n_tokens) const {
  const int ps = groups_[g].page_size;
  return (n_tokens + ps - 1) / ps;  // src/minigpt_infer/cache/paged.py:45-46
}

bool CacheManager::can_allocate(int n_tokens) const {
  for (size_t g = 0; g < groups_.size(); ++g)
    if (pages_needed((int)g, n_tokens) > (int)free_pages_[g].size()) return false;
  return true;
}

bool CacheManager::reserve(int slot, int n_tokens) {
  if (!slot_live(slot)) return false;
  Slot& s = slots_[slot];
  std::vector<int> extra(groups_.size(), 0);
  for (size_t g = 0; g < groups_.size(); ++g) {
    int need = pages_needed((int)g, n_tokens) - (int)s.tables[g].size();
    if (need > (int)free_pages_[g].size()) return false;
    extra[g] = std::max(need, 0);
  }
  for (size_t g = 0; g < groups_.size(); ++g) {
    for (int i = 0; i < extra[g]; ++i) {
      s.tables[g].push_back(free_pages_[g].back());
      free_pages_[g].pop_back();
    }
  }
  s.covered = std::max(s.covered, n_tokens);
  return true;
}

int CacheManager::release_passed(int slot, int n_computed) {
  if (!slot_live(slot)) return 0;
  Slot& s = slots_[slot];
  int released = 0;
  for (size_t g = 0; g < groups_.size(); ++g) {
    const int w = groups_[g].window;
    if (w <= 0) continue;
    // the query at position n_computed is the earliest still to come; it sees keys from here on
    const int earliest = n_computed - w + 1;
    if (earliest <= 0) continue;
    const int keep_from = std::min(earliest / groups_[g].page_size, (int)s.tables[g].size());
    for (int p = s.first_live[g]; p < keep_from; ++p) {
      if (s.tables[g][p] >= 0) {
        free_pages_[g].push_back(s.tables[g][p]);
        s.tables[g][p] = -1;
        ++released;
      }
    }
    s.first_live[g] = std::max(s.first_live[g], keep_from);
  }
  return released;
}

bool CacheManager::free_slot(int slot) {
  if (!slot_live(slot)) return false;
  Slot& s = slots_[slot];
  for (size_t g = 0; g < groups_.size(); ++g) {
    // in table order, as list.extend does (src/minigpt_infer/cache/paged.py:79-81)
    for (int page : s.tables[g])
      if (page >= 0) free_pages_[g].push_back(page);
    s.tables[g].clear();
    s.first_live[g] = 0;
  }
  s.live = false;
  s.covered = 0;
  free_slots_.push_back(slot);
  return true;
}

int CacheManager::held_pages(int slot, int g) const {
  int n = 0;
  for (int page : slots_[slot].tables[g]) n += page >= 0;
  return n;
}

long CacheManager::slot_of(int slot, int g, int position) const {
  const Slot& s = slots_[slot];
  const int ps = groups_[g].page_size;
  const int idx = position / ps;
  if (position < 0 || idx >= (int)s.tables[g].size() || s.tables[g][idx] < 0) return -1;
  // src/minigpt_infer/engine/engine.py:123-125
  return (long)s.tables[g][idx] * ps + position % ps;
}

int CacheManager::build_step(int n_req, const int* slots, const int* ctx_lens, const int* q_lens,
                             int n_stride, int r_stride, int max_blocks, int* positions, int* q_req,
                             int* cu_q, int* seq_lens, int* slot_mapping, int* block_tables) const {
  if (n_req < 0 || n_req > r_stride || max_blocks <= 0) return -3;
  const int G = (int)groups_.size();
  int n = 0;
  for (int i = 0; i < n_req; ++i) {
    if (!slot_live(slots[i]) || q_lens[i] < 0 || ctx_lens[i] < 0) return -3;
    n += q_lens[i];
  }
  if (n > n_stride) return -3;
  int t = 0;
  for (int i = 0; i < n_req; ++i) {
    const Slot& s = slots_[slots[i]];
    cu_q[i] = t;
    seq_lens[i] = ctx_lens[i] + q_lens[i];
    for (int j = 0; j < q_lens[i]; ++j, ++t) {
      const int pos = ctx_lens[i] + j;
      positions[t] = pos;
      q_req[t] = i;
      for (int g = 0; g < G; ++g) {
        long sl = slot_of(slots[i], g, pos);
        if (sl < 0) return -1;
        slot_mapping[(long)g * n_stride + t] = (int)sl;
      }
    }
    for (int g = 0; g < G; ++g) {
      const std::vector<int>& tab = s.tables[g];
      if ((int)tab.size() > max_blocks) return -2;
      int* row = block_tables + ((long)g * r_stride + i) * max_blocks;
      std::copy(tab.begin(), tab.end(), row);
      std::fill(row + tab.size(), row + max_blocks, -1);
    }
  }
  const int n_total = t;
  for (int i = n_req; i <= r_stride; ++i) {
    if (i < r_stride) {
      seq_lens[i] = 0;
      for (int g = 0; g < G; ++g) {
        int* row = block_tables + ((long)g * r_stride + i) * max_blocks;
        std::fill(row, row + max_blocks, -1);
      }
    }
    cu_q[i] = n_total;
  }
  for (; t < n_stride; ++t) {
    positions[t] = 0;
    q_req[t] = -1;
    for (int g = 0; g < G; ++g) slot_mapping[(long)g * n_stride + t] = -1;
  }
  return n_total;
}

int CacheManager::check() const {
  // slots: free list and live flags agree, no slot twice
  std::vector<int> seen_slot(slots_.size(), 0);
  for (int s : free_slots_) {
    if (s < 0 || s >= (int)slots_.size()) return 1;
    if (slots_[s].live) return 2;
    if (seen_slot[s]++) return 3;
  }
  for (size_t s = 0; s < slots_.size(); ++s)
    if (!slots_[s].live && !seen_slot[s]) return 4;  // a slot that is neither free nor live
  for (size_t g = 0; g < groups_.size(); ++g) {
    std::vector<int> owner(groups_[g].num_pages, 0);
    for (int p : free_pages_[g]) {
      if (p < 0 || p >= groups_[g].num_pages) return 5;
      if (owner[p]++) return 6;  // twice in the free list
    }
    for (const Slot& s : slots_) {
      if (!s.live) {
        if (!s.tables[g].empty()) return 7;
        continue;
      }
      for (int p : s.tables[g]) {
        if (p < 0) continue;
        if (p >= groups_[g].num_pages) return 5;
        if (owner[p]++) return 8;  // held twice, or held and free
      }
    }
    for (int c : owner)
      if (c != 1) return 9;  // a page lost
  }
  return 0;
}

}  // namespace mgpt
