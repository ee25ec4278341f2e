// The cache manager's host side: pages, block tables and slots.
//
// Each cache group (layers with the same need: all positions, or a window of them) has a pool
// of pages of its own and one block table row per live request.  A request is given a slot
// when it is opened; the slot indexes the block tables and the per-request state arenas.
// Pages are taken when a request's length grows, given back when it is closed or, in a
// windowed group, when the window has passed them, and then used again.
//
// The shape follows the reference's page allocator (src/cuda/qwen2/pages.rs:37-153: per-slot
// page lists that grow at the end, a LIFO free list, `ensure` that takes nothing when it
// cannot take everything, a seeded shuffle of the free list for tests, `check` invariants
// 318-351), extended by groups and windows.  Nothing here touches the device.
#include <stdint.h>

#include <string>
#include <vector>

#include "geometry.h"

namespace {

struct Group {
  GroupGeometry geo;
  std::vector<int> free_list;              // LIFO; page 0 handed out first
  std::vector<uint8_t> live;               // per page: held by a slot
  std::vector<std::vector<int>> pages;     // per slot: logical page -> physical, -1 once trimmed
  std::vector<int> first_live;             // per slot: first logical page not yet trimmed
};

struct Cache {
  std::vector<Group> groups;
  int max_seqs;
  int max_pages_per_seq;
  std::vector<uint8_t> open;
  std::vector<long> length;                // tokens covered by reserved pages, per slot
  std::vector<int> free_slots;             // LIFO, slot 0 first
  uint64_t rng;
  bool shuffle;
  std::string error;
};

uint64_t next_random(uint64_t& s) {
  s += 0x9e3779b97f4a7c15ull;
  uint64_t z = s;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

int take_page(Cache& c, Group& g) {
  size_t at = g.free_list.size() - 1;
  if (c.shuffle) at = (size_t)(next_random(c.rng) % g.free_list.size());
  const int page = g.free_list[at];
  g.free_list[at] = g.free_list.back();
  g.free_list.pop_back();
  g.live[page] = 1;
  return page;
}

void give_page(Group& g, int page) {
  g.live[page] = 0;
  g.free_list.push_back(page);
}

}  // namespace

extern "C" {

void* axh_cache_create(int n_groups, const int* n_pages, const int* page_size, const int* window, int max_seqs,
                       int max_pages_per_seq, long shuffle_seed) {
  if (n_groups < 0 || max_seqs < 1 || max_pages_per_seq < 1) return nullptr;
  Cache* c = new Cache();
  c->max_seqs = max_seqs;
  c->max_pages_per_seq = max_pages_per_seq;
  c->open.assign(max_seqs, 0);
  c->length.assign(max_seqs, 0);
  for (int s = max_seqs - 1; s >= 0; --s) c->free_slots.push_back(s);
  c->shuffle = shuffle_seed >= 0;
  c->rng = (uint64_t)shuffle_seed;
  for (int i = 0; i < n_groups; ++i) {
    if (n_pages[i] < 1 || page_size[i] < 1 || window[i] < 0) {
      delete c;
      return nullptr;
    }
    Group g;
    g.geo = GroupGeometry{n_pages[i], page_size[i], window[i]};
    for (int p = n_pages[i] - 1; p >= 0; --p) g.free_list.push_back(p);
    g.live.assign(n_pages[i], 0);
    g.pages.resize(max_seqs);
    g.first_live.assign(max_seqs, 0);
    c->groups.push_back(std::move(g));
  }
  return c;
}

void axh_cache_destroy(void* h) { delete (Cache*)h; }

const char* axh_cache_error(void* h) { return ((Cache*)h)->error.c_str(); }

// A slot for a new request, or -1 when all are taken.
int axh_cache_open(void* h) {
  Cache& c = *(Cache*)h;
  if (c.free_slots.empty()) {
    c.error = "no free slot: " + std::to_string(c.max_seqs) + " requests are live";
    return -1;
  }
  const int s = c.free_slots.back();
  c.free_slots.pop_back();
  c.open[s] = 1;
  c.length[s] = 0;
  return s;
}

// Give back everything the slot holds.  Returns the pages freed, or -1 if it is not open.
int axh_cache_close(void* h, int slot) {
  Cache& c = *(Cache*)h;
  if (slot < 0 || slot >= c.max_seqs || !c.open[slot]) {
    c.error = "slot " + std::to_string(slot) + " is not open";
    return -1;
  }
  int freed = 0;
  for (Group& g : c.groups) {
    for (int p : g.pages[slot])
      if (p >= 0) {
        give_page(g, p);
        ++freed;
      }
    g.pages[slot].clear();
    g.first_live[slot] = 0;
  }
  c.open[slot] = 0;
  c.length[slot] = 0;
  c.free_slots.push_back(slot);
  return freed;
}

// Pages for positions [0, n_tokens) in every group, or nothing at all: 0 on success, else
// the negative number of pages that were short (summed over groups), -1000000 for a bad call.
int axh_cache_reserve(void* h, int slot, long n_tokens) {
  Cache& c = *(Cache*)h;
  if (slot < 0 || slot >= c.max_seqs || !c.open[slot] || n_tokens < 0) {
    c.error = "reserve: slot " + std::to_string(slot) + " is not open";
    return -1000000;
  }
  int short_by = 0;
  for (Group& g : c.groups) {
    const int want = pages_covering(g.geo, n_tokens);
    if (want > c.max_pages_per_seq) {
      c.error = "reserve: " + std::to_string(n_tokens) + " tokens need " + std::to_string(want) +
                " pages, a request may hold " + std::to_string(c.max_pages_per_seq);
      return -1000000;
    }
    const int need = want - (int)g.pages[slot].size();
    if (need > (int)g.free_list.size()) short_by += need - (int)g.free_list.size();
  }
  if (short_by > 0) {
    c.error = "reserve: " + std::to_string(short_by) + " pages short";
    return -short_by;
  }
  for (Group& g : c.groups) {
    const int want = pages_covering(g.geo, n_tokens);
    while ((int)g.pages[slot].size() < want) g.pages[slot].push_back(take_page(c, g));
  }
  if (n_tokens > c.length[slot]) c.length[slot] = n_tokens;
  return 0;
}

// Pages for several requests at once (slot i up to n_tokens[i] positions), for all of them in
// every group or for none: a step's entries are reserved together, so that a step that does not
// fit leaves the cache as it found it.  Returns 0, or -(pages short), or -1000000 for a bad call.
int axh_cache_reserve_many(void* h, int n, const int* slots, const long* n_tokens) {
  Cache& c = *(Cache*)h;
  for (int i = 0; i < n; ++i) {
    const int slot = slots[i];
    if (slot < 0 || slot >= c.max_seqs || !c.open[slot] || n_tokens[i] < 0) {
      c.error = "reserve: slot " + std::to_string(slot) + " is not open";
      return -1000000;
    }
    for (int j = 0; j < i; ++j)
      if (slots[j] == slot) {
        c.error = "reserve: slot " + std::to_string(slot) + " is named twice";
        return -1000000;
      }
  }
  int short_by = 0;
  for (Group& g : c.groups) {
    long need = 0;
    for (int i = 0; i < n; ++i) {
      const int want = pages_covering(g.geo, n_tokens[i]);
      if (want > c.max_pages_per_seq) {
        c.error = "reserve: " + std::to_string(n_tokens[i]) + " tokens need " + std::to_string(want) +
                  " pages, a request may hold " + std::to_string(c.max_pages_per_seq);
        return -1000000;
      }
      need += std::max(0, want - (int)g.pages[slots[i]].size());
    }
    if (need > (long)g.free_list.size()) short_by += (int)(need - (long)g.free_list.size());
  }
  if (short_by > 0) {
    c.error = "reserve: " + std::to_string(short_by) + " pages short";
    return -short_by;
  }
  for (int i = 0; i < n; ++i) {
    for (Group& g : c.groups) {
      const int want = pages_covering(g.geo, n_tokens[i]);
      while ((int)g.pages[slots[i]].size() < want) g.pages[slots[i]].push_back(take_page(c, g));
    }
    if (n_tokens[i] > c.length[slots[i]]) c.length[slots[i]] = n_tokens[i];
  }
  return 0;
}

// After a step: `n_cached` tokens are in the cache.  Windowed groups give back the pages the
// window has passed.  Returns the pages freed.
int axh_cache_trim(void* h, int slot, long n_cached) {
  Cache& c = *(Cache*)h;
  if (slot < 0 || slot >= c.max_seqs || !c.open[slot]) return -1;
  int freed = 0;
  for (Group& g : c.groups) {
    const int upto = std::min(first_needed_page(g.geo, n_cached), (int)g.pages[slot].size());
    for (int i = g.first_live[slot]; i < upto; ++i) {
      if (g.pages[slot][i] >= 0) {
        give_page(g, g.pages[slot][i]);
        g.pages[slot][i] = -1;
        ++freed;
      }
    }
    if (upto > g.first_live[slot]) g.first_live[slot] = upto;
  }
  return freed;
}

// The slot's block table row for one group: physical page of each logical page; pages given
// back read as 0 (valid memory that is never used: the window excludes their positions).
int axh_cache_row(void* h, int group, int slot, int* out, int cap) {
  Cache& c = *(Cache*)h;
  if (group < 0 || group >= (int)c.groups.size() || slot < 0 || slot >= c.max_seqs) return -1;
  const std::vector<int>& p = c.groups[group].pages[slot];
  const int n = std::min((int)p.size(), cap);
  for (int i = 0; i < n; ++i) out[i] = p[i] >= 0 ? p[i] : 0;
  return n;
}

int axh_cache_free_pages(void* h, int group) {
  Cache& c = *(Cache*)h;
  if (group < 0 || group >= (int)c.groups.size()) return -1;
  return (int)c.groups[group].free_list.size();
}

int axh_cache_free_slots(void* h) { return (int)((Cache*)h)->free_slots.size(); }

int axh_cache_pages_of(void* h, int group, int slot) {
  Cache& c = *(Cache*)h;
  if (group < 0 || group >= (int)c.groups.size() || slot < 0 || slot >= c.max_seqs) return -1;
  int n = 0;
  for (int p : c.groups[group].pages[slot]) n += p >= 0;
  return n;
}

long axh_cache_length(void* h, int slot) {
  Cache& c = *(Cache*)h;
  return slot >= 0 && slot < c.max_seqs && c.open[slot] ? c.length[slot] : -1;
}

// Invariants: every page is free or held exactly once, never both; closed slots hold nothing;
// slots are free or open exactly once.  0 if all hold, else a negative code.
int axh_cache_check(void* h) {
  Cache& c = *(Cache*)h;
  for (size_t gi = 0; gi < c.groups.size(); ++gi) {
    Group& g = c.groups[gi];
    std::vector<int> seen(g.geo.n_pages, 0);
    for (int p : g.free_list) {
      if (p < 0 || p >= g.geo.n_pages || g.live[p]) { c.error = "a free page is out of range or marked live"; return -1; }
      if (seen[p]++) { c.error = "page " + std::to_string(p) + " is in the free list twice"; return -2; }
    }
    for (int s = 0; s < c.max_seqs; ++s) {
      if (!c.open[s] && !g.pages[s].empty()) { c.error = "a closed slot holds pages"; return -3; }
      if ((int)g.pages[s].size() > c.max_pages_per_seq) { c.error = "a slot holds more pages than allowed"; return -4; }
      for (int p : g.pages[s]) {
        if (p < 0) continue;
        if (p >= g.geo.n_pages || !g.live[p]) { c.error = "a held page is out of range or not marked live"; return -5; }
        if (seen[p]++) { c.error = "page " + std::to_string(p) + " is held twice, or held and free"; return -6; }
      }
    }
    for (int p = 0; p < g.geo.n_pages; ++p)
      if (!seen[p]) { c.error = "page " + std::to_string(p) + " is lost: neither free nor held"; return -7; }
  }
  std::vector<int> slot_seen(c.max_seqs, 0);
  for (int s : c.free_slots) {
    if (s < 0 || s >= c.max_seqs || c.open[s] || slot_seen[s]++) { c.error = "the free slot list is inconsistent"; return -8; }
  }
  for (int s = 0; s < c.max_seqs; ++s)
    if (!c.open[s] && !slot_seen[s]) { c.error = "a slot is lost"; return -9; }
  return 0;
}

}  // extern "C"
