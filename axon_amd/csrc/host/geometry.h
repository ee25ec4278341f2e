// Page arithmetic shared by the cache manager and the scheduler, so that what the scheduler
// plans is what the cache manager will do.
#pragma once

#include <algorithm>

struct GroupGeometry {
  int n_pages;    // pages in the group's pool
  int page_size;  // positions in one page
  int window;     // 0: every position is kept; w > 0: a token reads the last w positions only
};

// Pages that cover positions [0, n_tokens).
static inline int pages_covering(const GroupGeometry& g, long n_tokens) {
  return (int)((n_tokens + g.page_size - 1) / g.page_size);
}

// The first page still needed once `n_cached` tokens are in the cache: the next token, at
// position n_cached, reads from max(0, n_cached + 1 - window) on.
static inline int first_needed_page(const GroupGeometry& g, long n_cached) {
  if (g.window <= 0) return 0;
  const long lo = std::max(0L, n_cached + 1 - (long)g.window);
  return (int)(lo / g.page_size);
}

// Pages a request holds in this group after `n_cached` tokens (and trimming).
static inline int pages_held(const GroupGeometry& g, long n_cached) {
  return pages_covering(g, n_cached) - std::min(first_needed_page(g, n_cached), pages_covering(g, n_cached));
}

// New pages needed to go from n_cached to n_after tokens (pages are trimmed only after a step).
static inline int pages_to_grow(const GroupGeometry& g, long n_cached, long n_after) {
  return pages_covering(g, n_after) - pages_covering(g, n_cached);
}
