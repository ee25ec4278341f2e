// The scheduler's decisions, as functions of numbers: which requests run in the next step,
// with how many of their tokens, and who gives up its pages when they run out.
//
// It follows the shape of the reference's batch scheduler (src/serve/engine.rs:2037-2181
// `step_inner`; admission 1466-1521; portions 2376-2486; page growth and the victim rule
// 775-801, 2183-2276), simplified: requests are admitted first come first served; every step
// has one token budget; requests with one token left to run (decoding) are served first, the
// rest of the budget goes to prompt portions, oldest request first; a portion is cut to what
// the budget and the free pages allow.  When a request cannot grow, the youngest running
// request younger than it gives up all its pages and goes back to waiting; it is later fed
// again from position 0, its prompt and the tokens it generated, and continues where it was
// (the reference's preemption: src/serve/engine.rs:2244-2276).  The oldest request never
// yields, so it always makes progress.  A request whose prompt plus generation cannot fit the
// pool even alone is refused when it is added.
//
// The scheduler holds no pages itself: it is told the free pages per group, mirrors the cache
// manager's arithmetic (geometry.h) and returns a plan; the caller opens, reserves and closes.
#include <stdint.h>

#include <algorithm>
#include <string>
#include <vector>

#include "geometry.h"

namespace {

enum { WAITING = 0, RUNNING = 1 };

struct Request {
  int64_t id;
  long prompt_len;
  long max_new;
  long total;      // tokens the request consists of now: prompt + generated
  long computed;   // of these, already in the cache
  long arrival;
  int state;
  long planned;    // tokens planned for the step being built (0: not in the plan)
};

struct Scheduler {
  std::vector<GroupGeometry> groups;
  int max_batch_tokens;
  int max_seqs;
  long max_seq_len;
  std::vector<Request> reqs;  // in arrival order
  long next_arrival = 0;
  long preemptions = 0;
  std::string error;
};

Request* find(Scheduler& s, int64_t id) {
  for (Request& r : s.reqs)
    if (r.id == id) return &r;
  return nullptr;
}

void take(const Scheduler& s, std::vector<long>& free, long from, long to) {
  for (size_t g = 0; g < s.groups.size(); ++g) free[g] -= pages_to_grow(s.groups[g], from, to);
}

// The most tokens beyond `from` (at most `want`) that the free pages cover.
long coverable(const Scheduler& s, const std::vector<long>& free, long from, long want) {
  long n = want;
  for (size_t g = 0; g < s.groups.size(); ++g) {
    const GroupGeometry& geo = s.groups[g];
    const long cap = ((long)pages_covering(geo, from) + free[g]) * geo.page_size - from;
    n = std::min(n, cap);
  }
  return std::max(n, 0L);
}

// The youngest running request that arrived after `than` and holds or is about to hold
// pages; null if there is none.
Request* victim_younger_than(Scheduler& s, long than) {
  Request* v = nullptr;
  for (Request& r : s.reqs)
    if (r.state == RUNNING && r.arrival > than && (r.computed > 0 || r.planned > 0))
      if (!v || r.arrival > v->arrival) v = &r;
  return v;
}

void preempt(Scheduler& s, Request& v, std::vector<long>& free, long& budget, std::vector<int64_t>& preempted) {
  for (size_t g = 0; g < s.groups.size(); ++g)
    free[g] += pages_held(s.groups[g], v.computed) + pages_to_grow(s.groups[g], v.computed, v.computed + v.planned);
  budget += v.planned;
  v.planned = 0;
  v.computed = 0;
  v.state = WAITING;
  ++s.preemptions;
  preempted.push_back(v.id);
}

}  // namespace

extern "C" {

void* axh_sched_create(int n_groups, const int* n_pages, const int* page_size, const int* window,
                       int max_batch_tokens, int max_seqs, long max_seq_len) {
  if (n_groups < 0 || max_batch_tokens < 1 || max_seqs < 1 || max_seq_len < 1) return nullptr;
  Scheduler* s = new Scheduler();
  for (int i = 0; i < n_groups; ++i) s->groups.push_back(GroupGeometry{n_pages[i], page_size[i], window[i]});
  s->max_batch_tokens = max_batch_tokens;
  s->max_seqs = max_seqs;
  s->max_seq_len = max_seq_len;
  return s;
}

void axh_sched_destroy(void* h) { delete (Scheduler*)h; }

const char* axh_sched_error(void* h) { return ((Scheduler*)h)->error.c_str(); }

// A new request joins the waiting queue.  0, or -1 with a message: the id is in use, the
// prompt is empty, or prompt + generation exceeds the positions a request may reach or the
// pages of a pool.
int axh_sched_add(void* h, int64_t id, long prompt_len, long max_new) {
  Scheduler& s = *(Scheduler*)h;
  if (find(s, id)) { s.error = "request id " + std::to_string(id) + " is already in use"; return -1; }
  if (prompt_len < 1 || max_new < 0) { s.error = "a request needs at least one prompt token"; return -1; }
  const long most = prompt_len + max_new;
  if (most > s.max_seq_len) {
    s.error = "prompt of " + std::to_string(prompt_len) + " tokens plus " + std::to_string(max_new) +
              " new ones exceeds the " + std::to_string(s.max_seq_len) + " positions a request may reach";
    return -1;
  }
  for (const GroupGeometry& g : s.groups)
    if (pages_covering(g, most) > g.n_pages) {
      s.error = "the request needs " + std::to_string(pages_covering(g, most)) + " pages, the pool has " +
                std::to_string(g.n_pages);
      return -1;
    }
  s.reqs.push_back(Request{id, prompt_len, max_new, prompt_len, 0, s.next_arrival++, WAITING, 0});
  return 0;
}

// Build the next step.  `free_pages[g]`: free pages of each group now.  Fills, per planned
// request in serving order: id, first token index, token count, and whether the portion ends
// at the request's last token (its logits are wanted).  `preempted`: ids that must give up
// their pages before the step (at most `cap`).  Returns the number of entries, or -1.
int axh_sched_plan(void* h, const long* free_pages, int64_t* ids, long* starts, long* counts, int* wants, int cap,
                   int64_t* preempted_out, int* n_preempted) {
  Scheduler& s = *(Scheduler*)h;
  std::vector<long> free(free_pages, free_pages + s.groups.size());
  std::vector<int64_t> preempted;
  long budget = s.max_batch_tokens;
  for (Request& r : s.reqs) r.planned = 0;

  // 1. requests with one token left (decoding), oldest first; then 2. portions of the others.
  for (int phase = 0; phase < 2; ++phase) {
    for (size_t i = 0; i < s.reqs.size(); ++i) {
      Request& r = s.reqs[i];
      if (r.state != RUNNING || r.planned > 0) continue;
      const long remaining = r.total - r.computed;
      if ((phase == 0) != (remaining == 1)) continue;
      while (budget > 0) {
        long n = coverable(s, free, r.computed, std::min(remaining, budget));
        if (n > 0) {
          take(s, free, r.computed, r.computed + n);
          r.planned = n;
          budget -= n;
          break;
        }
        Request* v = victim_younger_than(s, r.arrival);
        if (!v) break;  // nobody younger to take pages from: it waits for the older ones
        preempt(s, *v, free, budget, preempted);
      }
    }
  }

  // 3. admission, first come first served: a slot, budget, and pages for the whole prompt and
  // one more token beyond what running prompts still need.
  int running = 0;
  for (const Request& r : s.reqs) running += r.state == RUNNING;
  for (size_t i = 0; i < s.reqs.size() && budget > 0 && running < s.max_seqs; ++i) {
    Request& r = s.reqs[i];
    if (r.state != WAITING) continue;
    if (std::find(preempted.begin(), preempted.end(), r.id) != preempted.end()) break;
    bool room = true;
    for (size_t g = 0; g < s.groups.size() && room; ++g) {
      long outstanding = 0;
      for (const Request& o : s.reqs)
        if (o.state == RUNNING) outstanding += pages_to_grow(s.groups[g], o.computed + o.planned, o.total);
      const long need = pages_covering(s.groups[g], std::min(r.total + 1, r.prompt_len + r.max_new));
      room = need <= free[g] - outstanding;
    }
    if (!room) break;
    const long n = coverable(s, free, 0, std::min(r.total, budget));
    if (n <= 0) break;
    r.state = RUNNING;
    ++running;
    take(s, free, 0, n);
    r.planned = n;
    budget -= n;
  }

  int n_entries = 0;
  for (int phase = 0; phase < 2; ++phase)
    for (const Request& r : s.reqs) {
      if (r.planned <= 0) continue;
      if ((phase == 0) != (r.total - r.computed == 1)) continue;
      if (n_entries >= cap) { s.error = "plan: more entries than the caller has room for"; return -1; }
      ids[n_entries] = r.id;
      starts[n_entries] = r.computed;
      counts[n_entries] = r.planned;
      wants[n_entries] = r.computed + r.planned == r.total;
      ++n_entries;
    }
  if ((int)preempted.size() > cap) { s.error = "plan: more preemptions than the caller has room for"; return -1; }
  for (size_t i = 0; i < preempted.size(); ++i) preempted_out[i] = preempted[i];
  *n_preempted = (int)preempted.size();
  return n_entries;
}

// The step ran `n_run` tokens of the request; `appended`: a new token was picked and joins
// it; `finished`: it is done (its pages are the caller's to give back).
int axh_sched_commit(void* h, int64_t id, long n_run, int appended, int finished) {
  Scheduler& s = *(Scheduler*)h;
  Request* r = find(s, id);
  if (!r || r->state != RUNNING || n_run != r->planned) {
    s.error = "commit: request " + std::to_string(id) + " was not planned with " + std::to_string(n_run) + " tokens";
    return -1;
  }
  r->computed += n_run;
  r->planned = 0;
  if (appended) r->total += 1;
  if (finished) s.reqs.erase(s.reqs.begin() + (r - s.reqs.data()));
  return 0;
}

// Drop a request wherever it is (cancelled).  1 if it was running (it held a slot), 0 if
// waiting, -1 if unknown.
int axh_sched_remove(void* h, int64_t id) {
  Scheduler& s = *(Scheduler*)h;
  Request* r = find(s, id);
  if (!r) return -1;
  const int was_running = r->state == RUNNING;
  s.reqs.erase(s.reqs.begin() + (r - s.reqs.data()));
  return was_running;
}

void axh_sched_counts(void* h, long* waiting, long* running, long* preemptions) {
  Scheduler& s = *(Scheduler*)h;
  long w = 0, r = 0;
  for (const Request& q : s.reqs) (q.state == RUNNING ? r : w) += 1;
  *waiting = w;
  *running = r;
  *preemptions = s.preemptions;
}

// computed / total of a request (for tests and for the caller's bookkeeping); -1 if unknown.
int axh_sched_progress(void* h, int64_t id, long* computed, long* total, int* state) {
  Scheduler& s = *(Scheduler*)h;
  Request* r = find(s, id);
  if (!r) return -1;
  *computed = r->computed;
  *total = r->total;
  *state = r->state;
  return 0;
}

}  // extern "C"
