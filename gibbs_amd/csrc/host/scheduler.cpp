// The decisions of continuous batching: which waiting requests are admitted, how a step's budget of
// prompt tokens is handed out, which request is preempted when pages run out, and when a request
// ends.  Plain C++ behind a C interface; it works on lengths and counts only (the tokens themselves,
// the sampling parameters and the results stay with the caller) and takes slots and pages from the
// cache core directly.
//
// Policy of the reference's scheduler (src/scheduler/mod.rs:1128-1580): first-in
// first-out admission that stops at the first request that does not fit (:1155-1221); decoders first,
// then the shortest remaining prompt, while the oldest prefilling request keeps up to half the budget
// (:1235-1246, :1271-1283); one token per decoding request per step (:1376-1487); a request ends on an
// end token (not emitted), at its limit of new tokens or at the context limit (:1357-1373, :1505-1528).
// When pages run out (the reference goes on without them, :1296-1299, :1397-1400): a decoding request
// that cannot get its next page preempts the youngest running request, which returns to the head of
// the queue to be recomputed; a prompt portion shrinks to what is free or waits; if nothing can move
// the youngest is preempted; admission leaves the running requests the page of their next token; a
// request larger than the pool fails.
#include <deque>

#include "cache_core.h"

using namespace gibbs_host;

namespace {

enum State { WAITING = 0, PREFILLING = 1, DECODING = 2, FINISHED = 3 };
// what a call reports back, as (kind, request, value) triples
enum Event {
  EV_ADMITTED = 1,        // value: the slot it took
  EV_RELEASED = 2,        // its slot and pages went back (finished or preempted)
  EV_PREEMPTED = 3,
  EV_FINISHED_STOP = 4,
  EV_FINISHED_LENGTH = 5,
  EV_ERROR_TOO_LARGE = 6, // value: the pages it would need
  EV_ERROR_POOL = 7,      // alone and still no room
  EV_ERROR_STEP = 8,      // the step it was part of failed as a whole
};

struct Seq {
  long prompt_len = 0, output_len = 0, max_new = 0, submitted = 0;
  bool ignore_eos = false;
  int state = WAITING, slot = -1, preemptions = 0;
  long total() const { return prompt_len + output_len; }
};

struct Scheduler {
  CacheCore* cache;
  long context_len, budget, chunk;       // chunk 0: none
  std::vector<Seq> seqs;                 // by request number
  std::deque<int> waiting;
  std::vector<int> active;
  std::vector<int> planned;              // requests of the last plan, for a step that fails as a whole
  std::vector<long> events;

  void event(int kind, int id, long value = 0) {
    events.push_back(kind);
    events.push_back(id);
    events.push_back(value);
  }
  long computed(const Seq& s) const { return s.slot >= 0 ? cache->requests[s.slot].tokens : 0; }
  long remaining(const Seq& s) const { return s.total() - computed(s); }
  bool fits(const Seq& s, long n) const {
    for (int g = 0; g < cache->n_groups(); ++g)
      if (cache->pages_needed(cache->requests[s.slot], n, g) > cache->pools[g].n_free()) return false;
    return true;
  }
  long largest_fit(const Seq& s, long n) const {   // the most tokens <= n whose pages are free now
    long lo = 0, hi = n;
    while (lo < hi) {
      const long mid = (lo + hi + 1) / 2;
      if (fits(s, mid)) lo = mid;
      else hi = mid - 1;
    }
    return lo;
  }
  void drop_active(int id) { active.erase(std::remove(active.begin(), active.end(), id), active.end()); }
  void give_back(int id) {
    Seq& s = seqs[id];
    if (s.slot >= 0) {
      gibbs_cache_release(cache, s.slot);
      s.slot = -1;
      event(EV_RELEASED, id);
    }
  }
  void finish(int id, int kind, long value = 0) {
    seqs[id].state = FINISHED;
    give_back(id);
    drop_active(id);
    event(kind, id, value);
  }
  void preempt(int id) {
    give_back(id);
    drop_active(id);
    seqs[id].state = WAITING;
    seqs[id].preemptions += 1;
    waiting.push_front(id);
    event(EV_PREEMPTED, id);
  }
  int youngest() const {
    int best = active[0];
    for (int id : active)
      if (seqs[id].submitted > seqs[best].submitted) best = id;
    return best;
  }
  // a sampled token arrives for a request whose tokens are all cached; true if the request goes on
  bool take_token(int id, bool is_eos) {
    Seq& s = seqs[id];
    s.state = DECODING;
    if (is_eos && !s.ignore_eos) {
      finish(id, EV_FINISHED_STOP);                 // the end token is not emitted
      return false;
    }
    s.output_len += 1;
    if (s.output_len >= s.max_new || s.total() >= context_len) {
      finish(id, EV_FINISHED_LENGTH);
      return false;
    }
    return true;
  }
};

// Copies what fits (whole triples) and returns the number of events that happened; a caller whose
// buffer was too small asks for all of them again with gibbs_sched_events.
long copy_events(const Scheduler* s, long* out, long cap) {
  const long n = std::min<long>(cap / 3 * 3, (long)s->events.size());
  std::copy(s->events.begin(), s->events.begin() + n, out);
  return (long)s->events.size() / 3;
}

}  // namespace

HOST_EXPORT void* gibbs_sched_create(void* cache_core, long context_len, long max_batch_tokens, long chunk) {
  if (!cache_core || max_batch_tokens < 1 || chunk < 0) return nullptr;
  Scheduler* s = new Scheduler();
  s->cache = (CacheCore*)cache_core;
  s->context_len = context_len;
  s->budget = max_batch_tokens;
  s->chunk = chunk;
  return s;
}
HOST_EXPORT void gibbs_sched_destroy(void* sched) { delete (Scheduler*)sched; }
// The budget of prompt tokens of the steps planned from now on (a caller that sizes it by measured
// costs sets it before every plan).
HOST_EXPORT int gibbs_sched_set_budget(void* sched, long max_batch_tokens) {
  if (max_batch_tokens < 1) return fail(ERR_ARGUMENT, "a budget of %ld prompt tokens", max_batch_tokens);
  ((Scheduler*)sched)->budget = max_batch_tokens;
  return 0;
}

// Queues a request of prompt_len tokens that may generate max_new more; returns its number.
HOST_EXPORT int gibbs_sched_submit(void* sched, long prompt_len, long max_new, int ignore_eos) {
  Scheduler* s = (Scheduler*)sched;
  Seq q;
  q.prompt_len = prompt_len;
  q.max_new = max_new;
  q.ignore_eos = ignore_eos != 0;
  q.submitted = (long)s->seqs.size();
  s->seqs.push_back(q);
  s->waiting.push_back((int)s->seqs.size() - 1);
  return (int)s->seqs.size() - 1;
}

HOST_EXPORT int gibbs_sched_counts(const void* sched, int* n_waiting, int* n_active) {
  const Scheduler* s = (const Scheduler*)sched;
  *n_waiting = (int)s->waiting.size();
  *n_active = (int)s->active.size();
  return 0;
}
// The waiting queue (head first) or the running requests (in the order of the last plan).
HOST_EXPORT int gibbs_sched_list(const void* sched, int which, int* out, int cap) {
  const Scheduler* s = (const Scheduler*)sched;
  int n = 0;
  if (which == 0) {
    for (int id : s->waiting)
      if (n < cap) out[n++] = id;
  } else {
    for (int id : s->active)
      if (n < cap) out[n++] = id;
  }
  return n;
}
// state, output length, preemptions, slot of a request
HOST_EXPORT int gibbs_sched_query(const void* sched, int id, long* out) {
  const Scheduler* s = (const Scheduler*)sched;
  if (id < 0 || id >= (int)s->seqs.size()) return fail(ERR_ARGUMENT, "no request %d", id);
  const Seq& q = s->seqs[id];
  out[0] = q.state; out[1] = q.output_len; out[2] = q.preemptions; out[3] = q.slot;
  return 0;
}

// The events of the last call (they are kept until the next one).
HOST_EXPORT long gibbs_sched_events(const void* sched, long* out, long cap) { return copy_events((const Scheduler*)sched, out, cap); }

// Plans one step: admission, order, portions, preemption; pages and slots are taken here, so that the
// batch that runs is the batch that fits.  plan: (request, first token, token count, 1 if its last token is
// among them, 1 if it decodes) per planned request, in batch order; events: what happened on the way.
// Returns the number of planned requests.
HOST_EXPORT int gibbs_sched_plan(void* sched, long* plan, int plan_cap, long* events, long events_cap, long* n_events) {
  Scheduler* s = (Scheduler*)sched;
  CacheCore* c = s->cache;
  s->events.clear();
  s->planned.clear();
  const long budget = s->budget;
  const long cap = s->chunk > 0 ? std::min(budget, s->chunk) : budget;

  // 1. admission: first in, first out; needs a slot and the pages of the first portion, beside the
  //    page that every running request needs for its next token.  (Without that margin a request that
  //    was preempted to make room takes the freed page back at once, fills it, is preempted again, and
  //    the running requests that wait for a page never move.)
  std::vector<long> margin(c->n_groups(), 0);
  for (int id : s->active)
    for (int g = 0; g < c->n_groups(); ++g) margin[g] += c->pages_needed(c->requests[s->seqs[id].slot], 1, g);
  while (!s->waiting.empty()) {
    const int id = s->waiting.front();
    Seq& q = s->seqs[id];
    if (q.max_new == 0 && q.output_len == 0) {
      s->waiting.pop_front();
      s->finish(id, EV_FINISHED_LENGTH);                  // src/scheduler/mod.rs:1357-1359
      continue;
    }
    const long total = q.total();
    // a request that no pool can ever hold: every key in a group without a window; in a group with one,
    // the window and the portion that is reserved before the window moves on
    long short_by = 0;
    for (int g = 0; g < c->n_groups(); ++g) {
      long need = c->pages_for(total + 1);
      if (c->window[g] > 0) need = std::min(need, c->pages_for(c->window[g] + std::min(total, cap)) + 2);
      if (need > c->pools[g].num_pages) short_by = std::max(short_by, need);
    }
    if (short_by > 0) {
      s->waiting.pop_front();
      s->finish(id, EV_ERROR_TOO_LARGE, short_by);
      continue;
    }
    const int slot = gibbs_cache_admit(c);
    if (slot < 0) break;
    bool room = true;
    for (int g = 0; g < c->n_groups(); ++g)
      room = room && c->pages_needed(c->requests[slot], std::min(total, cap), g) + margin[g] <= c->pools[g].n_free();
    if (!room || gibbs_cache_reserve(c, slot, std::min(total, cap)) < 0) {
      gibbs_cache_release(c, slot);
      break;
    }
    s->waiting.pop_front();
    q.slot = slot;
    q.state = PREFILLING;
    s->active.push_back(id);
    s->event(EV_ADMITTED, id, slot);
  }

  // 2. order: decoders first, then the shortest remaining prompt; the oldest prefilling request keeps up
  //    to half the budget
  auto decoding = [&](int id) { return s->seqs[id].state == DECODING; };
  std::stable_sort(s->active.begin(), s->active.end(), [&](int a, int b) {
    const long ka = decoding(a) ? 0 : s->remaining(s->seqs[a]), kb = decoding(b) ? 0 : s->remaining(s->seqs[b]);
    return ka != kb ? ka < kb : s->seqs[a].submitted < s->seqs[b].submitted;
  });
  int oldest = -1;
  for (int id : s->active)
    if (!decoding(id) && (oldest < 0 || s->seqs[id].submitted < s->seqs[oldest].submitted)) oldest = id;
  long reserved = oldest >= 0 ? std::min(s->remaining(s->seqs[oldest]), (budget + 1) / 2) : 0;

  // 3. the plan
  struct Item { int id; long n; };
  std::vector<Item> items;
  long left = budget;
  const std::vector<int> order = s->active;
  for (int id : order) {
    if (std::find(s->active.begin(), s->active.end(), id) == s->active.end()) continue;   // preempted meanwhile
    Seq& q = s->seqs[id];
    if (decoding(id)) {
      bool alive = true;
      while (!s->fits(q, 1)) {
        const int victim = s->youngest();
        items.erase(std::remove_if(items.begin(), items.end(), [&](const Item& it) { return it.id == victim; }), items.end());
        s->preempt(victim);
        if (victim == id) {
          alive = false;
          break;
        }
      }
      if (alive) {
        gibbs_cache_reserve(c, q.slot, 1);
        items.push_back({id, 1});
      }
      continue;
    }
    long available;
    if (id == oldest) {
      available = left;
      reserved = 0;
    } else {
      available = std::max<long>(0, left - reserved);
    }
    long n = std::min(std::min(s->remaining(q), available), cap);
    if (n > 0 && !s->fits(q, n)) n = s->largest_fit(q, n);
    if (n <= 0) continue;                                   // budget or pages exhausted: next step
    gibbs_cache_reserve(c, q.slot, n);
    items.push_back({id, n});
    left -= n;
  }
  if (items.empty() && !s->active.empty()) {
    // nothing can move: make room for the oldest by preempting the youngest
    const int victim = s->youngest();
    if (s->active.size() == 1) s->finish(victim, EV_ERROR_POOL);
    else s->preempt(victim);
  }
  int n_plan = 0;
  for (const Item& it : items) {
    if (n_plan >= plan_cap) return fail(ERR_ARGUMENT, "the plan holds more than %d requests", plan_cap);
    const Seq& q = s->seqs[it.id];
    const long at = s->computed(q);
    long* row = plan + 5 * n_plan++;
    row[0] = it.id; row[1] = at; row[2] = it.n; row[3] = at + it.n == q.total(); row[4] = q.state == DECODING;
    s->planned.push_back(it.id);
  }
  *n_events = copy_events(s, events, events_cap);
  return n_plan;
}

// The tokens that the step sampled, for the planned requests whose last token was in it (in plan order):
// is_eos[i] says whether token i ends its request.  emitted[i] = 1 if the token counts as output.
HOST_EXPORT int gibbs_sched_apply(void* sched, int n, const int* ids, const int* is_eos, int* emitted, long* events,
                                  long events_cap, long* n_events) {
  Scheduler* s = (Scheduler*)sched;
  s->events.clear();
  for (int i = 0; i < n; ++i) {
    if (ids[i] < 0 || ids[i] >= (int)s->seqs.size()) return fail(ERR_ARGUMENT, "no request %d", ids[i]);
    const long before = s->seqs[ids[i]].output_len;
    s->take_token(ids[i], is_eos[i] != 0);
    emitted[i] = s->seqs[ids[i]].output_len > before;
  }
  *n_events = copy_events(s, events, events_cap);
  return 0;
}

// The step failed as a whole: every planned request ends (the caller records the error).
HOST_EXPORT int gibbs_sched_fail_plan(void* sched, long* events, long events_cap, long* n_events) {
  Scheduler* s = (Scheduler*)sched;
  s->events.clear();
  for (int id : s->planned)
    if (s->seqs[id].state != FINISHED) s->finish(id, EV_ERROR_STEP);
  s->planned.clear();
  *n_events = copy_events(s, events, events_cap);
  return 0;
}

// Several decode steps back to back: when nothing waits and every running request decodes with one
// token to feed, the requests (oldest first) into out and the steps all of them can still take (at most
// cap); 0 when a step has anything else to do.  *longest: the steps until the last of them reaches its token
// limit (at most cap, and within every request's context): a burst may run that long, the tokens that a request
// samples beyond its limit are dropped when the burst is booked, as those behind an end-of-sequence token are.
HOST_EXPORT long gibbs_sched_burst_plan(const void* sched, long cap, int* out, int out_cap, int* n_out, long* longest) {
  const Scheduler* s = (const Scheduler*)sched;
  *n_out = 0;
  if (longest) *longest = 0;
  if (!s->waiting.empty() || s->active.empty() || (int)s->active.size() > out_cap) return 0;
  long n = cap, room = cap, last = 0;
  for (int id : s->active) {
    const Seq& q = s->seqs[id];
    if (q.state != DECODING || s->remaining(q) != 1) return 0;
    room = std::min(room, (long)(s->context_len - q.total()));
    n = std::min(n, (long)(q.max_new - q.output_len));
    last = std::max(last, (long)(q.max_new - q.output_len));
  }
  n = std::min(n, room);
  if (n < 1) return 0;
  if (longest) *longest = std::max(n, std::min(last, room));
  std::vector<int> order = s->active;
  std::sort(order.begin(), order.end(), [&](int a, int b) { return s->seqs[a].submitted < s->seqs[b].submitted; });
  std::copy(order.begin(), order.end(), out);
  *n_out = (int)order.size();
  return n;
}

// Books the tokens of a burst (all already cached), request by request and token by token, by the rules of a step:
// tokens[i * n + j] is what request ids[i] sampled at step j, eos the ids that end a sequence.  took[i]: how many of
// request i's tokens count as output (the request may end among them).
HOST_EXPORT int gibbs_sched_apply_burst(void* sched, int n_req, const int* ids, int n, const int* tokens, const int* eos,
                                        int n_eos, int* took, long* events, long events_cap, long* n_events) {
  Scheduler* s = (Scheduler*)sched;
  s->events.clear();
  for (int i = 0; i < n_req; ++i)
    if (ids[i] < 0 || ids[i] >= (int)s->seqs.size()) return fail(ERR_ARGUMENT, "no request %d", ids[i]);
  for (int i = 0; i < n_req; ++i) {
    const long before = s->seqs[ids[i]].output_len;
    for (int j = 0; j < n; ++j) {
      const int token = tokens[(long)i * n + j];
      const bool is_eos = std::find(eos, eos + n_eos, token) != eos + n_eos;
      if (!s->take_token(ids[i], is_eos)) break;
    }
    took[i] = (int)(s->seqs[ids[i]].output_len - before);
  }
  *n_events = copy_events(s, events, events_cap);
  return 0;
}
