// Host side of the cache manager: page pools with free lists, per-request block tables of every
// cache group, slots for per-request state, and the packing of one step's integer metadata into
// the staging buffer that travels to the device in one copy.  Plain C++ (no GPU calls), C interface.
//
// The accounting follows the reference's block pool (src/kv/mod.rs:337-430: a free
// list that allocation pops and release pushes) without its reference counts and prefix tree: a
// page belongs to at most one request.  Blocks are given back on the events the reference gives
// them back on (src/scheduler/mod.rs:1215-1217, :1561-1563), and, for a group with
// a window, as soon as no later query can see them.
//
// A live request is named by its slot index.  Every function returns 0 (or a count) on success
// and a negative code on failure; the text of the last failure is kept per thread.
#include "cache_core.h"

using namespace gibbs_host;

namespace {
int need_live(const CacheCore* c, int slot) {
  if (!c->is_live(slot)) return fail(ERR_ARGUMENT, "slot %d holds no live request", slot);
  return 0;
}

}  // namespace

HOST_EXPORT const char* gibbs_host_last_error() { return g_error; }
HOST_EXPORT int gibbs_host_abi_version() { return 1; }

// ------------------------------------------------------------------------------------------- page pool
HOST_EXPORT void* gibbs_pool_create(int num_pages) { return num_pages > 0 ? new PagePool(num_pages) : nullptr; }
HOST_EXPORT void gibbs_pool_destroy(void* pool) { delete (PagePool*)pool; }
HOST_EXPORT int gibbs_pool_free(const void* pool) { return ((const PagePool*)pool)->n_free(); }
HOST_EXPORT int gibbs_pool_is_held(const void* pool, int page) {
  const PagePool* p = (const PagePool*)pool;
  return page >= 0 && page < p->num_pages && p->held[page];
}
// n pages into out; ERR_NO_ROOM (and nothing taken) if fewer are free
HOST_EXPORT int gibbs_pool_allocate(void* pool, int n, int* out) {
  if (n < 0) return fail(ERR_ARGUMENT, "cannot allocate a negative number of pages");
  std::vector<int> got;
  if (!((PagePool*)pool)->allocate(n, got)) return fail(ERR_NO_ROOM, "%d pages wanted, %d free", n, ((PagePool*)pool)->n_free());
  std::copy(got.begin(), got.end(), out);
  return n;
}
HOST_EXPORT int gibbs_pool_release(void* pool, const int* pages, int n) {
  for (int i = 0; i < n; ++i)
    if (int e = ((PagePool*)pool)->release(pages[i])) return e;
  return 0;
}

// ------------------------------------------------------------------------------------------- cache core
// windows[g]: the window of group g, 0 for none; num_pages[g]: the pages of its pool (a group with a
// window needs fewer than one that keeps every key).
HOST_EXPORT void* gibbs_cache_create(int n_groups, const int* windows, int page_size, const int* num_pages, int max_requests) {
  if (n_groups < 0 || page_size <= 0 || max_requests <= 0) return nullptr;
  for (int g = 0; g < n_groups; ++g)
    if (num_pages[g] <= 0) return nullptr;
  CacheCore* c = new CacheCore();
  c->page_size = page_size;
  c->max_requests = max_requests;
  for (int g = 0; g < n_groups; ++g) {
    c->window.push_back(windows[g]);
    c->pools.emplace_back(num_pages[g]);
  }
  c->requests.resize(max_requests);
  for (int s = max_requests - 1; s >= 0; --s) c->free_slots.push_back(s);
  return c;
}
HOST_EXPORT void gibbs_cache_destroy(void* core) { delete (CacheCore*)core; }

HOST_EXPORT int gibbs_cache_free_pages(const void* core, int group) {
  const CacheCore* c = (const CacheCore*)core;
  if (group < 0 || group >= c->n_groups()) return fail(ERR_ARGUMENT, "no cache group %d", group);
  return c->pools[group].n_free();
}
HOST_EXPORT int gibbs_cache_free_slots(const void* core) { return (int)((const CacheCore*)core)->free_slots.size(); }

// A slot for a new request (cleared on the device before the next step), or ERR_NO_ROOM.
HOST_EXPORT int gibbs_cache_admit(void* core) {
  CacheCore* c = (CacheCore*)core;
  if (c->free_slots.empty()) return fail(ERR_NO_ROOM, "no free slot (%d live)", c->max_requests);
  const int slot = c->free_slots.back();
  c->free_slots.pop_back();
  Request& r = c->requests[slot];
  r.live = true;
  r.tokens = 0;
  r.pages.assign(c->n_groups(), {});
  c->fresh_slots.push_back(slot);
  return slot;
}

HOST_EXPORT long gibbs_cache_tokens(const void* core, int slot) {
  const CacheCore* c = (const CacheCore*)core;
  if (int e = need_live(c, slot)) return e;
  return c->requests[slot].tokens;
}

HOST_EXPORT int gibbs_cache_held_pages(const void* core, int slot, int group) {
  const CacheCore* c = (const CacheCore*)core;
  if (int e = need_live(c, slot)) return e;
  if (group < 0 || group >= c->n_groups()) return fail(ERR_ARGUMENT, "no cache group %d", group);
  return (int)c->requests[slot].pages[group].size();
}

// Per group: pages that a reservation of n_new more positions would have to take.
HOST_EXPORT int gibbs_cache_pages_needed(const void* core, int slot, long n_new, int* out) {
  const CacheCore* c = (const CacheCore*)core;
  if (int e = need_live(c, slot)) return e;
  for (int g = 0; g < c->n_groups(); ++g) out[g] = c->pages_needed(c->requests[slot], n_new, g);
  return 0;
}

// Pages for the next n_new positions in every group; all or nothing (ERR_NO_ROOM: nothing taken).
HOST_EXPORT int gibbs_cache_reserve(void* core, int slot, long n_new) {
  CacheCore* c = (CacheCore*)core;
  if (int e = need_live(c, slot)) return e;
  Request& r = c->requests[slot];
  for (int g = 0; g < c->n_groups(); ++g)
    if (c->pages_needed(r, n_new, g) > c->pools[g].n_free())
      return fail(ERR_NO_ROOM, "cache group %d: %d pages wanted, %d free", g, c->pages_needed(r, n_new, g), c->pools[g].n_free());
  for (int g = 0; g < c->n_groups(); ++g) c->pools[g].allocate(c->pages_needed(r, n_new, g), r.pages[g]);
  return 0;
}

// n_new more positions are cached now.  A window group gives back every page that no later query can
// see: page j holds positions [j * page_size, (j + 1) * page_size), the next query is at position
// >= tokens and sees keys > tokens - window.
HOST_EXPORT int gibbs_cache_commit(void* core, int slot, long n_new) {
  CacheCore* c = (CacheCore*)core;
  if (int e = need_live(c, slot)) return e;
  Request& r = c->requests[slot];
  for (int g = 0; g < c->n_groups(); ++g)
    if (c->pages_for(r.tokens + n_new) > (long)r.pages[g].size())
      return fail(ERR_PAGE, "commit of %ld tokens beyond its reserved pages", n_new);
  r.tokens += n_new;
  for (int g = 0; g < c->n_groups(); ++g) {
    if (c->window[g] <= 0) continue;
    const long first_visible = r.tokens - c->window[g] + 1;
    const long passed = std::min<long>(first_visible > 0 ? first_visible / c->page_size : 0, (long)r.pages[g].size());
    for (long j = 0; j < passed; ++j) {
      if (r.pages[g][j] == NO_PAGE) continue;
      if (int e = c->pools[g].release(r.pages[g][j])) return e;
      r.pages[g][j] = NO_PAGE;
    }
  }
  return 0;
}

// The same for several requests at once (the rows of a decode loop): pages for n_new more positions of every one
// of them, all or nothing.  Returns 1 if pages were taken, 0 if none were needed, ERR_NO_ROOM (nothing taken; need[g]
// says how many pages group g would have needed) or another error.  limit > 0: a request that would then hold more
// than `limit` positions is an argument error.
HOST_EXPORT int gibbs_cache_reserve_all(void* core, const int* slots, int n, long n_new, long limit, int* need) {
  CacheCore* c = (CacheCore*)core;
  std::vector<int> wanted(c->n_groups(), 0);
  for (int i = 0; i < n; ++i) {
    if (int e = need_live(c, slots[i])) return e;
    const Request& r = c->requests[slots[i]];
    if (limit > 0 && r.tokens + n_new > limit)
      return fail(ERR_ARGUMENT, "the request in slot %d would pass the context limit %ld", slots[i], limit);
    for (int g = 0; g < c->n_groups(); ++g) wanted[g] += c->pages_needed(r, n_new, g);
  }
  bool any = false, room = true;
  for (int g = 0; g < c->n_groups(); ++g) {
    if (need) need[g] = wanted[g];
    any = any || wanted[g] > 0;
    room = room && wanted[g] <= c->pools[g].n_free();
  }
  if (!room) return fail(ERR_NO_ROOM, "the decode steps want more pages than are free");
  for (int i = 0; i < n; ++i) {
    Request& r = c->requests[slots[i]];
    for (int g = 0; g < c->n_groups(); ++g) c->pools[g].allocate(c->pages_needed(r, n_new, g), r.pages[g]);
  }
  return any ? 1 : 0;
}

// n_new more positions of every one of several requests are cached now.
HOST_EXPORT int gibbs_cache_commit_all(void* core, const int* slots, int n, long n_new) {
  CacheCore* c = (CacheCore*)core;
  for (int i = 0; i < n; ++i) {      // (all of them or none)
    if (int e = need_live(c, slots[i])) return e;
    const Request& r = c->requests[slots[i]];
    for (int g = 0; g < c->n_groups(); ++g)
      if (c->pages_for(r.tokens + n_new) > (long)r.pages[g].size())
        return fail(ERR_PAGE, "commit of %ld tokens beyond its reserved pages", n_new);
  }
  for (int i = 0; i < n; ++i)
    if (int e = gibbs_cache_commit(core, slots[i], n_new)) return e;
  return 0;
}

// Gives back every page and the slot of a request that ended.
HOST_EXPORT int gibbs_cache_release(void* core, int slot) {
  CacheCore* c = (CacheCore*)core;
  if (int e = need_live(c, slot)) return e;
  Request& r = c->requests[slot];
  int status = 0;
  for (int g = 0; g < c->n_groups(); ++g)
    for (int p : r.pages[g])
      if (p != NO_PAGE)
        if (int e = c->pools[g].release(p)) status = e;
  r.live = false;
  r.pages.clear();
  c->free_slots.push_back(slot);
  // a slot that was taken and given back before any step ran is not fresh any more (its next taker
  // lists it again)
  c->fresh_slots.erase(std::remove(c->fresh_slots.begin(), c->fresh_slots.end(), slot), c->fresh_slots.end());
  return status;
}

// Slots taken since the last call (their state has to be cleared on the device); returns the count.
HOST_EXPORT int gibbs_cache_take_fresh_slots(void* core, int* out, int cap) {
  CacheCore* c = (CacheCore*)core;
  const int n = std::min<int>(cap, (int)c->fresh_slots.size());
  std::copy(c->fresh_slots.begin(), c->fresh_slots.begin() + n, out);
  c->fresh_slots.erase(c->fresh_slots.begin(), c->fresh_slots.begin() + n);
  return n;
}

HOST_EXPORT int gibbs_cache_table_width(const void* core, const int* slots, int n, int group) {
  const CacheCore* c = (const CacheCore*)core;
  if (group < 0 || group >= c->n_groups()) return fail(ERR_ARGUMENT, "no cache group %d", group);
  int width = 0;
  for (int i = 0; i < n; ++i) {
    if (int e = need_live(c, slots[i])) return e;
    width = std::max(width, (int)c->requests[slots[i]].pages[group].size());
  }
  return width;
}

// out[n, width]: page id of logical page j of each request (NO_PAGE beyond its pages and for pages a
// window has passed).
HOST_EXPORT int gibbs_cache_block_table(const void* core, const int* slots, int n, int group, int width, int* out) {
  const CacheCore* c = (const CacheCore*)core;
  if (group < 0 || group >= c->n_groups()) return fail(ERR_ARGUMENT, "no cache group %d", group);
  for (int i = 0; i < n; ++i) {
    if (int e = need_live(c, slots[i])) return e;
    const std::vector<int>& pages = c->requests[slots[i]].pages[group];
    if ((int)pages.size() > width)
      return fail(ERR_ARGUMENT, "entry %d holds %d pages, table width is %d", i, (int)pages.size(), width);
    int* row = out + (size_t)i * width;
    std::copy(pages.begin(), pages.end(), row);
    std::fill(row + pages.size(), row + width, NO_PAGE);
  }
  return 0;
}

// Invariants: no page lost, held twice or free while held; no slot shared or lost.
HOST_EXPORT int gibbs_cache_check(const void* core) {
  const CacheCore* c = (const CacheCore*)core;
  for (int g = 0; g < c->n_groups(); ++g) {
    const PagePool& pool = c->pools[g];
    std::vector<int> owner(pool.num_pages, -1);
    int owned = 0;
    for (int s = 0; s < c->max_requests; ++s) {
      if (!c->requests[s].live) continue;
      for (int p : c->requests[s].pages[g]) {
        if (p == NO_PAGE) continue;
        if (p < 0 || p >= pool.num_pages) return fail(ERR_PAGE, "group %d: slot %d holds page %d, not of the pool", g, s, p);
        if (owner[p] >= 0) return fail(ERR_PAGE, "group %d: page %d held by slots %d and %d", g, p, owner[p], s);
        if (!pool.held[p]) return fail(ERR_PAGE, "group %d: page %d of slot %d is on the free list", g, p, s);
        owner[p] = s;
        ++owned;
      }
    }
    if (owned != pool.num_pages - pool.n_free())
      return fail(ERR_PAGE, "group %d: %d pages held, %d owned: a page was lost", g, pool.num_pages - pool.n_free(), owned);
    std::vector<char> seen(pool.num_pages, 0);
    for (int p : pool.free_list) {
      if (seen[p]) return fail(ERR_PAGE, "group %d: page %d is on the free list twice", g, p);
      seen[p] = 1;
    }
  }
  std::vector<char> free_slot(c->max_requests, 0);
  for (int s : c->free_slots) {
    if (free_slot[s] || c->requests[s].live) return fail(ERR_PAGE, "slot %d is shared or free while held", s);
    free_slot[s] = 1;
  }
  int live = 0;
  for (int s = 0; s < c->max_requests; ++s) live += c->requests[s].live;
  if (live + (int)c->free_slots.size() != c->max_requests) return fail(ERR_PAGE, "a slot was lost");
  return 0;
}

// ------------------------------------------------------------------------------------------- one step
// Checks the entries of a step (slot[i] brings q_len[i] tokens, tokens flat in entry order; wanted
// places want[want_cu[i] .. want_cu[i+1]) relative to the entry) and takes their pages, all or nothing
// for the whole step.  On success info holds: total ints of the staging buffer, then per group the
// width of its block table.  On failure `bad` names the entry (ERR_STEP) or the group (ERR_NO_ROOM).
HOST_EXPORT int gibbs_cache_reserve_step(void* core, int n, const int* slots, const int* q_len, const int* tokens,
                                         const int* want_cu, const int* want, int vocab, long ctx_limit,
                                         long* info, int* bad) {
  CacheCore* c = (CacheCore*)core;
  if (n <= 0) return fail(ERR_STEP, "a step needs at least one entry");
  long rows = 0;
  for (int i = 0; i < n; ++i) {
    *bad = i;
    if (int e = need_live(c, slots[i])) return e;
    for (int j = 0; j < i; ++j)
      if (slots[j] == slots[i]) return fail(ERR_STEP, "appears twice in one step");
    if (q_len[i] <= 0) return fail(ERR_STEP, "no tokens");
    for (int t = 0; t < q_len[i]; ++t) {
      const int id = tokens[rows + t];
      if (id < 0 || id >= vocab) return fail(ERR_STEP, "token id %d outside the vocabulary (0..%d)", id, vocab - 1);
    }
    for (int w = want_cu[i]; w < want_cu[i + 1]; ++w)
      if (want[w] < 0 || want[w] >= q_len[i]) return fail(ERR_STEP, "wanted place outside its %d tokens", q_len[i]);
    const long after = c->requests[slots[i]].tokens + q_len[i];
    if (after > ctx_limit) return fail(ERR_STEP, "%ld tokens exceed the context limit %ld", after, ctx_limit);
    rows += q_len[i];
  }
  for (int g = 0; g < c->n_groups(); ++g) {
    long need = 0;
    for (int i = 0; i < n; ++i) need += c->pages_needed(c->requests[slots[i]], q_len[i], g);
    if (need > c->pools[g].n_free()) {
      *bad = g;
      return fail(ERR_NO_ROOM, "the step needs %ld pages of cache group %d, %d are free", need, g, c->pools[g].n_free());
    }
  }
  auto pad4 = [](long v) { return (v + 3) / 4 * 4; };   // every section starts on a 16-byte boundary
  long total = 3 * pad4(rows) + pad4(n + 1) + 2 * pad4(n) + pad4(want_cu[n]);
  for (int g = 0; g < c->n_groups(); ++g) {
    int width = 1;
    for (int i = 0; i < n; ++i) {
      Request& r = c->requests[slots[i]];
      c->pools[g].allocate(c->pages_needed(r, q_len[i], g), r.pages[g]);
      width = std::max(width, (int)r.pages[g].size());
    }
    info[1 + g] = width;
    total += pad4((long)n * width);
  }
  info[0] = std::max<long>(total, 4);
  return 0;
}

// Writes the step's metadata into out (the sizes that gibbs_cache_reserve_step reported) and the offset
// of every section into offsets: ids, pos, row_req, cu, ctx, slot, logit_rows, then one block table
// per group; then max q_len and the longest sequence after the step.
HOST_EXPORT int gibbs_cache_fill_step(const void* core, int n, const int* slots, const int* q_len, const int* tokens,
                                      const int* want_cu, const int* want, const long* info, int* out, long* offsets) {
  const CacheCore* c = (const CacheCore*)core;
  auto pad4 = [](long v) { return (v + 3) / 4 * 4; };
  long rows = 0;
  for (int i = 0; i < n; ++i) rows += q_len[i];
  long at = 0;
  int* ids = out + at; offsets[0] = at; at += pad4(rows);
  int* pos = out + at; offsets[1] = at; at += pad4(rows);
  int* row_req = out + at; offsets[2] = at; at += pad4(rows);
  int* cu = out + at; offsets[3] = at; at += pad4(n + 1);
  int* ctx = out + at; offsets[4] = at; at += pad4(n);
  int* slot = out + at; offsets[5] = at; at += pad4(n);
  int* logit_rows = out + at; offsets[6] = at; at += pad4(want_cu[n]);
  long row = 0, max_q = 0, max_seq = 0;
  for (int i = 0; i < n; ++i) {
    if (int e = need_live(c, slots[i])) return e;
    const long before = c->requests[slots[i]].tokens;
    cu[i] = (int)row;
    ctx[i] = (int)before;
    slot[i] = slots[i];
    for (int t = 0; t < q_len[i]; ++t) {
      ids[row + t] = tokens[row + t];
      pos[row + t] = (int)(before + t);
      row_req[row + t] = i;
    }
    for (int w = want_cu[i]; w < want_cu[i + 1]; ++w) logit_rows[w] = (int)row + want[w];
    row += q_len[i];
    max_q = std::max<long>(max_q, q_len[i]);
    max_seq = std::max<long>(max_seq, before + q_len[i]);
  }
  cu[n] = (int)row;
  for (int g = 0; g < c->n_groups(); ++g) {
    offsets[7 + g] = at;
    if (int e = gibbs_cache_block_table(core, slots, n, g, (int)info[1 + g], out + at)) return e;
    at += pad4((long)n * info[1 + g]);
  }
  offsets[7 + c->n_groups()] = max_q;
  offsets[8 + c->n_groups()] = max_seq;
  return 0;
}
