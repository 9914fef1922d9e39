// Declarations shared by the host runtime's sources: the failure channel, page pools and the
// cache core (see cache_core.cpp for what they do).
#pragma once
#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#define HOST_EXPORT extern "C" __attribute__((visibility("default")))

namespace gibbs_host {

constexpr int NO_PAGE = -1;

// failure codes (the Python side turns them into its exceptions)
constexpr int ERR_ARGUMENT = -1;     // a handle, group or size that does not exist
constexpr int ERR_PAGE = -2;         // a page freed twice, lost or held twice; a commit beyond the reserved pages
constexpr int ERR_NO_ROOM = -3;      // pages or slots ran out (nothing was taken)
constexpr int ERR_STEP = -4;         // an entry of a step is malformed (token id, wanted place, context limit)

inline thread_local char g_error[512] = "";

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

struct PagePool {
  int num_pages;
  std::vector<int> free_list;      // LIFO: a page that was just given back is the next to be used again
  std::vector<char> held;

  explicit PagePool(int n) : num_pages(n), held(n, 0) {
    free_list.reserve(n);
    for (int p = n - 1; p >= 0; --p) free_list.push_back(p);
  }
  int n_free() const { return (int)free_list.size(); }
  // n pages into out, or false (and nothing taken) if fewer are free
  bool allocate(int n, std::vector<int>& out) {
    if (n > n_free()) return false;
    for (int i = 0; i < n; ++i) {
      const int p = free_list.back();
      free_list.pop_back();
      held[p] = 1;
      out.push_back(p);
    }
    return true;
  }
  int release(int p) {
    if (p < 0 || p >= num_pages) return fail(ERR_PAGE, "page %d is not of this pool (0..%d)", p, num_pages - 1);
    if (!held[p]) return fail(ERR_PAGE, "page %d freed twice or never held", p);
    held[p] = 0;
    free_list.push_back(p);
    return 0;
  }
};

struct Request {
  bool live = false;
  long tokens = 0;                              // positions whose keys and state are cached
  std::vector<std::vector<int>> pages;          // group -> logical page -> id or NO_PAGE
};

struct CacheCore {
  int page_size, max_requests;
  std::vector<int> window;                      // per group; 0: every key stays visible
  std::vector<PagePool> pools;
  std::vector<Request> requests;                // by slot
  std::vector<int> free_slots, fresh_slots;

  int n_groups() const { return (int)pools.size(); }
  long pages_for(long n_tokens) const { return (n_tokens + page_size - 1) / page_size; }
  bool is_live(int slot) const { return slot >= 0 && slot < max_requests && requests[slot].live; }
  int pages_needed(const Request& r, long n_new, int group) const {
    return (int)std::max<long>(0, pages_for(r.tokens + n_new) - (long)r.pages[group].size());
  }
};

}  // namespace gibbs_host

// the cache core's interface, as the scheduler uses it (defined in cache_core.cpp)
HOST_EXPORT int gibbs_cache_admit(void* core);
HOST_EXPORT int gibbs_cache_reserve(void* core, int slot, long n_new);
HOST_EXPORT int gibbs_cache_release(void* core, int slot);
HOST_EXPORT long gibbs_cache_tokens(const void* core, int slot);
