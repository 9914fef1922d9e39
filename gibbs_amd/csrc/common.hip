// Error channel of the library: the last failure's text, per host thread.
#include "common.h"
#include "packed_layout.h"

static thread_local char g_error[512] = "";

int gibbs_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

GIBBS_EXPORT const char* gibbs_last_error() { return g_error; }

// Version of the C interface; the Python side refuses a library built from other sources.
GIBBS_EXPORT int gibbs_abi_version() { return 1; }

// 16-row tiles below which a packed matrix (or each of its row groups) is in the pair layout (packed_layout.h);
// whoever packs weights asks here, so that the rule stands in one place.
GIBBS_EXPORT int gibbs_pair_layout_below_tiles() { return PAIR_LAYOUT_BELOW_TILES; }
