"""Loads the host runtime (page accounting, block tables, step staging, the scheduler's decisions: plain C++) and declares
its C interface.  Built at the first use when no current library is there; there is no Python
twin of it."""
from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, c_int, c_long, c_void_p

from .. import build as _build

ABI_VERSION = 1
ERR_ARGUMENT, ERR_PAGE, ERR_NO_ROOM, ERR_STEP = -1, -2, -3, -4
_lock = threading.Lock()
_lib = None
_ip, _lp = POINTER(c_int), POINTER(c_long)

_SIGNATURES = {
    "gibbs_pool_create": ([c_int], c_void_p),
    "gibbs_pool_destroy": ([c_void_p], None),
    "gibbs_pool_free": ([c_void_p], c_int),
    "gibbs_pool_is_held": ([c_void_p, c_int], c_int),
    "gibbs_pool_allocate": ([c_void_p, c_int, _ip], c_int),
    "gibbs_pool_release": ([c_void_p, _ip, c_int], c_int),
    "gibbs_cache_create": ([c_int, _ip, c_int, _ip, c_int], c_void_p),
    "gibbs_cache_destroy": ([c_void_p], None),
    "gibbs_cache_free_pages": ([c_void_p, c_int], c_int),
    "gibbs_cache_free_slots": ([c_void_p], c_int),
    "gibbs_cache_admit": ([c_void_p], c_int),
    "gibbs_cache_tokens": ([c_void_p, c_int], c_long),
    "gibbs_cache_held_pages": ([c_void_p, c_int, c_int], c_int),
    "gibbs_cache_pages_needed": ([c_void_p, c_int, c_long, _ip], c_int),
    "gibbs_cache_reserve": ([c_void_p, c_int, c_long], c_int),
    "gibbs_cache_commit": ([c_void_p, c_int, c_long], c_int),
    "gibbs_cache_reserve_all": ([c_void_p, _ip, c_int, c_long, c_long, _ip], c_int),
    "gibbs_cache_commit_all": ([c_void_p, _ip, c_int, c_long], c_int),
    "gibbs_cache_release": ([c_void_p, c_int], c_int),
    "gibbs_cache_take_fresh_slots": ([c_void_p, _ip, c_int], c_int),
    "gibbs_cache_table_width": ([c_void_p, _ip, c_int, c_int], c_int),
    "gibbs_cache_block_table": ([c_void_p, _ip, c_int, c_int, c_int, c_void_p], c_int),
    "gibbs_cache_check": ([c_void_p], c_int),
    "gibbs_cache_reserve_step": ([c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_long,
                                  _lp, _ip], c_int),
    "gibbs_sched_create": ([c_void_p, c_long, c_long, c_long], c_void_p),
    "gibbs_sched_destroy": ([c_void_p], None),
    "gibbs_sched_set_budget": ([c_void_p, c_long], c_int),
    "gibbs_sched_submit": ([c_void_p, c_long, c_long, c_int], c_int),
    "gibbs_sched_counts": ([c_void_p, _ip, _ip], c_int),
    "gibbs_sched_list": ([c_void_p, c_int, _ip, c_int], c_int),
    "gibbs_sched_query": ([c_void_p, c_int, _lp], c_int),
    "gibbs_sched_events": ([c_void_p, _lp, c_long], c_long),
    "gibbs_sched_plan": ([c_void_p, _lp, c_int, _lp, c_long, _lp], c_int),
    "gibbs_sched_apply": ([c_void_p, c_int, _ip, _ip, _ip, _lp, c_long, _lp], c_int),
    "gibbs_sched_fail_plan": ([c_void_p, _lp, c_long, _lp], c_int),
    "gibbs_sched_burst_plan": ([c_void_p, c_long, _ip, c_int, _ip, _lp], c_long),
    "gibbs_sched_apply_burst": ([c_void_p, c_int, _ip, c_int, _ip, _ip, c_int, _ip, _lp, c_long, _lp], c_int),
    "gibbs_cache_fill_step": ([c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, _lp, c_void_p, _lp],
                              c_int),
}


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                lib = ctypes.CDLL(_build.ensure_host_built())
                lib.gibbs_host_last_error.restype = ctypes.c_char_p
                lib.gibbs_host_abi_version.restype = c_int
                if lib.gibbs_host_abi_version() != ABI_VERSION:
                    raise RuntimeError(f"host runtime has interface version {lib.gibbs_host_abi_version()}, "
                                       f"expected {ABI_VERSION}")
                for name, (argtypes, restype) in _SIGNATURES.items():
                    fn = getattr(lib, name)
                    fn.argtypes, fn.restype = argtypes, restype
                _lib = lib
    return _lib


def last_error() -> str:
    return library().gibbs_host_last_error().decode(errors="replace")


def ints(values) -> ctypes.Array:
    values = list(values)
    return (c_int * max(1, len(values)))(*values)
