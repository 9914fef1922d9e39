"""Builds the HIP kernels for gfx950 into one shared library and finds it again; and the host
runtime (cache accounting and step staging, plain C++) into a second one.

The library lives in-tree (`gibbs_amd/_lib/libgibbs_hip.so`) beside a stamp of the sources it
was built from.  `ensure_built()` returns the library if the stamp fits the sources; otherwise
it compiles (one hipcc process per file, a progress line per file), or fails loudly when there
is no compiler.  Nothing here needs a GPU: hipcc cross-compiles.
"""
from __future__ import annotations

import concurrent.futures
import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libgibbs_hip.so"
ARCH = "gfx950"
# packed-fp32 instructions are kept off for every kernel (the host pass warns that it does
# not know the feature; that is harmless).
HIPCC_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]
# In these files a kernel's first dwords of scalar arguments arrive in registers with the wave (gfx950 preloads
# them) instead of by a load that everything else in the kernel waits for; arguments passed as a struct are not
# preloaded.  It pays for the kernels of a decode step, which are short and many.
PRELOAD_FLAGS = ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
PRELOAD_FILES = {"gemm_skinny_fused.hip", "gemm_skinny_fused_rows.hip", "attention_decode.hip", "attention_decode_fused.hip"}


HOST_SRC = os.path.join(CSRC, "host")
HOST_LIB_NAME = "libgibbs_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall"]


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[gibbs_amd.build] {msg}", file=sys.stderr, flush=True)


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _stamp() -> str:
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS + PRELOAD_FLAGS + sorted(PRELOAD_FILES)).encode())
    return h.hexdigest()


def hipcc() -> str | None:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _lib_dirs() -> list[str]:
    """Where the library may live: in-tree first, else a per-user folder under the temp dir."""
    tmp = os.path.join(tempfile.gettempdir(), f"gibbs_amd-{os.getuid()}")
    return [os.path.join(HERE, "_lib"), tmp]


def _is_current(lib_dir: str, stamp: str, name: str = LIB_NAME) -> bool:
    lib, st = os.path.join(lib_dir, name), os.path.join(lib_dir, name + ".stamp")
    if not (os.path.isfile(lib) and os.path.isfile(st)):
        return False
    with open(st) as f:
        return f.read().strip() == stamp


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe-{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _compile_one(cc: str, src: str, obj: str, env: dict) -> tuple[str, float]:
    t0 = time.time()
    flags = HIPCC_FLAGS + (PRELOAD_FLAGS if os.path.basename(src) in PRELOAD_FILES else [])
    proc = subprocess.run([cc, *flags, "-c", src, "-o", obj], capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {os.path.basename(src)}:\n{proc.stderr[-4000:]}")
    return os.path.basename(src), time.time() - t0


def build(verbose: bool = True) -> str:
    """Compiles every kernel source and links the library; always compiles."""
    cc = hipcc()
    if cc is None:
        raise BuildError("hipcc not found: the HIP extension cannot be built (set HIPCC or install ROCm)")
    stamp = _stamp()
    lib_dir = next((d for d in _lib_dirs() if _writable(d)), None)
    if lib_dir is None:
        raise BuildError(f"no writable folder for the HIP extension among {_lib_dirs()}")
    obj_dir = os.path.join(lib_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())       # hipcc wants a HOME for its caches
    srcs = sources()
    if verbose:
        _say(f"compiling {len(srcs)} kernel files for {ARCH} into {lib_dir}")
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16))
    with concurrent.futures.ThreadPoolExecutor(workers) as pool:
        futures = [pool.submit(_compile_one, cc, s, o, env) for s, o in zip(srcs, objs)]
        for done, fut in enumerate(concurrent.futures.as_completed(futures), 1):
            name, secs = fut.result()
            if verbose:
                _say(f"  [{done}/{len(srcs)}] {name} ({secs:.1f}s)")
    tmp_lib = os.path.join(lib_dir, f".{LIB_NAME}.{os.getpid()}")
    # the library product (hipBLASLt) comes from the ROCm installation that hipcc belongs to; a process
    # that has loaded another copy of the same soname first (PyTorch brings one) keeps using that one
    rocm_lib = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(cc))), "lib")
    proc = subprocess.run([cc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, f"-L{rocm_lib}", "-lhipblaslt",
                           f"-Wl,-rpath,{rocm_lib}", "-o", tmp_lib], capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise BuildError(f"linking the HIP extension failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp_lib, os.path.join(lib_dir, LIB_NAME))
    with open(os.path.join(lib_dir, LIB_NAME + ".stamp"), "w") as f:
        f.write(stamp)
    if verbose:
        _say(f"built {os.path.join(lib_dir, LIB_NAME)}")
    return os.path.join(lib_dir, LIB_NAME)


def host_sources() -> list[str]:
    return sorted(glob.glob(os.path.join(HOST_SRC, "*.cpp")))


def _host_stamp() -> str:
    h = hashlib.sha256()
    for path in host_sources() + sorted(glob.glob(os.path.join(HOST_SRC, "*.h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()


def host_compiler() -> str | None:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"), hipcc()):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def build_host(verbose: bool = True) -> str:
    """Compiles the host runtime (no GPU code) into its library; always compiles."""
    cxx = host_compiler()
    if cxx is None:
        raise BuildError("no C++ compiler found: the host runtime cannot be built (set CXX)")
    lib_dir = next((d for d in _lib_dirs() if _writable(d)), None)
    if lib_dir is None:
        raise BuildError(f"no writable folder for the host runtime among {_lib_dirs()}")
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    tmp_lib = os.path.join(lib_dir, f".{HOST_LIB_NAME}.{os.getpid()}")
    t0 = time.time()
    proc = subprocess.run([cxx, *HOST_FLAGS, *host_sources(), "-o", tmp_lib], capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        raise BuildError(f"compiling the host runtime failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp_lib, os.path.join(lib_dir, HOST_LIB_NAME))
    with open(os.path.join(lib_dir, HOST_LIB_NAME + ".stamp"), "w") as f:
        f.write(_host_stamp())
    if verbose:
        _say(f"built {os.path.join(lib_dir, HOST_LIB_NAME)} ({time.time() - t0:.1f}s)")
    return os.path.join(lib_dir, HOST_LIB_NAME)


def ensure_host_built(verbose: bool = True) -> str:
    """The path of a host runtime library that fits its sources; builds it when there is none."""
    stamp = _host_stamp()
    for d in _lib_dirs():
        if _is_current(d, stamp, HOST_LIB_NAME):
            return os.path.join(d, HOST_LIB_NAME)
    return build_host(verbose=verbose)


def ensure_built(verbose: bool = True) -> str:
    """The path of a library that fits the sources; builds it when there is none."""
    stamp = _stamp()
    for d in _lib_dirs():
        if _is_current(d, stamp):
            return os.path.join(d, LIB_NAME)
    if hipcc() is None:
        stale = [d for d in _lib_dirs() if os.path.isfile(os.path.join(d, LIB_NAME))]
        raise BuildError(
            "the HIP extension is " + ("out of date" if stale else "missing") +
            " and hipcc was not found; build it with `python -c 'import __graft_entry__ as g; g.build()'`")
    return build(verbose=verbose)


if __name__ == "__main__":
    build_host()
    build()
