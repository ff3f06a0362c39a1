"""Builds and loads the host runtime library (csrc/host/*.cpp: plain C++17, no GPU calls).

The reference's runtime (block manager, paged cache bookkeeping, schedulers) is C++
(src/paged_kv.cpp, src/scheduler.cpp); so is this one. The Python classes
`llmengine.cache.CacheManager` and `llmengine.engine.ContinuousBatchScheduler` are its faces:
they translate names and errors and hold no state of their own. There is no Python
implementation behind them: without the library they raise `HostLibraryError`.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

_HERE = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "..", "csrc", "host"))
LIB_NAME = "libllmengine_host.so"
CXX_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wextra"]


class HostLibraryError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[llmengine build] {msg}", file=sys.stderr, flush=True)


def sources() -> list[str]:
    return sorted(os.path.join(SRC_DIR, f) for f in os.listdir(SRC_DIR) if f.endswith(".cpp"))


def source_digest() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(SRC_DIR)):
        if name.endswith((".cpp", ".h")):
            h.update(name.encode())
            with open(os.path.join(SRC_DIR, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(CXX_FLAGS).encode())
    return h.hexdigest()[:24]


def _candidate_dirs() -> list[str]:
    return [_HERE, os.path.join(tempfile.gettempdir(), f"llmengine-build-{os.getuid()}")]


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe-{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def built_library() -> str | None:
    digest = source_digest()
    for d in _candidate_dirs():
        lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, LIB_NAME + ".digest")
        try:
            if os.path.isfile(lib) and open(stamp).read().strip() == digest:
                return lib
        except OSError:
            pass
    return None


def find_cxx() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/bin/amdclang++"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise HostLibraryError("no C++ compiler found (looked at $CXX, g++, c++, clang++, /opt/rocm/bin/amdclang++)")


def build(force: bool = True) -> str:
    """Compiles csrc/host into the host runtime library; returns its path."""
    if not force:
        lib = built_library()
        if lib:
            return lib
    cxx = find_cxx()
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise HostLibraryError(f"no writable folder for the host runtime library (tried {_candidate_dirs()})")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".{os.getpid()}.tmp"
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    p = subprocess.run([cxx, *CXX_FLAGS, "-I", SRC_DIR, "-o", tmp, *sources()], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, env=env)
    if p.returncode != 0:
        raise HostLibraryError(f"compiling the host runtime failed:\n{p.stdout}")
    os.replace(tmp, lib)
    with open(lib + ".digest", "w") as f:
        f.write(source_digest() + "\n")
    _log(f"built {lib} in {time.time() - t0:.1f} s")
    return lib


_lib = None
_lock = threading.Lock()

_vp, _i, _l, _i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_int64
_f, _d = ctypes.c_float, ctypes.c_double
_pi, _pl, _pi64 = ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_long), ctypes.POINTER(ctypes.c_int64)

_SIGNATURES = {
    # name: (result, arguments)
    "llme_pool_create": (_vp, [_i]), "llme_pool_destroy": (None, [_vp]), "llme_pool_allocate": (_i, [_vp]),
    "llme_pool_free": (_i, [_vp, _i]), "llme_pool_free_pages": (_i, [_vp]), "llme_pool_is_held": (_i, [_vp, _i]),
    "llme_cm_create": (_vp, [_i, _pi, _pi, _pi, _i, _i]), "llme_cm_destroy": (None, [_vp]),
    "llme_cm_num_groups": (_i, [_vp]), "llme_cm_admit": (_i, [_vp, _i64]), "llme_cm_is_live": (_i, [_vp, _i64]),
    "llme_cm_slot": (_i, [_vp, _i64]), "llme_cm_length": (_l, [_vp, _i64]), "llme_cm_free_slots": (_i, [_vp]),
    "llme_cm_live": (_i, [_vp, _pi64, _i]), "llme_cm_pages_needed": (_i, [_vp, _i64, _l, _pi]),
    "llme_cm_can_reserve": (_i, [_vp, _i64, _l, _pi]), "llme_cm_reserve_batch": (_i, [_vp, _i, _pi64, _pl]),
    "llme_cm_commit": (_i, [_vp, _i64, _l]), "llme_cm_release": (_i, [_vp, _i64]),
    "llme_cm_table_len": (_i, [_vp, _i64, _i]), "llme_cm_table_copy": (_i, [_vp, _i64, _i, _i, _i, _pi]),
    "llme_cm_free_pages": (_i, [_vp, _i]), "llme_cm_num_pages": (_i, [_vp, _i]), "llme_cm_check": (_i, [_vp]),
    "llme_cm_decode_begin": (_i, [_vp, _i, _pi64, _pi, _l]), "llme_cm_commit_batch": (_i, [_vp, _i, _pi64, _l]),
    "llme_cm_fill_decode": (_i, [_vp, _i, _pi64, _i, _vp, _vp, _vp, _pi, _pi64]),
    "llme_cm_lengths": (_i, [_vp, _i, _pi64, _pl]),
    "llme_cm_fill_step": (_l, [_vp, _i, _pi64, _pi, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "llme_sched_create": (_vp, [_vp, _i, _l]), "llme_sched_destroy": (None, [_vp]),
    "llme_sched_set_budget": (_i, [_vp, _l]), "llme_sched_set_decode_round": (_i, [_vp, _i]),
    "llme_sched_set_row_round": (_i, [_vp, _l, _l]), "llme_sched_enqueue": (_l, [_vp, _pi, _l, _l]),
    "llme_sched_idle": (_i, [_vp]), "llme_sched_counts": (None, [_vp, _pi]),
    "llme_sched_plan": (_i, [_vp, _pi, _pi, _pi64, _pi, _pi, _pl, _pi, _l]),
    "llme_sched_complete": (_i, [_vp, _pi, _i, _pi, _i]), "llme_sched_num_results": (_i, [_vp]),
    "llme_sched_result_info": (_i, [_vp, _i, _pi64, _pl, _pl, _pi]), "llme_sched_result_tokens": (_i, [_vp, _i, _pi]),
    "llme_sched_clear_results": (None, [_vp]), "llme_sched_abort": (None, [_vp]), "llme_sched_fail": (_i, [_vp]),
    # launch planning (csrc/host/decode_plan.cpp)
    "llme_decode_cut": (_i, [_pi, _i, _i, _i, _i, _l, _i, _i, _d, _d, _d, _d, _d, _d, _d]),
    # plain C++ twins of the device kernels (csrc/host/plain_kernels.cpp), for tests
    "llme_plain_embed": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "llme_plain_rmsnorm": (_i, [_vp, _vp, _i, _i, _f, _vp]),
    "llme_plain_linear": (_i, [_vp, _vp, _i, _i, _i, _vp, _i]),
    "llme_plain_swiglu": (_i, [_vp, _vp, ctypes.c_size_t, _vp]),
    "llme_plain_inv_freq": (_i, [_i, _d, _i, _d, _d, _d, _d, _vp]),
    "llme_plain_rope_tables": (_i, [_vp, _vp, _i, _i, _vp, _vp]),
    "llme_plain_rope_apply": (_i, [_vp, _vp, _vp, _i, _i, _i]),
    "llme_plain_attention": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "llme_plain_argmax": (_i, [_vp, _i]),
    "llme_plain_sample": (_i, [_vp, _i, _f, _f]),
    # the whole model out of them (csrc/host/plain_model.cpp)
    "llme_plain_llama_forward": (_i, [_vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
}

# codes of csrc/host/host_api.h
ALREADY_LIVE, NO_SLOT, NOT_LIVE, NOT_RESERVED, NOT_HELD, BAD_ARGUMENT = -1, -2, -3, -4, -5, -6
CHECK_MESSAGES = {-10: "a page is in two block tables", -11: "pages held differ from pages in tables",
                  -12: "pages lost", -13: "a slot is held twice", -14: "a slot is lost"}


def library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            try:
                lib = ctypes.CDLL(built_library() or build(force=True))
            except OSError as e:
                raise HostLibraryError(f"the host runtime library cannot be loaded: {e}") from e
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype, fn.argtypes = res, args
            _lib = lib
    return _lib


if __name__ == "__main__":
    print(built_library() or build(force=True))
