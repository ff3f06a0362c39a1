"""Builds the HIP kernels of csrc/ into one shared library for gfx950.

hipcc compiles each source file to an object (in parallel, a progress line per
file on stderr) and links them into `libllmengine_hip.so` beside this module, or,
where the checkout is read-only, into a per-user folder under the temporary
directory. A digest of the sources and flags is kept beside the library, so a
library built from other sources is never loaded by mistake.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.normpath(os.path.join(_HERE, "..", "..", "csrc"))
LIB_NAME = "libllmengine_hip.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # Packed 32-bit float instructions are kept out of every kernel.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]
# Flags for single sources. The attention kernels rescale their accumulators with ordinary
# arithmetic between matrix instructions: with the accumulators in the general registers the
# compiler does not copy them to and from the accumulation registers around every such step.
SOURCE_FLAGS = {
    "attention_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def flags_for(src: str) -> list[str]:
    return HIPCC_FLAGS + SOURCE_FLAGS.get(os.path.basename(src), [])


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[llmengine build] {msg}", file=sys.stderr, flush=True)


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def source_digest() -> str:
    h = hashlib.sha256()
    for path in sources() + _headers():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(repr(sorted(SOURCE_FLAGS.items())).encode())
    return h.hexdigest()[:24]


def _object_digest(src: str) -> str:
    h = hashlib.sha256()
    for path in [src] + _headers():
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(flags_for(src)).encode())
    return h.hexdigest()[:16]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                     "the HIP kernels cannot be built")


def _candidate_dirs() -> list[str]:
    tmp = os.path.join(tempfile.gettempdir(), f"llmengine-build-{os.getuid()}")
    return [_HERE, tmp]


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
    """Path of a library that matches the current sources, if one is built."""
    digest = source_digest()
    for d in _candidate_dirs():
        lib = os.path.join(d, LIB_NAME)
        stamp = lib + ".digest"
        if os.path.isfile(lib) and os.path.isfile(stamp):
            try:
                with open(stamp) as f:
                    if f.read().strip() == digest:
                        return lib
            except OSError:
                pass
    return None


def _compile_one(hipcc: str, src: str, obj: str, env: dict, reuse: bool) -> tuple[str, float]:
    t0 = time.time()
    if reuse and os.path.isfile(obj):          # same source, headers and flags: keep the object
        return src, 0.0
    cmd = [hipcc, *flags_for(src), "-I", CSRC, "-c", src, "-o", obj]
    tmp = obj + f".{os.getpid()}.tmp"
    cmd[-1] = tmp
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if p.returncode != 0:
        raise BuildError(f"hipcc failed on {os.path.basename(src)}:\n{p.stdout}")
    os.replace(tmp, obj)
    return src, time.time() - t0


def build(force: bool = True, reuse_objects: bool = False) -> str:
    """Compiles every kernel source and links the library; returns its path.
    reuse_objects keeps objects whose source, headers and flags have not changed."""
    if not force:
        lib = built_library()
        if lib:
            return lib
    hipcc = find_hipcc()
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError(f"no writable folder for the kernel library (tried {_candidate_dirs()})")
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    env = dict(os.environ)
    # hipcc keeps temporary files under HOME/TMPDIR; both may be missing for a bare user.
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env.get("HOME", ""), os.W_OK):
        env["HOME"] = obj_dir
    srcs = sources()
    digest = source_digest()
    _log(f"compiling {len(srcs)} kernel files for gfx950 into {out_dir}")
    jobs = max(1, min(len(srcs), 8, int(os.environ.get("MAX_JOBS", "8"))))
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + f".{_object_digest(s)}.o") for s in srcs]
    t0 = last = time.time()
    done = 0
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(_compile_one, hipcc, s, o, env, reuse_objects) for s, o in zip(srcs, objs)]
        pending = set(futures)
        while pending:
            finished = {f for f in pending if f.done()}
            for f in finished:
                src, dt = f.result()
                done += 1
                last = time.time()
                _log(f"  [{done}/{len(srcs)}] {os.path.basename(src)} ({dt:.1f} s)")
            pending -= finished
            if pending:
                time.sleep(0.25)
                if time.time() - last > 15:
                    last = time.time()
                    _log(f"  still compiling ({len(pending)} files left, {time.time() - t0:.0f} s)")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp_lib = lib + f".{os.getpid()}.tmp"
    p = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp_lib, *objs],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if p.returncode != 0:
        raise BuildError(f"linking {LIB_NAME} failed:\n{p.stdout}")
    os.replace(tmp_lib, lib)
    with open(lib + ".digest", "w") as f:
        f.write(digest + "\n")
    for name in os.listdir(obj_dir):        # objects of older sources
        if name.endswith(".o") and os.path.join(obj_dir, name) not in objs:
            try:
                os.remove(os.path.join(obj_dir, name))
            except OSError:
                pass
    _log(f"built {lib} in {time.time() - t0:.1f} s")
    return lib


def ensure_built() -> str:
    """The library for the current sources: the built one, or a fresh build."""
    return built_library() or build(force=True, reuse_objects=True)


if __name__ == "__main__":
    print(ensure_built())
