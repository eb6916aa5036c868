"""Builds and loads the HIP kernel library for gfx950.

The sources under csrc/ are compiled with hipcc into one shared library that is
loaded with ctypes; kernels receive raw device pointers and the current HIP
stream.  Nothing here falls back to the CPU: if the library cannot be built or
loaded, `load()` raises.

The library is looked for in-tree (`_lib/` beside this package) and is rebuilt
when a source is newer than it.  If the tree is not writable the build goes to
a per-user folder under the system's temporary directory.
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
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")
LIB_NAME = "libtinyllm_gfx950.so"
ARCH = "gfx950"
# -packed-fp32-ops is switched off: hipcc would otherwise form v_pk_*_f32 from scalar code.
HIPCC_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument", "-Wno-unknown-attributes"]

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


class KernelLibraryError(RuntimeError):
    pass


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def _source_digest() -> str:
    h = hashlib.sha256()
    for p in sources() + _headers():
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelLibraryError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                             "the engine has no path without its HIP kernels")


def _intree_dir() -> str:
    return os.path.join(_PKG, "_lib")


def _intree_writable() -> bool:
    intree = _intree_dir()
    try:
        os.makedirs(intree, exist_ok=True)
        probe = os.path.join(intree, f".probe-{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _private_temp_dir() -> str:
    """A build folder of this user's own under the system's temporary directory: made with mode
    0700, and refused unless it belongs to this user and nobody else can write to it (another
    user could otherwise plant a library there that this process would load)."""
    d = os.path.join(tempfile.gettempdir(), f"tinyllm-amd-{os.getuid()}")
    try:
        os.mkdir(d, 0o700)
    except FileExistsError:
        pass
    st = os.lstat(d)
    import stat as _stat
    if not _stat.S_ISDIR(st.st_mode) or st.st_uid != os.getuid() or (st.st_mode & 0o022):
        return tempfile.mkdtemp(prefix="tinyllm-amd-")
    return d


def _writable_dir() -> str:
    return _intree_dir() if _intree_writable() else _private_temp_dir()


def _candidates() -> List[str]:
    """Where a built library may lie: in the tree; the private temporary folder only when the tree
    cannot be written to."""
    return [_intree_dir()] if _intree_writable() else [_intree_dir(), _private_temp_dir()]


def _is_current(lib_path: str) -> bool:
    stamp = lib_path + ".digest"
    if not (os.path.exists(lib_path) and os.path.exists(stamp)):
        return False
    try:
        with open(stamp) as f:
            return f.read().strip() == _source_digest()
    except OSError:
        return False


def build(force: bool = True, verbose: bool = True) -> str:
    """Compile every .hip source for gfx950 and link the library.  Returns its path."""
    out_dir = _writable_dir()
    lib_path = os.path.join(out_dir, LIB_NAME)
    if not force and _is_current(lib_path):
        return lib_path
    hipcc = _hipcc()
    # objects of this build alone: two processes that build at once never link each other's halves
    obj_dir = os.path.join(out_dir, f"obj.{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)  # hipcc wants a place for its caches
    t0 = time.time()

    def say(msg):
        if verbose:
            print(f"[tiny-llm_amd build] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} HIP sources for {ARCH} into {lib_path}")

    def compile_one(src):
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, env=env, text=True)
        if p.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src}:\n{p.stderr[-4000:]}")
        say(f"  {os.path.basename(src)} done ({time.time() - t0:.0f}s)")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        futs = [pool.submit(compile_one, s) for s in srcs]
        while True:
            pending = [f for f in futs if not f.done()]
            if not pending:
                break
            time.sleep(0.2)
            if verbose and int(time.time() - t0) % 20 == 0 and time.time() - t0 > 19:
                say(f"  still compiling, {len(pending)} sources left ({time.time() - t0:.0f}s)")
                time.sleep(1.0)
        objs = [f.result() for f in futs]
    tmp = lib_path + f".tmp{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, env=env, text=True)
    if p.returncode != 0:
        raise KernelLibraryError(f"linking {lib_path} failed:\n{p.stderr[-4000:]}")
    import fcntl
    with open(os.path.join(out_dir, ".lock"), "w") as lock:      # library and stamp change together
        fcntl.flock(lock, fcntl.LOCK_EX)
        os.replace(tmp, lib_path)
        with open(lib_path + ".digest", "w") as f:
            f.write(_source_digest())
    shutil.rmtree(obj_dir, ignore_errors=True)
    say(f"built in {time.time() - t0:.0f}s")
    return lib_path


def find_or_build(verbose: bool = True) -> str:
    for d in _candidates():
        p = os.path.join(d, LIB_NAME)
        if _is_current(p):
            return p
    # A library whose digest does not match the sources is stale; one that was
    # shipped without a digest file next to sources we cannot compile is used as is.
    try:
        return build(force=True, verbose=verbose)
    except KernelLibraryError:
        for d in _candidates():
            p = os.path.join(d, LIB_NAME)
            if os.path.exists(p) and not os.path.exists(p + ".digest"):
                return p
        raise


def load(verbose: bool = True) -> ctypes.CDLL:
    """The loaded library; built first if no current build exists."""
    global _lib
    with _lock:
        if _lib is None:
            path = find_or_build(verbose=verbose)
            try:
                _lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelLibraryError(f"cannot load {path}: {e}") from e
            _lib._path = path
        return _lib
