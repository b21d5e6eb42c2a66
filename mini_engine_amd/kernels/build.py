"""Compile the HIP sources for gfx950 into shared libraries and find them again.

Two kinds of library: ``libme_core.so`` (every kernel that takes its sizes at run
time) and ``libme_attn_d<D>.so`` (the MFMA attention kernels, specialised per
head size). A library is rebuilt when the hash of its sources and flags differs
from the one recorded beside it. Libraries live in ``mini_engine_amd/lib`` when
that folder can be written, else in a per-user folder under the temp directory.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
PKG_LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib")

ARCH = "gfx950"
# -packed-fp32-ops is switched off: the compiler must not form packed float32 instructions.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]
CORE_SOURCES = ["elementwise.hip", "rope_kv.hip", "attention_simple.hip",
                "gemm.hip", "gemm_mid.hip", "gemm_library.hip", "sampling.hip"]
ATTN_SOURCE = "attention_mfma.hip"
HEADERS = ["common.h", "errors.inc", "sampling.h"]
# Head sizes that build_all() compiles ahead of use; any other multiple of 16 up to 512 is compiled when a model first needs it.
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 128)

_locks: dict = {}
_locks_guard = threading.Lock()


def _lock_for(name: str) -> threading.Lock:
    with _locks_guard:
        return _locks.setdefault(name, threading.Lock())


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[mini_engine_amd] {msg}", file=sys.stderr, flush=True)


def hipcc_path() -> str | None:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _hash(sources: list, extra: list) -> str:
    h = hashlib.sha256()
    for name in sources + HEADERS:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS + extra).encode())
    return h.hexdigest()[:16]


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        fd, probe = tempfile.mkstemp(prefix=".w", dir=path)
        os.close(fd)
        os.remove(probe)
        return True
    except OSError:
        return False


def _own_private_dir(path: str) -> bool:
    """Whether `path` is a real folder of this user that nobody else can write to or read."""
    try:
        st = os.lstat(path)
    except OSError:
        return False
    import stat
    return stat.S_ISDIR(st.st_mode) and st.st_uid == os.getuid() and (st.st_mode & 0o077) == 0


_fallback: str | None = None


def _fallback_dir() -> str:
    """A per-user folder under the temp directory. A folder of that name that is someone else's, a link,
    or open to others is never used (a library planted there would be loaded): a fresh one is made."""
    global _fallback
    if _fallback is None:
        base = os.path.join(tempfile.gettempdir(), f"mini_engine_amd-{os.getuid()}")
        try:
            os.mkdir(base, 0o700)
        except FileExistsError:
            pass
        _fallback = base if _own_private_dir(base) else tempfile.mkdtemp(prefix=f"mini_engine_amd-{os.getuid()}-")
    return _fallback


def _lib_dirs() -> list:
    dirs = [PKG_LIB]
    fb = _fallback or os.path.join(tempfile.gettempdir(), f"mini_engine_amd-{os.getuid()}")
    if _own_private_dir(fb):
        dirs.append(fb)
    return dirs


def _up_to_date(lib: str, digest: str) -> bool:
    try:
        with open(lib + ".hash") as f:
            return f.read().strip() == digest and os.path.isfile(lib)
    except OSError:
        return False


def _run(cmd: list, what: str) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed (exit {proc.returncode}):\n{' '.join(cmd)}\n{proc.stderr[-4000:]}")


def _compile_lib(name: str, sources: list, extra: list, digest: str, out_dir: str) -> str:
    hipcc = hipcc_path()
    if hipcc is None:
        raise BuildError(f"{name} is not built and hipcc was not found (set HIPCC or add /opt/rocm/bin to PATH)")
    obj_dir = os.path.join(out_dir, "_build", name + "-" + digest)
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.splitext(s)[0] + ".o") for s in sources]

    def one(src, obj):
        _run([hipcc, *HIPCC_FLAGS, *extra, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj], src)
        return src

    t0 = time.time()
    _log(f"compiling {name} for {ARCH} ({len(sources)} source file(s)) ...")
    done = []
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        futures = [pool.submit(one, s, o) for s, o in zip(sources, objs)]
        pending = set(futures)
        while pending:
            finished = {f for f in pending if f.done()}
            for f in finished:
                done.append(f.result())
            pending -= finished
            if pending:
                time.sleep(0.5)
                if int(time.time() - t0) % 10 == 0 and time.time() - t0 > 1:
                    _log(f"  ... {name}: {len(done)}/{len(sources)} files after {time.time() - t0:.0f}s")
                    time.sleep(1.0)
    lib = os.path.join(out_dir, name)
    tmp = lib + f".tmp{os.getpid()}"
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs], name)
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(digest)
    shutil.rmtree(obj_dir, ignore_errors=True)
    _log(f"built {lib} in {time.time() - t0:.1f}s")
    return lib


def _ensure(name: str, sources: list, extra: list, force: bool) -> str:
    digest = _hash(sources, extra)
    with _lock_for(name):
        if not force:
            for d in _lib_dirs():
                lib = os.path.join(d, name)
                if _up_to_date(lib, digest):
                    return lib
            stale = [os.path.join(d, name) for d in _lib_dirs() if os.path.isfile(os.path.join(d, name))]
            if stale and hipcc_path() is None:
                raise BuildError(f"{stale[0]} was built from other sources and hipcc is not available to rebuild it")
        out_dir = PKG_LIB if _writable_dir(PKG_LIB) else _fallback_dir()
        return _compile_lib(name, sources, extra, digest, out_dir)


def core_library(force: bool = False) -> str:
    return _ensure("libme_core.so", CORE_SOURCES, [], force)


def attention_library(head_dim: int, force: bool = False) -> str:
    if head_dim % 16 or not 16 <= head_dim <= 512:
        raise BuildError(f"the bf16 attention kernels need a head size that is a multiple of 16 in 16..512, got {head_dim}")
    return _ensure(f"libme_attn_d{head_dim}.so", [ATTN_SOURCE], [f"-DME_HEAD_DIM={head_dim}"], force)


def build_all(head_dims=DEFAULT_HEAD_DIMS, force: bool = True) -> list:
    """Compile every library (used by the repository's build check)."""
    libs = [core_library(force=force)]
    with ThreadPoolExecutor(max_workers=4) as pool:
        libs += list(pool.map(lambda d: attention_library(d, force=force), head_dims))
    return libs
