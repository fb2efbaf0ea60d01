"""Building and loading the gfx950 kernel libraries.

Each ``csrc/<name>.hip`` becomes one shared object ``_build/<name>.so`` with plain
``extern "C"`` entry points, compiled by ``hipcc --offload-arch=gfx950`` and loaded through
``ctypes``.  A library is compiled the first time an op needs it (only what the running
model uses), or all at once by :func:`build_all`.  A stamp beside each object holds the
hash of its sources and flags, so an object built from older sources is rebuilt rather
than used.  There is no fallback: a library that cannot be built or loaded raises.
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
from typing import Dict, Iterable, List, Optional

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
HEADERS = ("common.h", "common_impl.h", "mfma.h", "qk_rope.h", "noalloc.h")
ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

LIBRARIES = ("elementwise", "gemm", "gemm_mfma", "attention_plain", "attention_mfma", "sampling", "peaks")

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelLibraryError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[agave_amd] {msg}", file=sys.stderr, flush=True)


def available() -> List[str]:
    return [n for n in LIBRARIES if os.path.isfile(os.path.join(CSRC, n + ".hip"))]


def _build_dir() -> str:
    """In-tree ``agave_amd/_build`` when writable, else a per-user folder under the
    system's temporary directory."""
    env = os.environ.get("AGAVE_AMD_BUILD_DIR")
    cands = [env] if env else []
    cands.append(os.path.join(os.path.dirname(CSRC), "_build"))
    cands.append(os.path.join(tempfile.gettempdir(), f"agave_amd_build_{os.getuid()}"))
    for d in cands:
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".w{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelLibraryError("no writable folder for the compiled kernel libraries; set AGAVE_AMD_BUILD_DIR")


def _find_built(name: str, digest: str) -> Optional[str]:
    """A current object in any of the known build folders (a read-only in-tree one counts)."""
    for d in (os.environ.get("AGAVE_AMD_BUILD_DIR"), os.path.join(os.path.dirname(CSRC), "_build"),
              os.path.join(tempfile.gettempdir(), f"agave_amd_build_{os.getuid()}")):
        if not d:
            continue
        so, stamp = os.path.join(d, name + ".so"), os.path.join(d, name + ".stamp")
        try:
            if os.path.isfile(so) and open(stamp).read().strip() == digest:
                return so
        except OSError:
            continue
    return None


def _digest(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for f in (name + ".hip",) + HEADERS:
        p = os.path.join(CSRC, f)
        if os.path.isfile(p):
            with open(p, "rb") as fh:
                h.update(f.encode() + b"\0" + fh.read())
    return h.hexdigest()


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.isfile(c):
            return c
    raise KernelLibraryError("hipcc not found: the HIP kernels cannot be built (no fallback exists)")


def _compile_many(names: Iterable[str]) -> None:
    """Compile the given libraries side by side, printing a line now and then."""
    names = list(names)
    if not names:
        return
    out_dir = _build_dir()
    hipcc = _hipcc()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)              # hipcc wants a HOME for its temporary files
    procs = []
    for n in names:
        src = os.path.join(CSRC, n + ".hip")
        if not os.path.isfile(src):
            raise KernelLibraryError(f"kernel source {src} not found")
        tmp = os.path.join(out_dir, f"{n}.{os.getpid()}.tmp.so")
        log = open(os.path.join(out_dir, f"{n}.{os.getpid()}.log"), "w+")
        cmd = [hipcc] + FLAGS + ["-I", CSRC, "-o", tmp, src]
        procs.append((n, tmp, log, subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT, env=env, cwd=out_dir)))
    _log(f"compiling {', '.join(names)} for {ARCH} into {out_dir}")
    start = last = time.time()
    pending = list(procs)
    while pending:
        pending = [p for p in pending if p[3].poll() is None]
        if pending:
            time.sleep(0.2)
            if time.time() - last > 10:
                last = time.time()
                _log(f"still compiling {', '.join(p[0] for p in pending)} ({int(last - start)} s)")
    failed = []
    for n, tmp, log, proc in procs:
        log.seek(0)
        text = log.read()
        log.close()
        try:
            os.remove(log.name)
        except OSError:
            pass
        if proc.returncode != 0 or not os.path.isfile(tmp):
            failed.append((n, text))
            continue
        os.replace(tmp, os.path.join(out_dir, n + ".so"))
        with open(os.path.join(out_dir, n + ".stamp"), "w") as f:
            f.write(_digest(n))
    _log(f"compiled in {time.time() - start:.1f} s")
    if failed:
        raise KernelLibraryError("hipcc failed for " + ", ".join(n for n, _ in failed) + ":\n" +
                                 "\n".join(t[-4000:] for _, t in failed))


def build_all(force: bool = True) -> None:
    """Compile every kernel library (always, when ``force``)."""
    names = available()
    todo = names if force else [n for n in names if _find_built(n, _digest(n)) is None]
    _compile_many(todo)


def ensure_built(names: Iterable[str]) -> None:
    """Compile those of ``names`` that have no current object, side by side."""
    _compile_many([n for n in names if n not in _loaded and _find_built(n, _digest(n)) is None])


def load(name: str) -> ctypes.CDLL:
    """The loaded library ``name``; compiled first if no current object exists."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        digest = _digest(name)
        path = _find_built(name, digest)
        if path is None:
            _compile_many([name])
            path = _find_built(name, digest)
            if path is None:
                raise KernelLibraryError(f"kernel library {name} was built but cannot be found")
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load kernel library {path}: {e}") from None
        lib.agave_last_error.restype = ctypes.c_char_p
        _loaded[name] = lib
        return lib


def loaded_paths() -> List[str]:
    return [lib._name for lib in _loaded.values()]


class OpProfile:
    """Wall time per class of op, from a pair of HIP events around every call
    (the reference's ``--profile``: ``src/perf.zig:28-131``).  Steps must run
    eagerly while it is on: events are not recorded into graphs."""

    def __init__(self):
        self.enabled = False
        self.label: Optional[str] = None       # set by a part for its next calls (a product's role)
        self._records: List[tuple] = []

    def reset(self) -> None:
        self._records = []

    def table(self) -> List[tuple]:
        """(op, calls, total ms) by falling total; waits for the device."""
        import torch
        torch.cuda.synchronize()
        total: Dict[str, List[float]] = {}
        for name, e0, e1 in self._records:
            t = total.setdefault(name, [0, 0.0])
            t[0] += 1
            t[1] += e0.elapsed_time(e1)
        return sorted(((k, int(v[0]), v[1]) for k, v in total.items()), key=lambda r: -r[2])


profile = OpProfile()


def call(lib: ctypes.CDLL, fn: str, *args) -> None:
    """Call an entry point; a non-zero return raises with the library's message."""
    if profile.enabled:
        import torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc = getattr(lib, fn)(*args)
        e1.record()
        name = fn[6:] if fn.startswith("agave_") else fn
        profile._records.append((f"{name}:{profile.label}" if profile.label else name, e0, e1))
    else:
        rc = getattr(lib, fn)(*args)
    if rc != 0:
        raise KernelLibraryError(f"{fn}: {lib.agave_last_error().decode(errors='replace')}")
