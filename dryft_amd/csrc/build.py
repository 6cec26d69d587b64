"""Compiling the HIP sources for gfx950 and loading them through ctypes.

Each ``.hip`` file becomes one shared library under ``dryft_amd/csrc/lib/`` (or, when
the package folder cannot be written, under a per-user folder in the temporary
directory). A library is compiled when it is first needed and missing or older than
its sources, so a program compiles what its model uses and nothing else; while a
compilation runs a line is printed every few seconds. There is no fallback: without
a library and without ``hipcc`` the call fails.
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

_HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
HIPCC_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
MODULES = ("batch", "embed", "norm", "activation", "rope_kv", "attn_rows", "attn_mfma", "gemm", "sampling")
_HEADERS = ("common.h",)                       # every library includes these
_OWN_HEADERS = {"sampling": ("sampling.h",)}    # and some a header of their own

_loaded: dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class ExtensionError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[dryft_amd] {msg}", file=sys.stderr, flush=True)


def _source_digest(name: str) -> str:
    h = hashlib.sha256()
    for f in (name + ".hip",) + _HEADERS + _OWN_HEADERS.get(name, ()):
        with open(os.path.join(_HERE, f), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _lib_dirs() -> list[str]:
    dirs = [os.path.join(_HERE, "lib")]
    user = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"dryft_amd-{user}", "lib"))
    return dirs


def _writable_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise ExtensionError(f"no writable folder for compiled kernels among {_lib_dirs()}")


def _lib_name(name: str) -> str:
    return f"dryft_{name}.so"


def _find_current(name: str) -> str | None:
    """Path of a library that matches the present sources, if one exists."""
    digest = _source_digest(name)
    for d in _lib_dirs():
        so = os.path.join(d, _lib_name(name))
        tag = so + ".digest"
        if os.path.isfile(so) and os.path.isfile(tag):
            try:
                with open(tag) as f:
                    if f.read().strip() == digest:
                        return so
            except OSError:
                pass
    return None


def hipcc_path() -> str | None:
    return shutil.which("hipcc") or (os.path.exists("/opt/rocm/bin/hipcc") and "/opt/rocm/bin/hipcc") or None


def _compile(name: str, out_dir: str) -> str:
    hipcc = hipcc_path()
    if hipcc is None:
        raise ExtensionError(f"kernel library {name!r} is not built and hipcc was not found; build it where ROCm is "
                             f"installed with `python -m dryft_amd build` (hipcc {' '.join(HIPCC_FLAGS)} "
                             f"{name}.hip -o {_lib_name(name)})")
    so = os.path.join(out_dir, _lib_name(name))
    tmp = so + f".tmp{os.getpid()}"
    cmd = [hipcc] + HIPCC_FLAGS + [os.path.join(_HERE, name + ".hip"), "-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())          # hipcc wants somewhere to keep its caches
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, cwd=out_dir)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise ExtensionError(f"hipcc failed on {name}.hip:\n{proc.stdout}")
    os.replace(tmp, so)
    with open(so + ".digest", "w") as f:
        f.write(_source_digest(name))
    return so


def build(names=MODULES, force: bool = False, jobs: int = 8) -> dict[str, str]:
    """Compile the named libraries (all by default); returns their paths."""
    names = list(names)
    todo = [n for n in names if force or _find_current(n) is None]
    paths = {n: _find_current(n) for n in names if n not in todo}
    if todo:
        out_dir = _writable_dir()
        _say(f"compiling {len(todo)} kernel librar{'y' if len(todo) == 1 else 'ies'} for {ARCH}: {', '.join(todo)}")
        t0 = time.time()
        with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as pool:
            futures = {n: pool.submit(_compile, n, out_dir) for n in todo}
            pending = set(todo)
            while pending:
                time.sleep(0.2)
                for n in list(pending):
                    if futures[n].done():
                        pending.discard(n)
                        paths[n] = futures[n].result()
                        _say(f"  {n} done ({time.time() - t0:.0f}s)")
                if pending and int((time.time() - t0) * 5) % 25 == 0:
                    _say(f"  still compiling: {', '.join(sorted(pending))} ({time.time() - t0:.0f}s)")
    return paths


def load(name: str) -> ctypes.CDLL:
    """The named library, compiled first if it is missing or out of date."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(name)
        if lib is None:
            if name not in MODULES:
                raise ExtensionError(f"unknown kernel library {name!r}")
            path = _find_current(name) or build([name])[name]
            lib = ctypes.CDLL(path)
            _loaded[name] = lib
    return lib


def ensure(names) -> None:
    """Compile (in parallel) and load every named library."""
    build([n for n in names if n not in _loaded])
    for n in names:
        load(n)
