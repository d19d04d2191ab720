"""Compiles the HIP sources of this folder for gfx950 and loads them through ctypes.

Each source file becomes one shared library with a C ABI.  A library is looked for
under `_build/` beside the sources (or, when that folder cannot be written, under the
temporary folder), under a name that carries a hash of the source text and of the
compiler flags, so a library built from other sources is never loaded.  What is
missing is compiled at its first use, with a line on stderr when it starts and every
few seconds while it runs; nothing is taken from a cache in the home folder.
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

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# -packed-fp32-ops off: hipcc otherwise forms packed float32 instructions by itself
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
SOURCES = ("elementwise", "rope_kv", "attn_rows", "attn_mfma", "gemm_tiled", "gemm_mfma", "skinny_gemm", "splitk_gemm", "sampling")
HEADERS = ("common.h", "attn_mfma.h")

_libs = {}
_lock = threading.Lock()


def header_constant(name: str, header: str = "common.h") -> int:
    """The integer that `#define name value` of a header gives: sizes that the kernels and the host code
    share (the cache's page length) are written down once, in the header."""
    import re
    with open(os.path.join(HERE, header)) as f:
        m = re.search(rf"^#define\s+{re.escape(name)}\s+\(?(-?\d+)u?\)?\s*(?://.*)?$", f.read(), re.M)
    if m is None:
        raise BuildError(f"{header} does not define {name} as an integer")
    return int(m.group(1))


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[bitnet.c_amd] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels "
                     "cannot be compiled and there is no other implementation to fall back to")


def _digest(name: str) -> str:
    h = hashlib.sha256()
    for fn in (name + ".hip",) + HEADERS:
        with open(os.path.join(HERE, fn), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def _build_dirs():
    yield os.path.join(HERE, "_build")
    yield os.path.join(tempfile.gettempdir(), f"bitnet_c_amd-build-{os.getuid()}")


def _writable_build_dir() -> str:
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}-{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.unlink(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the compiled kernels")


def find_built(name: str):
    fn = f"lib{name}.{_digest(name)}.so"
    for d in _build_dirs():
        p = os.path.join(d, fn)
        if os.path.isfile(p):
            return p
    return None


def compile_source(name: str, *, quiet: bool = False) -> str:
    """Compile one source now, whatever is there already; returns the library's path."""
    if name not in SOURCES:
        raise BuildError(f"unknown kernel source {name!r}")
    out_dir = _writable_build_dir()
    final = os.path.join(out_dir, f"lib{name}.{_digest(name)}.so")
    tmp = f"{final}.{os.getpid()}.{threading.get_ident()}.tmp"
    cmd = [_hipcc()] + FLAGS + [os.path.join(HERE, name + ".hip"), "-o", tmp]
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME"):                    # hipcc wants some HOME; any folder does
        env["HOME"] = tempfile.gettempdir()
    if not quiet:
        _say(f"compiling {name}.hip for {ARCH} ...")
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=out_dir)
    beat = t0
    while True:
        try:
            out, _ = proc.communicate(timeout=5)
            break
        except subprocess.TimeoutExpired:
            if not quiet and time.time() - beat >= 10:
                beat = time.time()
                _say(f"... still compiling {name}.hip ({beat - t0:.0f} s)")
    text = "\n".join(l for l in out.decode(errors="replace").splitlines()
                     if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise BuildError(f"hipcc failed on {name}.hip (exit {proc.returncode}):\n{text}")
    os.replace(tmp, final)
    for fn in os.listdir(out_dir):             # older builds of the same source
        if fn.startswith(f"lib{name}.") and fn.endswith(".so") and os.path.join(out_dir, fn) != final:
            try:
                os.unlink(os.path.join(out_dir, fn))
            except OSError:
                pass
    if not quiet:
        _say(f"built {name} in {time.time() - t0:.1f} s")
    return final


def build_all(*, force: bool = True, jobs: int = 8) -> dict:
    """Compile every source (all of them when `force`, else the missing ones)."""
    from concurrent.futures import ThreadPoolExecutor
    todo = [n for n in SOURCES if force or find_built(n) is None]
    paths = {n: find_built(n) for n in SOURCES if n not in todo}
    if todo:
        with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as ex:
            for n, p in zip(todo, ex.map(compile_source, todo)):
                paths[n] = p
    return paths


def load(name: str) -> ctypes.CDLL:
    """The loaded library of one source; compiled first when it is not there."""
    with _lock:
        lib = _libs.get(name)
        if lib is None:
            path = find_built(name) or compile_source(name)
            lib = ctypes.CDLL(path)
            _libs[name] = lib
        return lib


def loaded_libraries() -> dict:
    return {n: l._name for n, l in _libs.items()}
