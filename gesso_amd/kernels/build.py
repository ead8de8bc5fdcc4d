"""Compiling and loading the HIP extension.

The kernels under ``gesso_amd/csrc`` are compiled with ``hipcc`` for gfx950 into one shared
library with a C interface and loaded through ``ctypes``.  The library lies in the tree
(``gesso_amd/_lib``) when that folder can be written, else in a per-user temporary folder.
A digest of the sources and flags lies beside it; a library whose digest differs is built
again.  Nothing here falls back to another implementation: if the library cannot be built
or loaded, :class:`~gesso_amd.errors.KernelError` says why.
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

from ..errors import KernelError

ARCH = "gfx950"
CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_NAME = "libgesso_hip.so"
# packed float32 instructions are switched off: some of their forms have given wrong results
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

# the vendor's matrix product library (products of many rows, library_gemm.hip)
LINK = ["-lhipblaslt"]

_lock = threading.Lock()
_lib = None


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _digest() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + LINK).encode())
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise KernelError("hipcc not found: the HIP extension cannot be built (set HIPCC or ROCM_PATH)")


def _lib_dirs():
    """Candidate folders for the library, the in-tree one first."""
    tree = os.path.join(os.path.dirname(CSRC), "_lib")
    user = os.path.join(tempfile.gettempdir(), f"gesso_amd_{os.getuid()}")
    return [tree, user]


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _say(msg: str) -> None:
    print(f"[gesso_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = True, verbose: bool = True) -> str:
    """Compile every kernel source for gfx950 and link the library; returns its path."""
    digest = _digest()
    out_dir = next((d for d in _lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise KernelError("no writable folder for the HIP extension", tried=_lib_dirs())
    lib = os.path.join(out_dir, LIB_NAME)
    stamp = lib + ".digest"
    if not force and os.path.exists(lib) and os.path.exists(stamp) and open(stamp).read().strip() == digest:
        return lib
    hipcc = _hipcc()
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)   # hipcc's helpers want some HOME
    t0 = time.time()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(name):
        obj = os.path.join(obj_dir, name[:-4] + ".o")
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(CSRC, name), "-o", obj]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
        if p.returncode != 0:
            raise KernelError(f"hipcc failed on {name}:\n{p.stdout[-4000:]}")
        if verbose:
            _say(f"  {name} done ({time.time() - t0:.0f} s)")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = lib + f".tmp{os.getpid()}"
    p = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs + LINK,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if p.returncode != 0:
        raise KernelError(f"linking the HIP extension failed:\n{p.stdout[-4000:]}")
    os.replace(tmp, lib)
    with open(stamp, "w") as f:
        f.write(digest)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def find_built():
    """Path of a library whose digest matches the sources, or None."""
    digest = _digest()
    for d in _lib_dirs():
        lib = os.path.join(d, LIB_NAME)
        stamp = lib + ".digest"
        try:
            if os.path.exists(lib) and open(stamp).read().strip() == digest:
                return lib
        except OSError:
            continue
    return None


_C_TYPES = {"int": ctypes.c_int, "long": ctypes.c_long, "float": ctypes.c_float, "double": ctypes.c_double,
            "unsigned": ctypes.c_uint}


def entry_points():
    """``name -> (result type, argument types)`` of every ``extern "C"`` entry point, read from the sources' own
    declarations: with these set, a call passes plain Python numbers and addresses and ctypes converts them by table
    instead of guessing per argument (a third of a call's cost on the host)."""
    import re
    out = {}
    pattern = re.compile(r'extern\s+"C"\s+(const char\*|int|long)\s+(gs_\w+)\s*\(([^)]*)\)\s*\{')
    for name in sorted(os.listdir(CSRC)):
        if not name.endswith((".hip", ".h")):
            continue
        with open(os.path.join(CSRC, name), encoding="utf-8") as f:
            text = f.read()
        for res, fn, args in pattern.findall(text):
            types = []
            for a in (a.strip() for a in args.split(",") if a.strip()):
                if "*" in a or a.startswith("hipStream_t"):
                    types.append(ctypes.c_void_p)
                else:
                    words = a.replace("const ", "").split()
                    if words[0] not in _C_TYPES:
                        raise KernelError(f"{name}: {fn} takes {a!r}, which the loader has no ctypes type for")
                    types.append(_C_TYPES[words[0]])
            out[fn] = (ctypes.c_char_p if "char" in res else (ctypes.c_long if res == "long" else ctypes.c_int), types)
    return out


def load() -> ctypes.CDLL:
    """The loaded library; built first if no current build is found."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = find_built()
        if path is None:
            path = build(force=False)
        try:
            _lib = ctypes.CDLL(path)
        except OSError as err:
            raise KernelError(f"cannot load the HIP extension {path}: {err}") from err
        for fn, (res, args) in entry_points().items():
            try:
                f = getattr(_lib, fn)
            except AttributeError:
                continue
            f.restype, f.argtypes = res, args
        _lib.gs_last_error.restype = ctypes.c_char_p
        if _lib.gs_abi_version() != 9:
            raise KernelError("the HIP extension has another interface version; build it again")
        return _lib
