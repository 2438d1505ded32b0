"""Compiles the HIP sources under ``ullm_amd/csrc`` for gfx950 and loads them with ctypes.

One shared library per kernel family (``<family>.hip`` -> ``lib/<family>.<hash>.so``), built with
plain ``hipcc`` on first use and whenever the source text changes (the hash covers the source, the
headers and the flags, so a stale library is never loaded).  Libraries are built in the tree so
that they travel with it; if the tree is read-only they go to a per-user temporary folder.
There is no fallback: a family that cannot be built or loaded raises ``KernelBuildError``.
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
from typing import Dict, List, Optional

CSRC_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    # hipcc -O3 may form packed 32-bit float ops from ordinary code; they are switched off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results stay in ordinary vector registers: accumulators that are also scaled by
    # vector instructions otherwise travel between the two register classes around every product
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
]
HEADERS = ["common.h"]
FAMILY_HEADERS = {"attention_mfma": ["no_alloc.h"]}     # headers only this family includes

_lock = threading.Lock()
_loaded: Dict[str, ctypes.CDLL] = {}


class KernelBuildError(RuntimeError):
    pass


def families() -> List[str]:
    return sorted(f[:-4] for f in os.listdir(CSRC_DIR) if f.endswith(".hip"))


def _find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc): "
                           "the HIP kernels cannot be built and there is no other code path")


def _source_hash(family: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for name in [family + ".hip"] + HEADERS + FAMILY_HEADERS.get(family, []):
        with open(os.path.join(CSRC_DIR, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    return h.hexdigest()[:16]


def _lib_dirs() -> List[str]:
    dirs = [os.path.join(CSRC_DIR, "lib")]
    dirs.append(os.path.join(tempfile.gettempdir(), f"ullm_amd_lib_{os.getuid()}"))
    return dirs


def lib_path(family: str, for_write: bool = False) -> str:
    name = f"{family}.{_source_hash(family)}.so"
    dirs = _lib_dirs()
    if not for_write:
        for d in dirs:
            p = os.path.join(d, name)
            if os.path.isfile(p):
                return p
    for d in dirs:
        try:
            os.makedirs(d, exist_ok=True)
            if os.access(d, os.W_OK):
                return os.path.join(d, name)
        except OSError:
            continue
    raise KernelBuildError(f"no writable folder for built kernels among {dirs}")


def compile_family(family: str, force: bool = False, verbose: bool = True) -> str:
    """Build one family if its library is missing (or ``force``); returns the library path."""
    src = os.path.join(CSRC_DIR, family + ".hip")
    if not os.path.isfile(src):
        raise KernelBuildError(f"no kernel source {src}")
    if not force:
        existing = lib_path(family)
        if os.path.isfile(existing):
            return existing
    out = lib_path(family, for_write=True)
    hipcc = _find_hipcc()
    tmp = f"{out}.{os.getpid()}.tmp"
    cmd = [hipcc] + HIPCC_FLAGS + ["-I", CSRC_DIR, src, "-o", tmp]
    if verbose:
        print(f"[ullm_amd] compiling {family}.hip for {ARCH} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    # keep the terminal alive while the compiler works
    output: List[str] = []
    reader = threading.Thread(target=lambda: output.append(proc.stdout.read()), daemon=True)
    reader.start()
    while True:
        try:
            proc.wait(timeout=20)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(f"[ullm_amd] ... still compiling {family}.hip ({time.time() - t0:.0f} s)",
                      file=sys.stderr, flush=True)
    reader.join()
    text = "".join(output)
    if proc.returncode != 0 or not os.path.isfile(tmp):
        if os.path.exists(tmp):
            os.unlink(tmp)
        raise KernelBuildError(f"hipcc failed for {family}.hip (exit {proc.returncode}):\n{text}")
    os.replace(tmp, out)
    # drop libraries of older source versions of this family
    d = os.path.dirname(out)
    for f in os.listdir(d):
        if f.startswith(family + ".") and f.endswith(".so") and os.path.join(d, f) != out:
            try:
                os.unlink(os.path.join(d, f))
            except OSError:
                pass
    if verbose:
        print(f"[ullm_amd] built {os.path.basename(out)} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def build_all(force: bool = True, verbose: bool = True, jobs: int = 4) -> Dict[str, str]:
    """Compile every family (in parallel processes of hipcc); returns {family: path}."""
    fams = families()
    results: Dict[str, str] = {}
    errors: List[str] = []

    def work(f):
        try:
            results[f] = compile_family(f, force=force, verbose=verbose)
        except KernelBuildError as e:  # collected and raised together below
            errors.append(str(e))

    pending = list(fams)
    while pending:
        batch, pending = pending[:jobs], pending[jobs:]
        threads = [threading.Thread(target=work, args=(f,)) for f in batch]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    if errors:
        raise KernelBuildError("\n\n".join(errors))
    return results


def load(family: str) -> ctypes.CDLL:
    """The loaded library of a family, building it first if need be."""
    lib = _loaded.get(family)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(family)
        if lib is None:
            path = compile_family(family, force=False)
            try:
                lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelBuildError(f"cannot load {path}: {e}") from None
            _loaded[family] = lib
    return lib


def loaded_libraries() -> Dict[str, str]:
    return {k: v._name for k, v in _loaded.items()}
