"""Compiles the HIP kernels for gfx950 into ``libbc4g.so`` beside this file.

Objects go to ``_build/`` under this folder.  Sources are compiled in parallel
and a line is printed as each one finishes, so a first call that has to
compile shows that it is alive.  Where this folder cannot be written and holds
no library built from the sources beside it (a checkout that belongs to someone
else), library and objects go to a folder of the user's own under the system's
temporary folder instead.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import List

from ..errors import KernelError

HERE = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(HERE, "kernels")
BUILD_DIR = os.path.join(HERE, "_build")          # (both moved by _settle() below where HERE cannot be written)
LIB_PATH = os.path.join(HERE, "libbc4g.so")

ARCH = "gfx950"
# -packed-fp32-ops is switched off: the compiler must not form packed float32
# instructions from ordinary float code on this hardware.
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelError("hipcc not found: the kernel library cannot be compiled")


def sources() -> List[str]:
    return sorted(f for f in os.listdir(SRC_DIR) if f.endswith(".hip"))


def sources_digest() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(SRC_DIR)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(SRC_DIR, name), "rb") as fh:
                h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


_MARKER = b"bc4g-sources-digest:"


def built_digest(path: str = "") -> str:
    """The digest of the sources the library file was built from, read from the file itself (it
    carries it behind a marker), without loading it; empty if there is none."""
    import mmap
    try:
        with open(path or LIB_PATH, "rb") as fh, mmap.mmap(fh.fileno(), 0, access=mmap.ACCESS_READ) as mm:
            at = mm.find(_MARKER)
            if at < 0:
                return ""
            raw = mm[at + len(_MARKER):at + len(_MARKER) + 64]
            return raw.split(b"\0", 1)[0].decode("ascii", "replace")
    except (OSError, ValueError):
        return ""


def _settle() -> None:
    """Where the library lives: beside this file, if that folder can be written or already holds a library of
    these sources; else in a folder that belongs to this user alone (a library that someone else could have put
    there is not loaded)."""
    global BUILD_DIR, LIB_PATH
    if os.access(HERE, os.W_OK) or built_digest(LIB_PATH) == sources_digest():
        return
    home = os.path.join(tempfile.gettempdir(), f"bc4g-{os.getuid()}")
    os.makedirs(home, mode=0o700, exist_ok=True)
    st = os.stat(home)
    if st.st_uid != os.getuid() or st.st_mode & 0o022:
        raise KernelError(f"{HERE} cannot be written, and {home} is not this user's own folder: nowhere to build")
    BUILD_DIR, LIB_PATH = os.path.join(home, "_build"), os.path.join(home, "libbc4g.so")


_settle()


def is_stale() -> bool:
    """Whether the built library comes from other sources (or flags) than those beside it."""
    return built_digest() != sources_digest()


def can_build() -> bool:
    try:
        _hipcc()
        return True
    except KernelError:
        return False


def _compile_one(hipcc: str, name: str, digest: str) -> str:
    obj = os.path.join(BUILD_DIR, name[:-4] + ".o")
    cmd = [hipcc, *HIPCC_FLAGS, "-I", SRC_DIR, "-c", os.path.join(SRC_DIR, name), "-o", obj]
    if name == "common.hip":      # the library carries the digest of what it was built from
        cmd.insert(1, f'-DBC4G_SOURCES_DIGEST="{digest}"')
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise KernelError(f"hipcc failed on {name}:\n{proc.stderr[-4000:]}")
    return obj


TWIN_DIR = os.path.join(HERE, "twin")


def twins_path() -> str:
    """The program of the C++ twin tests, beside the library it is linked against."""
    return os.path.join(os.path.dirname(LIB_PATH), "bc4g_twins")


def build_twins(verbose: bool = True) -> str:
    """Compile twin/twins.cpp (every kernel family beside a plain C++ twin) against the built library; returns the
    program's path.  `bc4g_twins [name ...]` runs the tests named (all without names, --list names them) and
    returns non-zero if one fails; twin/CMakeLists.txt registers the same program with ctest, one test a family."""
    hipcc = _hipcc()
    if not is_built():
        raise KernelError(f"{LIB_PATH} is not built: the twin tests are linked against it")
    out = twins_path()
    t0 = time.time()
    cmd = [hipcc, "--offload-arch=" + ARCH, "-O2", "-std=c++17", "-Wno-unused-command-line-argument", "-I", SRC_DIR,
           os.path.join(TWIN_DIR, "twins.cpp"), "-o", out + f".tmp{os.getpid()}", "-L", os.path.dirname(LIB_PATH), "-lbc4g",
           "-Wl,-rpath,$ORIGIN"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise KernelError(f"hipcc failed on the twin tests:\n{proc.stderr[-4000:]}")
    os.replace(out + f".tmp{os.getpid()}", out)
    if verbose:
        print(f"[bc4g] built {out} in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
    return out


def build(verbose: bool = True, jobs: int = 0) -> str:
    """Compile every kernel source and link the library; returns its path."""
    hipcc = _hipcc()
    os.makedirs(BUILD_DIR, exist_ok=True)
    names = sources()
    digest = sources_digest()
    jobs = jobs or min(len(names), max(1, min(16, os.cpu_count() or 1)))
    t0 = time.time()
    out = sys.stderr
    if verbose:
        print(f"[bc4g] compiling {len(names)} kernel sources for {ARCH} with {jobs} jobs ...", file=out, flush=True)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futs = {pool.submit(_compile_one, hipcc, n, digest): n for n in names}
        for fut in concurrent.futures.as_completed(futs):
            objs.append(fut.result())
            if verbose:
                print(f"[bc4g]   {futs[fut]} done ({time.time() - t0:.0f} s)", file=out, flush=True)
    tmp = LIB_PATH + f".tmp{os.getpid()}"
    proc = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp, *sorted(objs)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise KernelError(f"linking libbc4g.so failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[bc4g] built {LIB_PATH} in {time.time() - t0:.0f} s", file=out, flush=True)
    return LIB_PATH
