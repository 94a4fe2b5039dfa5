"""Compiles the HIP sources under `atomserve_amd/csrc` for gfx950 and finds the results.

Each `<name>.hip` becomes one shared library `lib_<name>.so` beside its source (or,
if that folder cannot be written, under a per-user temporary folder).  A library is
rebuilt when the hash of its sources and flags differs from the one recorded next
to it, so an edited source is never run stale and an unchanged one is never rebuilt.
Libraries are compiled one at a time, at the first use of one of their kernels.
"""

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
# Packed fp32 instructions are switched off for every kernel of this package.
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]  # fmt: skip
HEADERS = ["common.h", "no_alloc.h"]
LIBRARIES = ("elementwise", "attention", "gemm", "sampling", "blas")
LINK = {"blas": ["-lhipblaslt"]}  # what a library links beside the HIP runtime


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    found = shutil.which("hipcc")
    for candidate in (found, "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise BuildError("hipcc not found: the HIP kernels of atomserve_amd cannot be compiled")


def _source_hash(name: str) -> str:
    h = hashlib.sha256(" ".join([*FLAGS, *LINK.get(name, [])]).encode())
    for rel in [f"{name}.hip", *HEADERS]:
        with open(os.path.join(CSRC, rel), "rb") as f:
            h.update(rel.encode())
            h.update(f.read())
    return h.hexdigest()


def _candidate_dirs() -> list:
    dirs = []
    if os.environ.get("ATOMSERVE_AMD_BUILD_DIR"):
        dirs.append(os.environ["ATOMSERVE_AMD_BUILD_DIR"])
    dirs.append(CSRC)
    dirs.append(os.path.join(tempfile.gettempdir(), f"atomserve_amd_build_{os.getuid()}"))
    return dirs


def _is_current(path: str, digest: str) -> bool:
    try:
        with open(path + ".sha") as f:
            return os.path.isfile(path) and f.read().strip() == digest
    except OSError:
        return False


def _writable(directory: str) -> bool:
    try:
        os.makedirs(directory, exist_ok=True)
        probe = os.path.join(directory, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def compile_library(name: str, out_dir: str, quiet: bool = False) -> str:
    """Run hipcc for one library; returns the path of the .so."""
    digest = _source_hash(name)
    target = os.path.join(out_dir, f"lib_{name}.so")
    tmp = f"{target}.{os.getpid()}.tmp"
    cmd = [_hipcc(), *FLAGS, os.path.join(CSRC, f"{name}.hip"), "-o", tmp, *LINK.get(name, [])]
    if not quiet:
        print(f"atomserve_amd: compiling {name}.hip for {ARCH} ...", file=sys.stderr, flush=True)
    start = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.run(cmd, capture_output=True, text=True, env=env)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"hipcc failed for {name}.hip:\n{proc.stderr[-4000:]}")
    os.replace(tmp, target)
    with open(target + ".sha", "w") as f:
        f.write(digest)
    if not quiet:
        print(f"atomserve_amd: built lib_{name}.so in {time.time() - start:.1f}s", file=sys.stderr, flush=True)
    return target


def library_path(name: str, force: bool = False) -> str:
    """Path of an up-to-date lib_<name>.so, compiling it if there is none."""
    if name not in LIBRARIES:
        raise BuildError(f"unknown kernel library {name!r}")
    digest = _source_hash(name)
    if not force:
        for d in _candidate_dirs():
            path = os.path.join(d, f"lib_{name}.so")
            if _is_current(path, digest):
                return path
    for d in _candidate_dirs():
        if _writable(d):
            return compile_library(name, d)
    raise BuildError("no writable folder for the compiled kernels")


def build_all(force: bool = True) -> list:
    """Compile every library (always, when `force`); returns their paths."""
    return [library_path(name, force=force) for name in LIBRARIES]
