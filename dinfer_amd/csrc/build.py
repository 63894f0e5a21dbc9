"""Compiles the sources of this folder, one shared library per entry of SOURCES,
into ``dinfer_amd/_lib/`` (or a per-user temporary folder when the package folder
is read-only): the HIP kernels for gfx950 with hipcc, the host core (page pools,
cache manager, scheduler, batch fill; plain C++) with the host compiler.

A library is built on first use and reused afterwards; ``build_all(force=True)``
recompiles everything. Only what a caller asks for is compiled, so a program
that never samples never builds the sampling library.
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
from pathlib import Path

CSRC = Path(__file__).resolve().parent
PACKAGE = CSRC.parent

# library name -> source file. Headers that all of them include are hashed too.
SOURCES = {
    "elementwise": "elementwise.hip",
    "norm": "norm.hip",
    "rope": "rope.hip",
    "attention_ref": "attention_ref.hip",
    "attention": "attention.hip",
    "gemm_ref": "gemm_ref.hip",
    "gemm": "gemm.hip",
    "gemm_mid": "gemm_mid.hip",
    "gemm_wide": "gemm_wide.hip",
    "sampling": "sampling.hip",
    "ceilings": "ceilings.hip",
    "host": "host/api.cpp",
}
HEADERS = ["common.cuh"]
# headers of single libraries (their C interface), hashed with them
OWN_HEADERS = {"gemm_mid": ["gemm_mid.h"]}
# libraries without device code, and the headers each is made of
HOST_ONLY = {"host": ["host/dinfer_host.h", "host/errors.hpp", "host/block_pool.hpp", "host/cache_manager.hpp",
                      "host/step_batch.hpp", "host/scheduler.hpp"]}
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC", "-Wall"]

ARCH = "gfx950"
# -packed-fp32-ops is switched off for device code: hipcc -O3 otherwise forms packed
# float instructions from ordinary float code. The host pass does not know the
# feature and says so on stderr; that is harmless and filtered out below.
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first kernel arguments arrive in scalar registers with the wave instead of by a load that every kernel's
    # first addresses would wait for (a decode step is a chain of some 200 short kernels)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wno-unused-result",
]


def _host_cxx() -> str:
    for cand in (os.environ.get("CXX"), "g++", "c++", "clang++"):
        path = shutil.which(cand) if cand else None
        if path:
            return path
    return _hipcc()  # hipcc compiles plain C++ too


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the HIP kernels cannot be built (looked in $HIPCC, PATH, /opt/rocm/bin)")


_lib_dir: Path | None = None
_lib_dir_lock = threading.Lock()


def lib_dir() -> Path:
    """Folder for built libraries: in the package if writable, else per-user temporary.
    Decided once per process (parallel builds must all land in the same folder)."""
    global _lib_dir
    with _lib_dir_lock:
        if _lib_dir is None:
            d = PACKAGE / "_lib"
            try:
                d.mkdir(exist_ok=True)
                probe = d / f".w{os.getpid()}.{threading.get_ident()}"
                probe.write_text("")
                probe.unlink()
                _lib_dir = d
            except OSError:
                alt = Path(tempfile.gettempdir()) / f"dinfer_amd_lib_{os.getuid()}"
                alt.mkdir(parents=True, exist_ok=True)
                _lib_dir = alt
        return _lib_dir


def source_hash(name: str) -> str:
    h = hashlib.sha256()
    for f in HOST_ONLY.get(name, HEADERS) + OWN_HEADERS.get(name, []) + [SOURCES[name]]:
        h.update((CSRC / f).read_bytes())
    h.update(" ".join(HOST_FLAGS if name in HOST_ONLY else FLAGS).encode())
    return h.hexdigest()[:16]


def lib_path(name: str) -> Path:
    return lib_dir() / f"libdinfer_{name}.so"


def find_built(name: str, fresh_only: bool = True) -> Path | None:
    """A library built earlier from today's sources, in the package or in the per-user folder; None if there
    is none (fresh_only False: also one built from other sources)."""
    for d in (PACKAGE / "_lib", Path(tempfile.gettempdir()) / f"dinfer_amd_lib_{os.getuid()}"):
        p = d / f"libdinfer_{name}.so"
        if p.exists() and not (fresh_only and is_stale(name, p)):
            return p
    return None


def is_stale(name: str, path: Path) -> bool:
    tag = path.with_suffix(".hash")
    try:
        return tag.read_text().strip() != source_hash(name)
    except OSError:
        return True


def build(name: str, verbose: bool = True) -> Path:
    """Compiles one library and returns its path. Prints a line now and then while the compiler runs."""
    if name not in SOURCES:
        raise KeyError(f"unknown library {name!r}; known: {sorted(SOURCES)}")
    out = lib_path(name)
    tmp = out.with_name(f".{out.name}.{os.getpid()}.tmp")
    if name in HOST_ONLY:
        cmd = [_host_cxx(), *HOST_FLAGS, str(CSRC / SOURCES[name]), "-o", str(tmp)]
        what = "the host"
    else:
        cmd = [_hipcc(), *FLAGS, str(CSRC / SOURCES[name]), "-o", str(tmp)]
        what = ARCH
    t0 = time.time()
    if verbose:
        print(f"[dinfer_amd] compiling {SOURCES[name]} for {what} ...", file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=str(CSRC))
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            print(f"[dinfer_amd] still compiling {SOURCES[name]} ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)

    th = threading.Thread(target=ticker, daemon=True)
    if verbose:
        th.start()
    log, _ = proc.communicate()
    done.set()
    log = "\n".join(l for l in log.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise RuntimeError(f"{Path(cmd[0]).name} failed for {SOURCES[name]}:\n{log}")
    os.replace(tmp, out)
    out.with_suffix(".hash").write_text(source_hash(name))
    if verbose:
        print(f"[dinfer_amd] built {out.name} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def build_all(force: bool = True, jobs: int = 4, verbose: bool = True) -> dict[str, Path]:
    """Compiles every library (in parallel processes of hipcc)."""
    from concurrent.futures import ThreadPoolExecutor

    names = [n for n in SOURCES if (CSRC / SOURCES[n]).exists()]

    def one(n):
        p = find_built(n)
        if not force and p is not None:
            return n, p
        return n, build(n, verbose=verbose)

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        return dict(ex.map(one, names))


if __name__ == "__main__":
    build_all(force=True)
