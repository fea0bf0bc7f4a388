"""Compiling the HIP sources for gfx950 and loading the result.

Libraries are built with ``hipcc`` into ``csrc/_build`` inside the package (or, when that is not
writable, into a per-user folder under the temporary directory) and loaded with ``ctypes``.  A
library is rebuilt when its sources or flags change.  The core library holds every kernel whose
sizes are run-time arguments; the matrix-core attention kernels keep their accumulators in
registers and address pages with constant arithmetic; they are therefore compiled once per (head size,
page size), on first use of that pair.

There is no fallback: if ``hipcc`` is missing or a source does not compile, loading raises.
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
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

CORE_SOURCES = ["elementwise.hip", "gemm_generic.hip", "attn_generic.hip", "sampling.hip", "gemm_bf16.hip", "gemm_wide.hip", "graph.hip"]
ATTN_SOURCES = ["attn_mfma.hip"]

_loaded: dict[str, ctypes.CDLL] = {}


_build_dir_found: Path | None = None
_build_dir_lock = threading.Lock()


def _build_dir() -> Path:
    """Where libraries are built: beside the sources, or a per-user temporary folder if that cannot be written.  Found
    once per process (several compilers run at a time, and all of them must land in the same place)."""
    global _build_dir_found
    with _build_dir_lock:
        if _build_dir_found is None:
            d = CSRC / "_build"
            try:
                d.mkdir(exist_ok=True)
                probe = d / f".w{os.getpid()}"
                probe.write_text("")
                probe.unlink()
            except OSError:
                d = Path(tempfile.gettempdir()) / f"nanospec_amd_build_{os.getuid()}"
                d.mkdir(parents=True, exist_ok=True)
            _build_dir_found = d
        return _build_dir_found


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("nanospec_amd needs hipcc (ROCm) to build its kernels; none was found")


def _digest(sources: list[str], defines: list[str]) -> str:
    h = hashlib.sha256()
    for name in sorted(set(sources) | {h.name for h in CSRC.glob("*.h")}):
        h.update(name.encode())
        h.update((CSRC / name).read_bytes())
    h.update(" ".join(FLAGS + defines).encode())
    return h.hexdigest()


def _say(msg: str) -> None:
    print(f"[nanospec_amd] {msg}", file=sys.stderr, flush=True)


def compile_library(name: str, sources: list[str], defines: list[str] = (), force: bool = False) -> Path:
    """Build ``lib<name>.so`` if it is missing or stale (or ``force``); return its path."""
    defines = list(defines)
    out_dir = _build_dir()
    lib = out_dir / f"lib{name}.so"
    stamp = out_dir / f"lib{name}.sha256"
    digest = _digest(sources, defines)
    if not force and lib.exists() and stamp.exists() and stamp.read_text().strip() == digest:
        return lib
    tmp = out_dir / f"lib{name}.{os.getpid()}.tmp.so"
    cmd = [_hipcc(), *FLAGS, *defines, *[str(CSRC / s) for s in sources], "-o", str(tmp)]
    _say(f"compiling lib{name}.so for {ARCH} ({', '.join(sources)}) ...")
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    while True:
        try:
            log, _ = proc.communicate(timeout=15)
            break
        except subprocess.TimeoutExpired:
            _say(f"  still compiling lib{name}.so, {time.time() - t0:.0f} s")
    log = "\n".join(l for l in log.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise RuntimeError(f"hipcc failed for lib{name}.so:\n{log}")
    os.replace(tmp, lib)
    stamp.write_text(digest)
    _say(f"built lib{name}.so in {time.time() - t0:.0f} s")
    return lib


def load_library(name: str, sources: list[str], defines: list[str] = ()) -> ctypes.CDLL:
    if name not in _loaded:
        path = compile_library(name, sources, defines)
        try:
            _loaded[name] = ctypes.CDLL(str(path))
        except OSError as e:
            raise RuntimeError(f"nanospec_amd could not load its kernel library {path}: {e}") from e
    return _loaded[name]


def core() -> ctypes.CDLL:
    return load_library("ns_core", CORE_SOURCES)


def attn_name(head_dim: int, page_size: int) -> str:
    return f"ns_attn_hd{head_dim}_p{page_size}"


def _attn_defines(head_dim: int, page_size: int) -> list[str]:
    return [f"-DNS_HEAD_DIM={head_dim}", f"-DNS_PAGE_SIZE={page_size}"]


def attn(head_dim: int, page_size: int) -> ctypes.CDLL:
    """The matrix-core attention kernels for one head size and one page size."""
    return load_library(attn_name(head_dim, page_size), ATTN_SOURCES, _attn_defines(head_dim, page_size))


def build_all(attn_variants=((16, 4), (32, 8), (64, 16), (128, 16)), force: bool = True, jobs: int | None = None) -> None:
    """Compile the core library and the attention library of each given (head size, page size), ``jobs`` compilers at a
    time (by default one per processor, at most eight)."""
    from concurrent.futures import ThreadPoolExecutor

    work = [("ns_core", CORE_SOURCES, [])] + [(attn_name(hd, page), ATTN_SOURCES, _attn_defines(hd, page)) for hd, page in attn_variants]
    jobs = jobs or max(1, min(8, os.cpu_count() or 1))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for done in [pool.submit(compile_library, name, sources, defines, force) for name, sources, defines in work]:
            done.result()
