"""Compiles the HIP sources under ``velox_amd/csrc`` for gfx950 into shared libraries and finds them again.

Two kinds of library: ``core`` (everything whose sizes are run-time arguments) and ``attn_d<N>``
(the attention kernels for one head size, a compile-time constant).  A library's file name
carries a hash of the sources and flags it was built from, so a stale build is never loaded.
Libraries are built in-tree (``velox_amd/_build``) when that folder can be written, otherwise
under ``$VELOX_AMD_BUILD_DIR``, the user's cache folder or the temporary folder.  A build
prints a line every few seconds so that a caller waiting on it sees it is alive.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import Dict, List, Optional, Sequence

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE_DIR = os.path.join(PACKAGE_DIR, "csrc")
ARCH = "gfx950"
# hipcc -O3 must not form packed float32 operations from scalar code on this target
FLAGS = ["-O3", f"--offload-arch={ARCH}", "-shared", "-fPIC", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CORE_SOURCES = ["elementwise.hip", "gemm.hip", "skinny_gemm.hip", "sampling.hip", "probe.hip"]
ATTENTION_SOURCES = ["attention.hip"]
HEADERS = ["common.h", "no_alloc.h"]
# head sizes built ahead of time by build_all(); any other multiple of 16 up to 256 is built at first use
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 192, 256)


class BuildError(RuntimeError):
    pass


def find_hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise BuildError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH); the HIP kernels cannot be built")


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = tempfile.NamedTemporaryFile(dir=path, delete=True)
        probe.close()
        return True
    except OSError:
        return False


def build_dirs() -> List[str]:
    dirs = []
    if os.environ.get("VELOX_AMD_BUILD_DIR"):
        dirs.append(os.environ["VELOX_AMD_BUILD_DIR"])
    dirs.append(os.path.join(PACKAGE_DIR, "_build"))
    home = os.path.expanduser("~")
    if home and home != "~":
        dirs.append(os.path.join(home, ".cache", "velox_amd"))
    dirs.append(os.path.join(tempfile.gettempdir(), f"velox_amd_build_{os.getuid()}"))
    return dirs


def _digest(sources: Sequence[str], defines: Dict[str, object]) -> str:
    h = hashlib.sha1()
    for name in list(sources) + HEADERS:
        with open(os.path.join(SOURCE_DIR, name), "rb") as handle:
            h.update(name.encode())
            h.update(handle.read())
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(defines.items())).encode())
    return h.hexdigest()[:12]


def library_name(stem: str, sources: Sequence[str], defines: Dict[str, object]) -> str:
    return f"libvelox_{stem}_{_digest(sources, defines)}.so"


def find_library(stem: str, sources: Sequence[str], defines: Dict[str, object]) -> Optional[str]:
    name = library_name(stem, sources, defines)
    for directory in build_dirs():
        path = os.path.join(directory, name)
        if os.path.isfile(path):
            return path
    return None


def compile_library(stem: str, sources: Sequence[str], defines: Dict[str, object], quiet: bool = False) -> str:
    hipcc = find_hipcc()
    target_dir = next((d for d in build_dirs() if _writable(d)), None)
    if target_dir is None:
        raise BuildError(f"no writable folder to build into (tried {build_dirs()})")
    name = library_name(stem, sources, defines)
    final = os.path.join(target_dir, name)
    partial = os.path.join(target_dir, f".{name}.{os.getpid()}.tmp")
    command = [hipcc, *FLAGS, *[f"-D{k}={v}" for k, v in defines.items()], *[os.path.join(SOURCE_DIR, s) for s in sources], "-o", partial]
    started = time.time()
    if not quiet:
        print(f"[velox_amd] compiling {stem} kernels for {ARCH} ...", file=sys.stderr, flush=True)
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    with tempfile.TemporaryFile(mode="w+") as log:
        process = subprocess.Popen(command, stdout=log, stderr=subprocess.STDOUT, cwd=target_dir, env=env)
        last = started
        while True:
            try:
                process.wait(timeout=1.0)
                break
            except subprocess.TimeoutExpired:
                if not quiet and time.time() - last >= 5.0:
                    last = time.time()
                    print(f"[velox_amd]   still compiling {stem} ({int(last - started)} s)", file=sys.stderr, flush=True)
        log.seek(0)
        output = log.read()
    if process.returncode != 0 or not os.path.isfile(partial):
        if os.path.exists(partial):
            os.unlink(partial)
        raise BuildError(f"hipcc failed for {stem} (exit {process.returncode}):\n{' '.join(command)}\n{output}")
    os.replace(partial, final)
    # older builds of the same library are of no use any more
    for other in os.listdir(target_dir):
        if other.startswith(f"libvelox_{stem}_") and other.endswith(".so") and other != name:
            try:
                os.unlink(os.path.join(target_dir, other))
            except OSError:
                pass
    if not quiet:
        print(f"[velox_amd] built {name} in {time.time() - started:.1f} s", file=sys.stderr, flush=True)
    return final


def ensure_library(stem: str, sources: Sequence[str], defines: Dict[str, object], force: bool = False) -> str:
    if not force:
        found = find_library(stem, sources, defines)
        if found is not None:
            return found
    return compile_library(stem, sources, defines)


def ensure_core(force: bool = False) -> str:
    return ensure_library("core", CORE_SOURCES, {}, force)


def ensure_attention(head_dim: int, force: bool = False) -> str:
    if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
        raise BuildError(f"head_dim={head_dim}: the attention kernels take multiples of 16 from 16 to 256")
    return ensure_library(f"attn_d{head_dim}", ATTENTION_SOURCES, {"VELOX_HEAD_DIM": head_dim}, force)


def build_all(head_dims: Sequence[int] = DEFAULT_HEAD_DIMS, force: bool = True) -> List[str]:
    """Compiles every library (in parallel, one hipcc per library)."""
    from concurrent.futures import ThreadPoolExecutor

    jobs = [("core", CORE_SOURCES, {})] + [(f"attn_d{d}", ATTENTION_SOURCES, {"VELOX_HEAD_DIM": d}) for d in head_dims]
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        return list(pool.map(lambda job: ensure_library(job[0], job[1], job[2], force), jobs))
