"""Build the gfx950 shared library ``libvllm_amd_qlinear.so`` in-tree with hipcc.

``python -m vllm_amd.build`` (or ``build_library()``) compiles every ``csrc/*.hip`` for gfx950 and links one
shared object next to this file.  There is no CMake step and no torch dependency in the native code: the library
exposes the plain C ABI declared in ``include/vllm_amd_qlinear.h``.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libvllm_amd_qlinear.so"
BENCH_PROBE_PATH = PKG_DIR / "libvaq_bench_probe.so"      # csrc/bench/*.hip: measurement kernels, loaded by bench.py only
OBJ_DIR = PKG_DIR / "build"

# -packed-fp32-ops is switched off on purpose: the packed fp32 VALU forms are not trusted on this fleet.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the gfx950 library cannot be built")
    return exe


def _compile_one(src: Path, obj: Path, verbose: bool) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if verbose and err:
        print(err, file=sys.stderr)


def _link(objs: list[Path], out: Path) -> None:
    tmp = out.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, out)


def build_library(verbose: bool = False, jobs: int | None = None, only: list[str] | None = None) -> Path:
    """Compile all sources (always; no staleness check) and link the shared library (and the benchmark's probe
    library beside it).  `only` = source stems to recompile, the other objects being reused as they are (development
    aid; the default compiles everything).  Returns the library's path."""
    OBJ_DIR.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    probes = sorted((CSRC / "bench").glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    objs = [OBJ_DIR / (s.stem + ".o") for s in sources]
    probe_objs = [OBJ_DIR / ("bench_" + s.stem + ".o") for s in probes]
    todo = [(s, o) for s, o in zip(sources + probes, objs + probe_objs) if only is None or s.stem in only or not o.exists()]
    jobs = jobs or min(8, max(1, len(todo)), os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _compile_one(so[0], so[1], verbose), todo))
    _link(objs, LIB_PATH)
    if probe_objs:
        _link(probe_objs, BENCH_PROBE_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True, only=sys.argv[1:] or None))
