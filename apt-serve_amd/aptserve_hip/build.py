"""Build libaptserve_hip.so from csrc/*.hip, and the benchmark's measurement kernels
(csrc/probes/*.hip) into libaptserve_probes.so, with hipcc for gfx950.

Run ``python apt-serve_amd/aptserve_hip/build.py`` (add ``--force`` to
recompile objects that look up to date).  The library is written next to this
file so that it travels with the source tree; nothing is installed.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR.parent / "csrc"
INCLUDE = PKG_DIR.parent.parent / "include"
BUILD_DIR = PKG_DIR.parent / "build"
LIB_PATH = PKG_DIR / "libaptserve_hip.so"
PROBES_LIB_PATH = PKG_DIR / "libaptserve_probes.so"

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# packed-fp32 VALU forms are switched off for every device compile
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def _stale(obj: Path, src: Path) -> bool:
    if not obj.exists():
        return True
    deps = [src, *CSRC.glob("*.h"), *INCLUDE.glob("*.h"), Path(__file__)]
    return any(d.stat().st_mtime > obj.stat().st_mtime for d in deps)


def _compile(src: Path, obj: Path) -> None:
    # APS_EXTRA_FLAGS: additional -D switches for a one-off build (the kernels' tuning macros)
    cmd = [HIPCC, *FLAGS, *os.environ.get("APS_EXTRA_FLAGS", "").split(), "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the device-only target feature and says so
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{' '.join(cmd)}\n{r.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def _build_lib(sources, lib_path: Path, force: bool, verbose: bool) -> Path:
    BUILD_DIR.mkdir(exist_ok=True)
    if not sources:
        raise RuntimeError(f"no HIP sources for {lib_path.name}")
    jobs = []
    objs = []
    for src in sources:
        obj = BUILD_DIR / (src.stem + ".o")
        objs.append(obj)
        if force or _stale(obj, src):
            jobs.append((src, obj))
    if verbose:
        print(f"[aptserve_hip.build] {lib_path.name}: compiling {len(jobs)}/{len(sources)} sources for gfx950",
              flush=True)
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(lambda j: _compile(*j), jobs))
    if jobs or not lib_path.exists():
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
               *map(str, objs), "-o", str(lib_path)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"[aptserve_hip.build] {lib_path}", flush=True)
    return lib_path


def build(force: bool = False, verbose: bool = True) -> Path:
    """Compile both libraries; returns the path of the product library."""
    lib = _build_lib(sorted(CSRC.glob("*.hip")), LIB_PATH, force, verbose)
    _build_lib(sorted((CSRC / "probes").glob("*.hip")), PROBES_LIB_PATH, force, verbose)
    return lib


if __name__ == "__main__":
    build(force="--force" in sys.argv)
