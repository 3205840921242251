"""Build ``libnpamd.so`` (HIP kernels + C ABI) for gfx950 with hipcc.

    python -m neuropress_amd.build [--force]

Each ``csrc/*.hip`` is compiled to an object file (in parallel) and the
objects are linked into ``neuropress_amd/lib/libnpamd.so``.  hipcc
cross-compiles, so no GPU is needed to build.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libnpamd.so"
OBJ_DIR = LIB_DIR / "obj"

ARCH = "gfx950"
# Packed-FP32 VALU ops are switched off for every device function.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers_mtime() -> float:
    hdrs = list(CSRC.glob("*.hpp")) + list((PKG_DIR.parent / "include").glob("*.h"))
    return max(h.stat().st_mtime for h in hdrs)


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    newest = max(src.stat().st_mtime, _headers_mtime())
    if not force and obj.exists() and obj.stat().st_mtime >= newest:
        return obj
    extra = os.environ.get("NPAMD_HIPCC_FLAGS", "").split()  # e.g. -DNPAMD_TILE2_ABLATIONS for a tuning build
    cmd = [_hipcc(), *CXXFLAGS, *DEVICE_FLAGS, *extra, "-c", os.fspath(src), "-o", os.fspath(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stderr}")
    noise = "is not a recognized feature for this target"
    warn = [ln for ln in res.stderr.splitlines() if ln.strip() and noise not in ln]
    if warn:
        sys.stderr.write("\n".join(warn) + "\n")
    return obj


def build(force: bool = False, jobs: int | None = None) -> Path:
    """Compile every kernel source and link the shared library; return its path."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), os.cpu_count() or 4, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), srcs))
    if force or not LIB_PATH.exists() or any(o.stat().st_mtime > LIB_PATH.stat().st_mtime for o in objs):
        cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", os.fspath(LIB_PATH)]
        cmd += [os.fspath(o) for o in objs]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv)
    print(path)
