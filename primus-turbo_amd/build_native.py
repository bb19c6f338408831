"""Build libprimus_turbo_amd.so (the C-ABI library) with hipcc for gfx950.

Usage:  python primus-turbo_amd/build_native.py [--force] [-j N]

Every ``csrc/*.hip`` translation unit is compiled to an object file under
``primus-turbo_amd/build/`` and linked into ``primus-turbo_amd/lib/``. hipcc
cross-compiles for gfx950, so no GPU is needed to build.
"""

from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
BUILD = ROOT / "build"
LIBDIR = ROOT / "lib"
LIBNAME = "libprimus_turbo_amd.so"
HEADER = ROOT.parent / "include" / "primus_turbo_amd.h"

ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-fno-gpu-rdc",
    # hipcc -O3 may otherwise form packed-fp32 VALU ops from scalar float code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-result",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def lib_path() -> Path:
    return LIBDIR / LIBNAME


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _deps_mtime() -> float:
    deps = list(CSRC.glob("*.h")) + [HEADER]
    return max(p.stat().st_mtime for p in deps)


def _extra_flags(src: Path) -> list[str]:
    """Per-file compiler flags: a leading ``// hipcc-flags: ...`` comment line in the source."""
    with open(src) as f:
        first = f.readline()
    tag = "// hipcc-flags:"
    return first[len(tag):].split() if first.startswith(tag) else []


def _compile_one(hipcc: str, src: Path, force: bool, verbose: bool) -> Path:
    obj = BUILD / (src.stem + ".o")
    if not force and obj.exists():
        if obj.stat().st_mtime >= max(src.stat().st_mtime, _deps_mtime()):
            return obj
    cmd = [hipcc, *HIPCC_FLAGS, *_extra_flags(src), "-c", str(src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(
        l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()
    )
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err and verbose:
        print(err, file=sys.stderr)
    return obj


def build(force: bool = False, jobs: int | None = None, verbose: bool = False) -> Path:
    hipcc = hipcc_path()
    BUILD.mkdir(exist_ok=True)
    LIBDIR.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    jobs = jobs or min(8, len(srcs))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile_one(hipcc, s, force, verbose), srcs))
    out = lib_path()
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(out)] + [str(o) for o in objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return out


def ensure_built() -> Path:
    """Return the library path, building it only when no library exists yet."""
    out = lib_path()
    if not out.exists():
        build()
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("-q", "--quiet", action="store_true")
    a = ap.parse_args()
    p = build(force=a.force, jobs=a.j, verbose=not a.quiet)
    print(f"built {p}")
