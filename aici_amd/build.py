"""Builds libhipattn.so (the HIP kernels + C ABI) and libmembench.so (the benchmark's memory-system
yardsticks, csrc/bench/) for gfx950 with hipcc.

    python -m aici_amd.build [--force] [-j N]

Every source under csrc/ is compiled to an object in csrc/build/ (in parallel)
and linked into aici_amd/libhipattn.so.  hipcc cross-compiles, so this runs on
a machine without a GPU.  Objects are rebuilt when their source or any header
is newer, or always with --force.
"""
from __future__ import annotations

import argparse
import concurrent.futures
import os
import subprocess
import sys
import time
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = CSRC / "build"
LIB = PKG / "libhipattn.so"
BENCH_SRC = CSRC / "bench" / "membench.hip"
BENCH_LIB = PKG / "libmembench.so"

# -packed-fp32-ops: keep hipcc from forming packed FP32 instructions; the
# host pass does not know the feature and says so, which is harmless.
FLAGS = [
    "-c", "-fPIC", "-O3", "-std=c++17", "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers_mtime() -> float:
    hs = list(CSRC.glob("*.h")) + [PKG.parent / "include" / "hipattn.h"]
    return max(h.stat().st_mtime for h in hs)


def _compile(src: Path, force: bool, hdr_mtime: float) -> tuple[str, float, str]:
    obj = OBJ / (src.stem + ".o")
    if not force and obj.exists():
        if obj.stat().st_mtime >= max(src.stat().st_mtime, hdr_mtime):
            return src.name, 0.0, ""
    t0 = time.time()
    r = subprocess.run(["hipcc", *FLAGS, str(src), "-o", str(obj)], capture_output=True, text=True)
    msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{msgs}")
    return src.name, time.time() - t0, msgs


def build(force: bool = False, jobs: int | None = None, verbose: bool = True) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 4)
    hdr = _headers_mtime()
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for name, dt, msgs in ex.map(lambda s: _compile(s, force, hdr), srcs):
            if verbose and (dt > 0 or msgs):
                print(f"[build] {name}: {dt:.1f}s" + (f"\n{msgs}" if msgs.strip() else ""), flush=True)
    objs = [str(OBJ / (s.stem + ".o")) for s in srcs]
    newest = max(os.path.getmtime(o) for o in objs)
    if force or not LIB.exists() or LIB.stat().st_mtime < newest:
        r = subprocess.run(["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", str(LIB)],
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}{r.stderr}")
        if verbose:
            print(f"[build] linked {LIB}", flush=True)
    if force or not BENCH_LIB.exists() or BENCH_LIB.stat().st_mtime < BENCH_SRC.stat().st_mtime:
        r = subprocess.run(["hipcc", "-shared", "-fPIC", "-O3", "-std=c++17", "--offload-arch=gfx950", str(BENCH_SRC),
                            "-o", str(BENCH_LIB)], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {BENCH_SRC.name}:\n{r.stdout}{r.stderr}")
        if verbose:
            print(f"[build] linked {BENCH_LIB}", flush=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    a = ap.parse_args()
    try:
        build(force=a.force, jobs=a.j)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
