"""Build recipe for the HIP library: hipcc cross-compiles every csrc/*.hip for gfx950
and links one shared object next to the sources (in-tree, so it travels with the
tree and is the file the loader opens)."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_PATH = CSRC / "libgptq4.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-parameter",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the gfx950 library cannot be built here")
    return exe


def _run(cmd, verbose):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, cmd)) + "\n" + out)
    if verbose and out.strip():
        print(out)


def build_library(verbose: bool = False, extra_flags=()) -> Path:
    """Compile csrc/*.hip -> csrc/libgptq4.so.  Always recompiles."""
    hipcc = _hipcc()
    sources = sorted(CSRC.glob("*.hip"))
    objdir = CSRC / "build"
    objdir.mkdir(exist_ok=True)
    objs = [objdir / (s.stem + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-c", str(src), "-o", str(obj)], verbose)

    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


PROBE_SRC = CSRC / "probe" / "floor_probe.hip"
PROBE_PATH = CSRC / "probe" / "floor_probe"


def build_probe(verbose: bool = False) -> Path:
    """Compile the stand-alone floor probe (launch floor, plain-read rate; `bench.py --floor-probe` runs it)."""
    _run([_hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          str(PROBE_SRC), "-o", str(PROBE_PATH)], verbose)
    return PROBE_PATH


if __name__ == "__main__":
    path = build_library(verbose=True, extra_flags=sys.argv[1:])
    print("built", path)
    print("built", build_probe(verbose=True))
