"""Builds libpdw.so (the C-ABI HIP library) in-tree with hipcc for gfx950.

    python -m pyramidconvblock_amd.build [--force]

Every csrc/*.hip file is compiled to an object (in parallel) and linked into
pyramidconvblock_amd/libpdw.so.  hipcc cross-compiles, so no GPU is needed.
With PDW_TUNE_BUILD=1 in the environment of the build the library is compiled with -DPDW_TUNE, which makes
its planners honour the PDW_* override variables (for experiments; the product build reads no environment).
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libpdw.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = (["-DPDW_TUNE"] if os.environ.get("PDW_TUNE_BUILD") else []) + [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-ffp-contract=fast",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def _stale(out, deps):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, headers, force):
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
    if force or _stale(obj, [src] + headers):
        cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{err}")
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int | None = None) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    headers = sorted(glob.glob(os.path.join(CSRC, "*.h"))) + [os.path.join(HERE, "..", "include", "pdw.h")]
    jobs = jobs or min(len(srcs), os.cpu_count() or 4, 16)
    with ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, headers, force), srcs))
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
