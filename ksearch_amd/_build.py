"""Builds libksearch_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

The library is built in-tree (ksearch_amd/lib/) so that it travels with the
source snapshot to the GPU machine; nothing is compiled at import time.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB_PATH = os.path.join(LIBDIR, "libksearch_hip.so")
# the timeline build: the same sources with -DKSH_STAMPS (phase timestamps inside the decode step's kernels); a
# measuring aid that bench.py --only timeline loads, never the library the tests or the other benchmarks use
STAMPS_LIB_PATH = os.path.join(LIBDIR, "libksearch_hip_stamps.so")

ARCH = "gfx950"
# packed FP32 instructions stay off for every device translation unit
BASE = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# sources whose arithmetic must round like the unfused CPU expressions
NO_CONTRACT = {"dequant.hip", "glue.hip", "ple_ops.hip", "quantize.hip", "sdpa_q40_lanes.hip"}


def sources() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _compile(src: str, stamps: bool = False) -> str:
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + (".stamps.o" if stamps else ".o"))
    cmd = ["hipcc", "-x", "hip", *BASE]
    if stamps:
        cmd.append("-DKSH_STAMPS")
    if src in NO_CONTRACT:
        cmd.append("-ffp-contract=off")
    cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only feature flag; that warning is noise
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err:
        sys.stderr.write(f"[{src}]\n{err}\n")
    return obj


# the sources that carry timestamps; the timeline build shares every other object with the product build
STAMPED = {"matvec_q4k.hip", "matvec_q6k.hip", "sdpa_q40_lanes.hip"}


def _link(objs: list[str], path: str) -> str:
    tmp = path + ".tmp"
    cmd = ["hipcc", "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, path)
    return path


def build(jobs: int = 8) -> str:
    """Compiles every source and links the library, then the timeline build beside it."""
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
        stamped = dict(zip(sorted(STAMPED), ex.map(lambda f: _compile(f, True), sorted(STAMPED))))
    _link(objs, LIB_PATH)
    _link([stamped.get(f, o) for f, o in zip(srcs, objs)], STAMPS_LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
