"""Compile the HIP sources in ../csrc for gfx950 into mvpa_hip/libmvpa_hip.so (in-tree)."""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG), "include")
LIB = os.path.join(HERE, "libmvpa_hip.so")

SOURCES = ["mvpa_api.hip", "mvpa_generic.hip", "mvpa_mfma.hip", "mvpa_mfma64.hip", "mvpa_mfma128.hip", "mvpa_dense.hip", "mvpa_backward.hip",
           "mvpa_backward_mfma.hip", "mvpa_static_ws.hip", "mvpa_fp8.hip"]

# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU instructions.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I", INCLUDE, "-I", CSRC,
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src: str, extra) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def build(verbose: bool = True, extra_flags=()) -> str:
    """Compile every source (always, even if the library exists) and link the shared library."""
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with cf.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(lambda s: _compile(s, list(extra_flags)), sources))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB}", file=sys.stderr)
    return LIB


if __name__ == "__main__":
    build()
