"""Builds the HIP kernels into one shared library, in-tree, for gfx950.

`python -m sla_amd.build` or `sla_amd.build.build()`.  Each source is compiled
to an object with hipcc and the objects are linked into
``sla_amd/lib/libsla_hip.so``; nothing is installed outside the tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBPATH = os.path.join(LIBDIR, "libsla_hip.so")

SOURCES = ["capi.hip", "block_map.hip", "sparse_fwd.hip", "linear.hip", "linear_bwd.hip", "sparse_bwd.hip", "sage.hip",
           "linear_complement.hip", "module_bwd.hip"]

COMMON_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]
# sources whose results must follow a fixed fp32 rounding sequence
NO_CONTRACT = {"block_map.hip"}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
    srcp = os.path.join(CSRC, src)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps = [srcp, *headers, os.path.join(HERE, "..", "include", "sla_hip.h"), __file__]
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj
    flags = list(COMMON_FLAGS)
    if src in NO_CONTRACT:
        flags.append("-ffp-contract=off")
    cmd = [_hipcc(), *flags, "-c", srcp, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIBPATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIBPATH}")
    return LIBPATH


if __name__ == "__main__":
    build(force="--incremental" not in sys.argv, verbose=True)
