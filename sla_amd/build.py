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


# Host-side sanitizers for the validation layer (every entry point checks its arguments before it launches anything):
# address and undefined-behaviour checks in the host code only; the device code is compiled as usual.
SANITIZE_FLAGS = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
                  "-fno-omit-frame-pointer", "-g"]
SAN_LIBPATH = os.path.join(LIBDIR, "libsla_hip_san.so")


def _compile(src: str, force: bool, sanitized: bool = False) -> str:
    obj = os.path.join(LIBDIR, src.replace(".hip", ".san.o" if sanitized else ".o"))
    srcp = os.path.join(CSRC, src)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps = [srcp, *headers, os.path.join(HERE, "..", "include", "sla_hip.h"), __file__]
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj
    flags = list(COMMON_FLAGS)
    if sanitized:
        flags += SANITIZE_FLAGS
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


def build_sanitized(force: bool = False) -> str:
    """The same library with AddressSanitizer and UndefinedBehaviorSanitizer in its host code
    (``sla_amd/lib/libsla_hip_san.so``), for running the argument-validation tests under them on a machine without a GPU.
    Load it with the sanitizer runtime preloaded (``asan_runtime()``)."""
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, sanitized=True), SOURCES))
    if not force and os.path.exists(SAN_LIBPATH) and all(os.path.getmtime(SAN_LIBPATH) >= os.path.getmtime(o) for o in objs):
        return SAN_LIBPATH
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fsanitize=address", "-fsanitize=undefined",
           "-shared-libsan", "-o", SAN_LIBPATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return SAN_LIBPATH


def asan_runtime() -> str:
    """Path of the AddressSanitizer runtime the sanitized library needs preloaded."""
    res = subprocess.run([_hipcc(), "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True, text=True)
    path = res.stdout.strip()
    if res.returncode != 0 or not os.path.isabs(path):
        raise RuntimeError("no AddressSanitizer runtime found next to hipcc")
    return os.path.realpath(path)


if __name__ == "__main__":
    build(force="--incremental" not in sys.argv, verbose=True)
