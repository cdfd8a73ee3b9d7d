"""Builds libmi355x_fattn.so (hand-written HIP for gfx950) in-tree with hipcc."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmi355x_fattn.so")
SOURCES = ["api.hip", "fattn_vec.hip", "fattn_mma.hip", "fattn_decode.hip", "cpy.hip", "relpos.hip", "fattn_relpos.hip"]

# packed-fp32 VALU ops are switched off for all device code of this library
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


PER_FILE_FLAGS: dict = {}


def _compile(src: str, extra) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_FILE_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(extra_flags=(), jobs: int = 4) -> str:
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    return LIB


HOST_SRC = os.path.join(HERE, "host", "attn_protocol.cpp")
HOST_BIN = os.path.join(HERE, "host", "mi355x_attn_protocol")


def build_host_driver() -> str:
    """The native host driver above the C ABI (plain g++; it links only libmi355x_fattn.so)."""
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-I", os.path.join(os.path.dirname(HERE), "include"), HOST_SRC, "-o", HOST_BIN,
           "-L", HERE, "-lmi355x_fattn", "-Wl,-rpath,$ORIGIN/.."]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("host driver build failed:\n" + res.stderr)
    return HOST_BIN


if __name__ == "__main__":
    print(build_library(sys.argv[1:]))
    print(build_host_driver())
