"""Builds quant_flash_attn_amd/libqfa.so from csrc/ with hipcc for gfx950.

    python -m quant_flash_attn_amd.build          # compile every translation unit, then link

The library is built in-tree so that a source snapshot carries it along; nothing is
JIT-compiled at import time.  Compilation needs no GPU (hipcc cross-compiles).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libqfa.so")
OBJ_DIR = os.path.join(HERE, "build")

# -packed-fp32-ops: keep hipcc from forming v_pk_*_f32 out of scalar float code.
COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# the quantizer must evaluate its expressions as single IEEE operations (bit-exact codes)
PER_FILE = {"qfa_quant.hip": ["-ffp-contract=off", "-fno-fast-math"]}
SOURCES = ["qfa_api.cpp", "qfa_quant.hip", "qfa_fwd.hip", "qfa_bwd.hip", "qfa_skv.hip", "qfa_skv_bwd.hip", "qfa_skv_bwd_long.hip"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src: str, extra=()) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *COMMON, *PER_FILE.get(src, []), *extra, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless, not shown
    noise = ("packed-fp32-ops", "is not a recognized feature")
    for line in res.stderr.splitlines():
        if line.strip() and not any(n in line for n in noise):
            print(line, file=sys.stderr)
    return obj


def build_library(extra_flags=(), jobs: int = 4) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, extra_flags), SOURCES))
    tmp = LIB + ".tmp"
    res = subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build_library())
