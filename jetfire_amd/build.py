"""Builds libjetfire_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

`python -m jetfire_amd.build` compiles every source under jetfire_amd/csrc and links the shared
library next to the package; `--debug-hooks` adds the measurement / test entry points the tests and bench.py use.
Nothing here needs a GPU: hipcc cross-compiles.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "libjetfire_amd.so")

SOURCES = (     # (the long compilations first: the pool starts them together)
    "fused_full_a.hip",
    "fused_full_b.hip",
    "fused_full_c.hip",
    "fused_full_d.hip",
    "fused_full_e.hip",
    "quant_write.hip",
    "unpack.hip",
    "shadow_write.hip",
    "qk_scores.hip",
    "topk.hip",
    "softmax_v.hip",
    "fused_scan.hip",
    "fused_stage_a.hip",
    "fused_stage_b.hip",
    "blend.hip",
    "calibrate.hip",
    "cpu_topk_attn.cpp",
)

COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-fast-math",
    "-fhip-fp32-correctly-rounded-divide-sqrt",   # the quantiser needs IEEE division
    "-ffp-contract=off",                          # fused multiply-adds only where the source spells them
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def _extra_flags(debug_hooks: bool) -> list:
    extra = os.environ.get("JETFIRE_BUILD_FLAGS", "").split()   # e.g. -DNAME for a measurement variant
    if debug_hooks or os.environ.get("JETFIRE_DEBUG_HOOKS", "0") == "1":
        extra.append("-DJF_DEBUG_HOOKS")                         # the hooks of include/jetfire_amd_debug.h
    return extra


def build_id(extra: list) -> str:
    """Digest of everything the library is made from (sources, headers, flags): jf_version() carries it, so a
    measurement can name the exact code it ran."""
    h = hashlib.sha256()
    names = sorted(os.listdir(CSRC)) + ["../../include/jetfire_amd.h", "../../include/jetfire_amd_debug.h"]
    for name in names:
        path = os.path.join(CSRC, name)
        if os.path.isfile(path):
            h.update(name.encode())
            with open(path, "rb") as f:
                h.update(f.read())
    h.update(" ".join(COMMON_FLAGS + sorted(extra)).encode())
    return h.hexdigest()[:12]


def _compile(src: str, extra: list) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *COMMON_FLAGS, *extra, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    noise = ("packed-fp32-ops", "is not a recognized feature")
    warn = "\n".join(l for l in res.stderr.splitlines() if l.strip() and not any(n in l for n in noise))
    if "warning:" in warn:
        sys.stderr.write(warn + "\n")
    return obj


def build_library(verbose: bool = True, debug_hooks: bool = False) -> str:
    """Compile all sources (always, even when a library is already there) and link the .so.  `debug_hooks` (or
    JETFIRE_DEBUG_HOOKS=1) compiles the measurement / test entry points of include/jetfire_amd_debug.h in: the tests
    and bench.py need them, a product build leaves them out."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    extra = _extra_flags(debug_hooks)
    extra = extra + [f'-DJF_BUILD_ID="{build_id(extra)}"']
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda src: _compile(src, extra), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp, "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[jetfire_amd] built {LIB_PATH} ({os.path.getsize(LIB_PATH) // 1024} KiB)")
    return LIB_PATH


if __name__ == "__main__":
    build_library(debug_hooks="--debug-hooks" in sys.argv[1:])
