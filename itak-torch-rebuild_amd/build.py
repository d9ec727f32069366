"""Compiles the HIP sources in csrc/ for gfx950 into lib/libitak_hip_kv.so.

Run as `python build.py` from this directory, or call build() from Python. The library is
built in-tree so that it travels with the source tree; nothing is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libitak_hip_kv.so")
TIMELINE_LIB_PATH = os.path.join(LIB_DIR, "libitak_hip_kv_timeline.so")
OBJ_DIR = os.path.join(HERE, "build")

ARCH = "gfx950"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed FP32 VALU forms are kept off: ordinary float code must compile to scalar FP32 ops.
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    "-Rpass-analysis=kernel-resource-usage", "-fno-caret-diagnostics",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


# Sources whose kernels the timeline run never reads stamps of: in the measurement build they are
# compiled as in the ordinary one (the stamps cost registers, and the block kernel's forms at
# head dims other than 128 have none to spare).
NO_STAMPS = {"attn_prefill_f16_dims.hip"}


def _compile(src: str, timeline: bool = False) -> str:
    obj = os.path.join(OBJ_DIR + ("_timeline" if timeline else ""), src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, *(["-DITAK_TIMELINE"] if timeline and src not in NO_STAMPS else []), "-c",
           os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    raw = res.stderr.splitlines()
    # (Notes and remarks about code in a header arrive under an "In file included from" line.)
    lines = [l for i, l in enumerate(raw) if noise not in l and not (
        l.startswith("In file included from") and i + 1 < len(raw) and
        (noise in raw[i + 1] or "remark:" in raw[i + 1]))]
    remarks = [l for l in lines if "-Rpass-analysis=kernel-resource-usage" in l]
    err = "\n".join(l for l in lines if l not in remarks and "remark" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    # No kernel may spill registers to scratch memory: spilled variants of the attention
    # kernels have produced wrong results on the target, and they are slow anyway.
    name = "?"
    for l in remarks:
        if "Function Name:" in l:
            name = l.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in l:
            size = int(l.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if size:
                raise RuntimeError(f"{src}: kernel {name} spills {size} bytes/lane to scratch")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False, timeline: bool = False) -> str:
    """Builds lib/libitak_hip_kv.so; with `timeline`, lib/libitak_hip_kv_timeline.so instead: the
    same library with stage timestamps compiled into the attention kernels (csrc/timeline.h),
    which `bench.py --timeline` loads. The measurement build is never the one tests or
    benchmarks of throughput run."""
    os.makedirs(OBJ_DIR + ("_timeline" if timeline else ""), exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(lambda src: _compile(src, timeline), srcs))
    lib_path = TIMELINE_LIB_PATH if timeline else LIB_PATH
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-pthread", "-o", lib_path, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {lib_path}")
    return lib_path


if __name__ == "__main__":
    build(verbose=True, timeline="--timeline" in sys.argv[1:])
