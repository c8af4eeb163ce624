"""Build recipe for libclgrpo.so (HIP kernels + C ABI), gfx950 only.

``python -m chatlearn_amd.build`` compiles every source under ``csrc/`` with
hipcc and links them into ``chatlearn_amd/csrc/libclgrpo.so`` (in-tree, so the
library travels with the source tree).  hipcc cross-compiles without a GPU.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(CSRC, "libclgrpo.so")

SOURCES = [
    "common.hip",
    "lmhead_fwd.hip",
    "lmhead_bwd.hip",
    "loss_kernels.hip",
    "index_kernels.hip",
    "advantage.hip",
    "softmax_stats.hip",
    "packing_host.cpp",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON_FLAGS = ["-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function"]
# Packed-fp32 instruction selection is switched off for all device code.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# advantage.hip reproduces numpy's float64 rounding step by step: no fused multiply-adds there.
PER_FILE_FLAGS = {"advantage.hip": ["-ffp-contract=off"]}


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + COMMON_FLAGS
    if src.endswith(".hip"):
        cmd += DEVICE_FLAGS
    cmd += PER_FILE_FLAGS.get(src, [])
    cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build()
