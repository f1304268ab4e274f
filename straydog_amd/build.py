"""Builds libstraydog_gpu.so (and libstraydog_gpu.a for static linking, as the reference's Rust host links it)
from straydog_amd/csrc/*.hip with hipcc for gfx950.  Run as `python -m straydog_amd.build`."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libstraydog_gpu.so")
ARCHIVE = os.path.join(HERE, "libstraydog_gpu.a")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    # packed FP32 arithmetic is kept off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# The attention kernels never form a NaN from finite inputs (masked scores are -inf, the running maximum starts at a large
# finite negative number), so their maxima need no NaN-quieting instructions.
EXTRA = {"paged_attention.hip": ["-fno-honor-nans"], "prefill_attention.hip": ["-fno-honor-nans"]}


def _compile(source):
    obj = os.path.join(OBJ, os.path.basename(source) + ".o")
    subprocess.run(["hipcc", *FLAGS, *EXTRA.get(os.path.basename(source), []), "-c", source, "-o", obj], check=True)
    return obj


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objects = list(pool.map(_compile, sources))
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objects], check=True)
    if os.path.exists(ARCHIVE):
        os.remove(ARCHIVE)
    subprocess.run(["ar", "rcs", ARCHIVE, *objects], check=True)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
