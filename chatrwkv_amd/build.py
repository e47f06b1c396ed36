"""Builds chatrwkv_amd/librwkv_hip.so from csrc/*.hip with hipcc for gfx950.

    python -m chatrwkv_amd.build

Cross-compiles without a GPU.  The shared library has no dependency on torch: it links
only the HIP runtime, and is loaded with ctypes (chatrwkv_amd/lib.py).
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "librwkv_hip.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(src):
    obj = os.path.join(CSRC, "build", os.path.basename(src)[:-4] + ".o")
    cmd = ["hipcc", *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{log}")
    return obj, log


def build(verbose=True):
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(_compile, srcs))
    for obj, log in results:
        if verbose and log.strip():
            print(log, file=sys.stderr)
    objs = [o for o, _ in results]
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", OUT)
    return OUT


if __name__ == "__main__":
    build()
