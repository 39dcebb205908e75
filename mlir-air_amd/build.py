"""Build libw4a16_hip.so (gfx950) in-tree with hipcc.

    python mlir-air_amd/build.py [-j JOBS]

Output: mlir-air_amd/lib/libw4a16_hip.so.  Cross-compiles without a GPU.
"""

import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libw4a16_hip.so")
SOURCES = ["capi.hip", "dequant.hip", "stream.hip", "gemv_ws.hip", "gemm_ws.hip", "gemm_wsk.hip", "gemm.hip", "attention.hip", "q4nx.hip", "lm_head.hip", "prefill_block.hip", "prefill_attention.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    *os.environ.get("W4A16_EXTRA", "").split(),
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU ops are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first kernel arguments arrive in SGPRs with the wave instead of through scalar loads at its start
    # (decode GEMV 6.09 -> 5.88 us); only kernels with plain scalar / pointer arguments gain
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


# Per-file flags.  The prompt-pass attention takes maxima over MFMA results: without the promise that they are not
# NaN the compiler canonicalises every one of them first (one more VALU instruction per score).
FILE_FLAGS = {"prefill_attention.hip": ["-fno-honor-nans"]}


def _compile(src, extra):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *FILE_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(
        line for line in (res.stdout + res.stderr).splitlines()
        if "packed-fp32-ops" not in line and "unrecognized feature" not in line
    )
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{out}")
    return obj, out


def build(jobs=4, extra=(), verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda s: _compile(s, list(extra)), SOURCES))
    for _, out in results:
        if out.strip() and verbose:
            print(out)
    objs = [o for o, _ in results]
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=4)
    ap.add_argument("-v", action="store_true")
    ap.add_argument("--save-temps", action="store_true", help="keep ISA (.s) files under build/")
    a = ap.parse_args()
    extra = ["-save-temps=obj"] if a.save_temps else []
    print(build(a.j, extra, a.v or True))
