"""Build libinfmoe.so (host C++ + gfx950 HIP kernels) in-tree with hipcc.

    python -m infmoe_amd.build                 # compile every source, then link
    python -m infmoe_amd.build --incremental   # recompile only what is older than its source or any header
Objects go to infmoe_amd/csrc/build/, the library to infmoe_amd/lib/libinfmoe.so.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libinfmoe.so")

SOURCES = [
    "kernels/dispatch.hip",
    "kernels/norm.hip",
    # the six instantiations of the matrix-core expert kernel first: they take longest
    "kernels/expert_gemm_grouped_gated.hip",
    "kernels/expert_gemm_one_gated.hip",
    "kernels/expert_gemm_grouped_relu.hip",
    "kernels/expert_gemm_one_relu.hip",
    "kernels/expert_gemm_grouped.hip",
    "kernels/expert_gemm_one.hip",
    "kernels/expert_gemm_small_grouped_relu.hip",
    "kernels/expert_gemm_small_grouped.hip",
    "kernels/expert_gemm_small_one_relu.hip",
    "kernels/expert_gemm_small_one.hip",
    "kernels/expert_gemm.hip",
    "kernels/gating.hip",
    "kernels/gating_slab.hip",
    "kernels/expert_skinny.hip",
    "sublayers/t5ff_layer.cpp",
    "sublayers/sublayer.cpp",
    "npz_reader.cpp",
    "moe_layer.cpp",
    "c_api.cpp",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result"]
# packed FP32 instructions are switched off for all device code
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _newest_header() -> float:
    newest = 0.0
    for top in (os.path.join(HERE, "..", "include"), CSRC):  # the public headers are included by the sources too
        for root, _, files in os.walk(top):
            for f in files:
                if f.endswith(".h"):
                    newest = max(newest, os.path.getmtime(os.path.join(root, f)))
    return newest


def _compile(src: str, incremental: bool = False) -> str:
    obj = os.path.join(OBJ_DIR, src.replace("/", "_") + ".o")
    if incremental and os.path.isfile(obj):
        if os.path.getmtime(obj) > max(os.path.getmtime(os.path.join(CSRC, src)), _newest_header()):
            return obj
    cmd = [HIPCC, *COMMON, *DEVICE, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(f"[{src}]\n{warn}\n")
    return obj


def build(jobs: int = 8, incremental: bool = False) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, incremental), SOURCES))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-lz", "-o", LIB_PATH]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(incremental="--incremental" in sys.argv[1:]))
