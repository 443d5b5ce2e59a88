"""Builds libscanet_hip.so (gfx950 only) from csrc/*.hip with hipcc.

    python scanet3_amd/build.py

The objects and the library stay in-tree next to this file; nothing is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libscanet_hip.so")

SOURCES = ["runtime.hip", "optim_kernels.hip", "elementwise_kernels.hip", "batchnorm_kernels.hip", "random_kernels.hip", "gemm_kernels.hip", "conv_ring_kernels.hip", "conv_wgrad_kernels.hip", "gemm_bf16.hip", "lstm_kernels.hip", "lstm_wgrad_kernels.hip", "mlp2_kernels.hip", "model.hip"]

# -ffp-contract=off: one rounding per reference op (TensorFlow evaluates Mul and Add separately).
# -packed-fp32-ops is switched off: some packed fp32 forms have produced wrong values on this hardware.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def build_library(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    missing = [s for s in SOURCES if not os.path.exists(os.path.join(CSRC, s))]
    if missing:
        raise FileNotFoundError(f"sources listed in build.py are missing from {CSRC}: {missing}")
    sources = list(SOURCES)
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(_compile, sources))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(objs)} objects")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
