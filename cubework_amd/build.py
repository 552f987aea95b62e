"""Build libcubework_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc.

    python -m cubework_amd.build          # compile every source, link

hipcc cross-compiles for gfx950 without a GPU. The library is written next to
this file so that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libcubework_hip.so")

SOURCES = ["cw_api.hip", "gemm_bf16.hip", "gemm_bf16_nn.hip", "gemm_bf16_nt.hip", "gemm_bf16_tn.hip", "gemm_bf16_dma_nn.hip", "gemm_bf16_dma_nt.hip", "gemm_bf16_dma_tn.hip",
           "gemm_f32.hip", "epilogue.hip", "layernorm.hip", "vpce.hip"]

# Packed-fp32 VALU forms are kept off: plain float code only.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, proc.stdout, proc.stderr))
    return obj


def build(verbose=True):
    """Compile every HIP source for gfx950 and link the shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (proc.stdout, proc.stderr))
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH, os.path.getsize(LIB_PATH), "bytes")
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
