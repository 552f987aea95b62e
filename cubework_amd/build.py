"""Build libcubework_hip.so (the gfx950 kernels + C ABI) and libcubework_diag.so (measurement aids that only
bench.py and their tests load) in-tree with hipcc.

    python -m cubework_amd.build          # compile every source, link both

hipcc cross-compiles for gfx950 without a GPU. The libraries are written next to
this file so that they travel with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libcubework_hip.so")

SOURCES = ["gemm_bf16_tn.hip", "gemm_f16_tn.hip", "gemm_bf16_nn.hip", "gemm_f16_nn.hip", "gemm_bf16_nt.hip", "gemm_f16_nt.hip",  # slowest first
           "gemm_bf16_dma_nn.hip", "gemm_bf16_dma_nt.hip", "gemm_bf16_dma_tn.hip", "gemm_f16_dma_nn.hip", "gemm_f16_dma_nt.hip", "gemm_f16_dma_tn.hip",
           "cw_runtime.hip", "cw_api.hip", "gemm_plan.hip", "gemm_bf16.hip", "gemm_half_small.hip", "gemm_f32.hip", "epilogue.hip", "layernorm.hip", "vpce.hip", "attention.hip", "attention_bwd.hip", "embedding.hip", "embed_sort.hip", "clip_grad.hip"]
# the measurement library: its own kernels plus the runtime services (error text, device check), nothing else
DIAG_SOURCES = ["diag_gemm.hip", "diag.hip"]
DIAG_LIB_PATH = os.path.join(HERE, "libcubework_diag.so")

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


def _compile(src, extra=(), obj_dir=None):
    obj = os.path.join(obj_dir or OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, proc.stdout, proc.stderr))
    return obj


def build(verbose=True, extra_flags=(), lib_path=None, obj_dir=None):
    """Compile every HIP source for gfx950 and link the shared library.
    extra_flags / lib_path / obj_dir build a variant beside the default one."""
    lib_path = lib_path or LIB_PATH
    obj_dir = obj_dir or OBJ_DIR
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(lambda src: _compile(src, extra_flags, obj_dir), SOURCES + DIAG_SOURCES))
    by_src = dict(zip(SOURCES + DIAG_SOURCES, objs))

    def link(members, path):
        tmp = path + ".tmp"
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *[by_src[m] for m in members], "-o", tmp]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (proc.stdout, proc.stderr))
        os.replace(tmp, path)
        if verbose:
            print("built", path, os.path.getsize(path), "bytes")

    link(SOURCES, lib_path)
    diag_path = DIAG_LIB_PATH if lib_path == LIB_PATH else os.path.splitext(lib_path)[0] + "_diag.so"
    link(DIAG_SOURCES + ["cw_runtime.hip"], diag_path)
    return lib_path


if __name__ == "__main__":
    build()
    sys.exit(0)
