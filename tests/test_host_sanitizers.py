"""The library's host-side planning and validation code under the address and undefined-behaviour sanitizers, on
the CPU: tests/host/plan_harness.hip drives cubework_amd/csrc/gemm_plan.hip (argument checks of cw_gemm_ksteps,
the choice of kernel, strip / k-tail / split-k cuts, scratch sizes, the column sums' slabs) over ragged, huge,
zero and misaligned shapes and checks that every launch a plan describes stays inside the caller's buffers.
No GPU call is made. hipcc compiles the three small translation units in a few seconds."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "cubework_amd", "csrc")


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    return None


def test_planning_code_is_clean_under_asan_and_ubsan(tmp_path):
    hipcc = _hipcc()
    if hipcc is None:
        pytest.skip("hipcc not found")
    exe = str(tmp_path / "plan_harness")
    cmd = [hipcc, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined",
           os.path.join(ROOT, "tests", "host", "plan_harness.hip"), os.path.join(CSRC, "gemm_plan.hip"),
           os.path.join(CSRC, "cw_runtime.hip"), "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stdout + build.stderr
    syms = subprocess.run(["nm", exe], capture_output=True, text=True).stdout
    assert "__asan_init" in syms and "__ubsan_handle" in syms, "the harness was built without the sanitizers"
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr, run.stderr
    m = re.match(r"ok (\d+) routes (.*)", run.stdout.strip())
    assert m, run.stdout
    routes = dict((k, int(v)) for k, v in (kv.split("=") for kv in m.group(2).split()))
    assert int(m.group(1)) > 100000
    assert all(v > 0 for v in routes.values()), "a kernel route was never planned: %s" % routes
