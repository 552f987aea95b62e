"""cw_colsum_static -- the entry point that allocates nothing -- against cw_colsum, both through the C ABI.

The static variant runs cw_colsum's kernels over the library's own scratch array instead of a caller's
workspace, so the bar is bit equality with cw_colsum (and the fp32 bar against a float64 sum). Two calls in
a row share the array; the second, smaller one must not see what the first left there.
"""
import ctypes

import pytest
import torch

from tests.util import randn, rel_err

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _colsum_ws(lib, dy):
    from cubework_amd import _lib
    M, N = dy.shape
    nbytes = lib.cw_colsum_workspace_bytes(M, N)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dy.device)
    out = torch.empty(N, dtype=torch.float32, device=dy.device)
    dt = {torch.bfloat16: _lib.CW_BF16, torch.float32: _lib.CW_F32, torch.float16: _lib.CW_F16}[dy.dtype]
    _lib.check(lib.cw_colsum(M, N, dy.data_ptr(), dy.stride(0), out.data_ptr(), _lib.CW_F32, ws.data_ptr(), nbytes, dt, _stream()),
               "cw_colsum")
    return out


def _colsum_static(lib, dy, out):
    from cubework_amd import _lib
    M, N = dy.shape
    dt = {torch.bfloat16: _lib.CW_BF16, torch.float32: _lib.CW_F32, torch.float16: _lib.CW_F16}[dy.dtype]
    _lib.check(lib.cw_colsum_static(M, N, dy.data_ptr(), dy.stride(0), out.data_ptr(), _lib.CW_F32, dt, _stream()),
               "cw_colsum_static")
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_colsum_matches_colsum_on_two_calls_in_a_row(dtype):
    from cubework_amd import _lib
    lib = _lib.load()
    torch.cuda.set_device(0)
    big = randn((8192, 2048), dtype, 11).to(DEV)
    small = randn((300, 520), dtype, 12).to(DEV)
    out_big = torch.empty(2048, dtype=torch.float32, device=DEV)
    out_small = torch.empty(520, dtype=torch.float32, device=DEV)
    _colsum_static(lib, small, out_small)   # the first call on the device looks the scratch array's address up
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]   # hipMemGetInfo: sees any hipMalloc / hipFree, torch's or not
    # back to back on one stream, the second call smaller than the first
    _colsum_static(lib, big, out_big)
    _colsum_static(lib, small, out_small)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed by the calls"
    for dy, got in ((big, out_big), (small, out_small)):
        assert torch.equal(got, _colsum_ws(lib, dy)), "static scratch and caller scratch give different bits"
        want = dy.cpu().double().sum(0)
        # one fp32 rounding per addition of M terms of magnitude <= max|dy|: error <= M * 2^-24 * max|dy| per column,
        # measured against the largest column sum
        bound = dy.shape[0] * 2.0 ** -24 * dy.abs().max().item() / want.abs().max().item()
        err = rel_err(got, want)
        print("colsum_static %s %s: rel err %.2e (bound %.2e)" % (tuple(dy.shape), dtype, err, bound))
        assert err <= max(1e-5, bound)


def test_static_colsum_unaligned_and_empty():
    from cubework_amd import _lib
    lib = _lib.load()
    parent = randn((77, 131), torch.float32, 13).to(DEV)
    view = parent[:, 1:128]  # unaligned base, ragged width: the element-wise kernel
    out = torch.empty(127, dtype=torch.float32, device=DEV)
    _colsum_static(lib, view, out)
    assert torch.equal(out, _colsum_ws(lib, view))
    assert rel_err(out, view.cpu().double().sum(0)) <= 1e-5
    # no rows: zeros
    out.fill_(7.0)
    _lib.check(lib.cw_colsum_static(0, 127, None, 127, out.data_ptr(), _lib.CW_F32, _lib.CW_F32, _stream()), "empty")
    assert torch.equal(out, torch.zeros_like(out))


def test_static_colsum_refuses_what_does_not_fit():
    from cubework_amd import _lib
    lib = _lib.load()
    assert lib.cw_colsum_static_max_bytes() == 4 << 20
    # ragged width: one partial row per 64 rows, 128 * 8201 floats do not fit
    dy = torch.zeros((8192, 8201), dtype=torch.bfloat16, device=DEV)
    out = torch.empty(8201, dtype=torch.float32, device=DEV)
    rc = lib.cw_colsum_static(8192, 8201, dy.data_ptr(), 8201, out.data_ptr(), _lib.CW_F32, _lib.CW_BF16, _stream())
    assert rc == -3 and b"static scratch" in lib.cw_last_error()
    # 128 * 8191 floats do
    dy = randn((8192, 8191), torch.bfloat16, 14).to(DEV)
    out = torch.empty(8191, dtype=torch.float32, device=DEV)
    _colsum_static(lib, dy, out)
    assert torch.equal(out, _colsum_ws(lib, dy))
    # aligned operands keep one partial row per block of rows: a wide aligned operand fits
    dy = randn((1024, 16384), torch.bfloat16, 15).to(DEV)
    out = torch.empty(16384, dtype=torch.float32, device=DEV)
    _colsum_static(lib, dy, out)
    assert torch.equal(out, _colsum_ws(lib, dy))


def test_static_colsum_small_call_after_a_large_one_that_left_nan_in_the_scratch():
    """Calls share the scratch array, which keeps the last call's contents: a large first call whose input holds
    NaN fills its partial rows with NaN; the smaller call that follows must not read any of them."""
    from cubework_amd import _lib
    lib = _lib.load()
    big = torch.full((8192, 2048), float("nan"), dtype=torch.float32, device=DEV)
    out_big = torch.empty(2048, dtype=torch.float32, device=DEV)
    _colsum_static(lib, big, out_big)
    torch.cuda.synchronize()
    assert torch.isnan(out_big).all()
    for shape, seed in (((300, 520), 31), ((77, 127), 32), ((4096, 1024), 33)):
        small = randn(shape, torch.float32, seed).to(DEV)
        out = torch.empty(shape[1], dtype=torch.float32, device=DEV)
        _colsum_static(lib, small, out)
        torch.cuda.synchronize()
        assert torch.isfinite(out).all(), "stale partial rows of the previous call were read"
        assert torch.equal(out, _colsum_ws(lib, small))


def test_static_colsum_in_a_hip_graph():
    """What the entry point is for: after one call outside a capture (the address lookup), the call is recorded
    into a HIP graph; three replays, with eager work and synchronisations between them and new input values each
    time, equal cw_colsum bit for bit."""
    from cubework_amd import _lib
    lib = _lib.load()
    dy = randn((4096, 1024), torch.bfloat16, 41).to(DEV)
    out = torch.empty(1024, dtype=torch.float32, device=DEV)
    _colsum_static(lib, dy, out)       # outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _colsum_static(lib, dy, out)
    torch.cuda.current_stream().wait_stream(side)
    for k in range(3):
        dy.copy_(randn((4096, 1024), torch.bfloat16, 50 + k).to(DEV))   # eager work between the replays
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, _colsum_ws(lib, dy)), "replay %d" % k


def test_static_colsum_first_call_inside_a_capture_is_refused():
    """In a fresh process the first call on a device, made on a capturing stream, returns CW_ERR_UNSUPPORTED with
    the reason and records nothing; the capture goes on, and after a call outside a capture the entry point can
    be captured."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import ctypes, sys, torch
sys.path.insert(0, %r)
from cubework_amd import _lib
lib = _lib.load()
dev = "cuda:0"
dy = torch.ones((256, 512), dtype=torch.float32, device=dev)
out = torch.zeros(512, dtype=torch.float32, device=dev)
marker = torch.zeros(4, device=dev)
torch.cuda.synchronize()
side = torch.cuda.Stream()
g = torch.cuda.CUDAGraph()
with torch.cuda.stream(side):
    with torch.cuda.graph(g, stream=side):
        raw = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.cw_colsum_static(256, 512, dy.data_ptr(), 512, out.data_ptr(), _lib.CW_F32, _lib.CW_F32, raw)
        marker.add_(1.0)
assert rc == _lib.CW_ERR_UNSUPPORTED, rc
assert b"capture" in lib.cw_last_error(), lib.cw_last_error()
g.replay(); torch.cuda.synchronize()
assert float(marker[0]) == 1.0 and float(out.abs().sum()) == 0.0     # the graph holds the add only
raw = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
assert lib.cw_colsum_static(256, 512, dy.data_ptr(), 512, out.data_ptr(), _lib.CW_F32, _lib.CW_F32, raw) == 0
torch.cuda.synchronize()
assert bool((out == 256.0).all())
print("ok")
''' % root
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and "ok" in proc.stdout, proc.stdout + proc.stderr
