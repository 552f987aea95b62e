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
    _lib.check(lib.cw_colsum(M, N, dy.data_ptr(), dy.stride(0), out.data_ptr(), ws.data_ptr(), nbytes, dt, _stream()),
               "cw_colsum")
    return out


def _colsum_static(lib, dy, out):
    from cubework_amd import _lib
    M, N = dy.shape
    dt = {torch.bfloat16: _lib.CW_BF16, torch.float32: _lib.CW_F32, torch.float16: _lib.CW_F16}[dy.dtype]
    _lib.check(lib.cw_colsum_static(M, N, dy.data_ptr(), dy.stride(0), out.data_ptr(), dt, _stream()),
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
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    # back to back on one stream, the second call smaller than the first
    _colsum_static(lib, big, out_big)
    _colsum_static(lib, small, out_small)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
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
    _lib.check(lib.cw_colsum_static(0, 127, None, 127, out.data_ptr(), _lib.CW_F32, _stream()), "empty")
    assert torch.equal(out, torch.zeros_like(out))


def test_static_colsum_refuses_what_does_not_fit():
    from cubework_amd import _lib
    lib = _lib.load()
    assert lib.cw_colsum_static_max_bytes() == 4 << 20
    # ragged width: one partial row per 64 rows, 128 * 8201 floats do not fit
    dy = torch.zeros((8192, 8201), dtype=torch.bfloat16, device=DEV)
    out = torch.empty(8201, dtype=torch.float32, device=DEV)
    rc = lib.cw_colsum_static(8192, 8201, dy.data_ptr(), 8201, out.data_ptr(), _lib.CW_BF16, _stream())
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
