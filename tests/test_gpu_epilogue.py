"""GPU parity of the bias-gradient column sum and the fused-activation
backward (through the C ABI) against the CPU oracle."""
import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
SHAPES = [(8192, 2048), (100, 1000), (33, 8), (5, 7), (1000, 520), (4096, 64)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
def test_colsum(shape, dtype):
    import oracle
    from cubework_amd import ops

    M, N = shape
    dy = randn((M, N), dtype, 1)
    got = ops.colsum(dy.to(DEV))
    with oracle.precision(torch.float64):
        want = oracle.colsum(dy)
    # a sum of M terms per column, against its float64 value
    assert_parity(got, want, torch.float32, "colsum")
    # determinism: two runs are bit identical
    assert torch.equal(got, ops.colsum(dy.to(DEV)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("act", [None, "gelu_tanh", "gelu_erf", "relu"])
@pytest.mark.parametrize("shape", [(1024, 512), (77, 130), (9, 5)])
def test_act_bwd_colsum(shape, act, dtype):
    import oracle
    from cubework_amd import ops

    M, N = shape
    dy = randn((M, N), dtype, 2)
    pre = randn((M, N), dtype, 3, std=1.5)
    dpre, dbias = ops.act_bwd_colsum(act, dy.to(DEV), pre.to(DEV))
    with oracle.precision(torch.float64):
        want_dpre, want_dbias = oracle.act_bwd_colsum(act, dy, pre)
    assert_parity(dpre, want_dpre, dtype, "dPre")
    assert_parity(dbias, want_dbias, torch.float32, "dbias")
    dpre2, none = ops.act_bwd_colsum(act, dy.to(DEV), pre.to(DEV), want_dbias=False)
    assert none is None and torch.equal(dpre, dpre2)


def test_colsum_padded_rows():
    import oracle
    from cubework_amd import ops

    parent = randn((300, 136), torch.bfloat16, 4).to(DEV)
    view = parent[:, :128]
    with oracle.precision(torch.float64):
        want = oracle.colsum(view.cpu())
    assert_parity(ops.colsum(view), want, torch.float32, "padded colsum")


def test_mfma_rate_diagnostic_runs_in_every_mode():
    """cw_diag_mfma_rate (the measurement aid behind bench.py's MFMA ceilings, in the measurement library): zero
    operands leave zero sums; random operands, from registers or read from LDS, leave finite non-zero ones, the
    same on every call."""
    from cubework_amd import _diag

    lib = _diag.load()
    sink = torch.full((65536,), float("nan"), dtype=torch.float32, device=DEV)
    assert lib.cw_diag_mfma_rate(3, 1, sink.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(sink, torch.zeros_like(sink))
    for mode in (0, 2):
        runs = []
        for _ in range(2):
            sink.fill_(float("nan"))
            assert lib.cw_diag_mfma_rate(4, mode, sink.data_ptr(), None) == 0
            torch.cuda.synchronize()
            runs.append(sink.clone())
        assert torch.isfinite(runs[0]).all() and (runs[0] != 0).any()
        assert torch.equal(runs[0], runs[1])


def test_gemm_part_diagnostic_whole_kernel_matches_the_library():
    """cw_diag_gemm_part with part 0 is the library's ring kernel for the benchmark's shape: bit-equal to
    cw_gemm_ksteps; parts 1 to 3 (no operand loads / no epilogue / no LDS reads in the k loop) run and return."""
    import ctypes
    from cubework_amd import _diag, ops

    lib = _diag.load()
    M, N, K = 8192, 2048, 512   # 256 tiles: the shape class the library gives to this kernel
    A = [randn((M, K), torch.bfloat16, 40 + i).to(DEV) for i in range(2)]
    B = [randn((K, N), torch.bfloat16, 50 + i, 0.05).to(DEV) for i in range(2)]
    bias = randn((N,), torch.bfloat16, 60, 0.1).to(DEV)
    want = ops.gemm_ksteps("NN", A, B, bias, "gelu_tanh")
    ta = (ctypes.c_void_p * 2)(*[t.data_ptr() for t in A])
    tb = (ctypes.c_void_p * 2)(*[t.data_ptr() for t in B])
    out = torch.empty_like(want)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.cw_diag_gemm_part(0, M, N, K, 2, ta, K, tb, N, bias.data_ptr(), out.data_ptr(), N, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    for part in (1, 2, 3):
        assert lib.cw_diag_gemm_part(part, M, N, K, 2, ta, K, tb, N, bias.data_ptr(), out.data_ptr(), N, stream) == 0
    torch.cuda.synchronize()
