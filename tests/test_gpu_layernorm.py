"""GPU parity of the LayerNorm entry points (through the C ABI) against the
CPU oracle: 2D flavour (one-pass statistics, peers' partial sums added
between the kernels) and 3D flavour (two-pass), forward and backward.

Expected values are the oracle's formulas evaluated in float64 (oracle.precision), so they carry no
rounding of their own. Bars: 1e-2 for bf16 results, 1e-3 for float16, 1e-5 for every fp32 result, sums over
up to 16392 columns or 2100 rows included (achieved: at most 3e-7; tests/conftest.py prints the largest).
"""
import pytest
import torch

from tests.util import assert_parity, rand_uniform, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
SHAPES = [(64, 1024), (33, 520), (16, 100), (5, 7), (300, 2048), (9, 4096), (3, 8200), (7, 512), (1, 256), (2050, 264),
          (1500, 3072), (5, 16384), (2, 16392)]


def _rounded(t, dtype):
    """A float64 expected value as the kernel's output type would hold it: rounded once for the 16-bit
    types, unchanged for fp32 (whose bar then covers the kernel's own rounding)."""
    return t.to(dtype) if dtype in (torch.bfloat16, torch.float16) else t


def _inputs(R, C, dtype, seed):
    x = randn((R, C), dtype, seed)
    dy = randn((R, C), dtype, seed + 1)
    gamma = rand_uniform((C,), dtype, seed + 2, 0.9, 1.1)
    beta = randn((C,), dtype, seed + 3, std=0.02)
    return x, dy, gamma, beta


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
def test_ln2d_forward_backward_with_peer_partials(shape, dtype):
    """One rank of a q=2 row group: the peer's partial sums are pre-staged."""
    import oracle
    from cubework_amd import ops

    R, C = shape
    H = 2 * C
    eps = 1e-5
    x, dy, gamma, beta = _inputs(R, C, dtype, 0)
    x_peer, dy_peer, gamma_peer, _ = _inputs(R, C, dtype, 50)

    with oracle.precision(torch.float64):
        # forward: local partials -> (+ peer) -> normalise
        st_want = oracle.ln2d_partial_stats(x)
        st_got = ops.ln_partial_stats(x.to(DEV))
        assert_parity(st_got, st_want, torch.float32, "partial stats")
        stats_global = (st_want + oracle.ln2d_partial_stats(x_peer)).float()  # what the all-reduce hands back
        y_want, mr_want = oracle.ln2d_normalize(x, stats_global, H, eps, gamma, beta)
        y_got, mr_got = ops.ln_normalize(x.to(DEV), stats_global.to(DEV), H, eps, gamma.to(DEV), beta.to(DEV))
        assert_parity(mr_got, mr_want, torch.float32, "mean/rstd")
        assert_parity(y_got, y_want, dtype, "normalise")

        # backward: local partials -> (+ peer) -> dx
        mr32 = mr_want.float()
        rs_want, dg_want, db_want = oracle.ln2d_backward_partials(dy, x, mr32, gamma)
        rs_got, dg_got, db_got = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr32.to(DEV), gamma.to(DEV))
        assert_parity(rs_got, rs_want, torch.float32, "row sums")
        assert_parity(dg_got, dg_want, torch.float32, "dgamma")
        assert_parity(db_got, db_want, torch.float32, "dbeta")
        peer_mr = oracle.ln2d_mean_rstd(stats_global, H, eps)
        rs_global = (rs_want + oracle.ln2d_backward_partials(dy_peer, x_peer, peer_mr, gamma_peer)[0]).float()
        dx_want = oracle.ln2d_backward_dx(dy, x, mr32, rs_global, H, gamma)
        dx_got = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr32.to(DEV), rs_global.to(DEV), H, gamma.to(DEV))
        assert_parity(dx_got, dx_want, dtype, "dx")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("mode", ["one_pass", "two_pass"])
@pytest.mark.parametrize("shape", [(64, 1024), (17, 200), (4, 2048), (33, 4096), (70, 8192), (9, 12288), (2100, 2560),
                                   (1100, 5120), (3, 16384), (2, 20480)])
def test_ln_fused_matches_nn_layernorm(shape, mode, dtype):
    """tensor-parallel size 1: against F.layer_norm and its autograd, the
    oracle the reference's 3D test uses (tests/test_3d/check_3d_modules.py:132)."""
    from cubework_amd import ops
    from cubework_amd._lib import CW_LN_ONE_PASS, CW_LN_TWO_PASS

    R, C = shape
    eps = 1e-5
    x, dy, gamma, beta = _inputs(R, C, dtype, 7)
    xr = x.double().requires_grad_(True)
    gr = gamma.double().requires_grad_(True)
    br = beta.double().requires_grad_(True)
    y_ref = torch.nn.functional.layer_norm(xr, (C,), gr, br, eps)
    y_ref.backward(dy.double())
    code = CW_LN_ONE_PASS if mode == "one_pass" else CW_LN_TWO_PASS
    y, mr = ops.ln_forward_fused(x.to(DEV), eps, gamma.to(DEV), beta.to(DEV), mode=code)
    assert_parity(y, _rounded(y_ref.detach(), dtype), dtype, "fused forward %s" % mode)
    rs, dg, db = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr, gamma.to(DEV))
    dx = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr, rs, C, gamma.to(DEV))
    assert_parity(dx, _rounded(xr.grad, dtype), dtype, "dx vs autograd")
    assert_parity(dg, gr.grad, torch.float32, "dgamma vs autograd")
    assert_parity(db, br.grad, torch.float32, "dbeta vs autograd")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("shape", [(64, 1024), (17, 200), (4, 2048), (1000, 512), (33, 4096), (5, 1001), (3, 5000), (300, 64),
                                   (70, 8192), (9, 12288), (600, 3072), (2100, 2560), (3, 16384), (2, 20480),
                                   (600, 10240)])
def test_ln_backward_fused_matches_autograd(shape, affine, dtype):
    """Rows complete on this rank: one pass gives dx, dgamma, dbeta. Against F.layer_norm's autograd, and
    bit-identical to the two-kernel path (partials, then dx with H = C) that it replaces. Shapes cover
    every chunk count of the one-pass kernel, the kernel that splits wide rows over wavefronts (blocks of one
    to four row groups, several trips, rows past the end), ragged widths and the generic fallback."""
    from cubework_amd import ops

    R, C = shape
    eps = 1e-5
    x, dy, gamma, beta = _inputs(R, C, dtype, 11)
    xr = x.double().requires_grad_(True)
    gr = gamma.double().requires_grad_(True)
    br = beta.double().requires_grad_(True)
    y_ref = torch.nn.functional.layer_norm(xr, (C,), gr if affine else None, br if affine else None, eps)
    y_ref.backward(dy.double())
    g_dev = gamma.to(DEV) if affine else None
    _, mr = ops.ln_forward_fused(x.to(DEV), eps, g_dev, beta.to(DEV) if affine else None)
    dx, dg, db = ops.ln_backward_fused(dy.to(DEV), x.to(DEV), mr, g_dev)
    assert_parity(dx, _rounded(xr.grad, dtype), dtype, "fused dx vs autograd")
    if affine:
        assert_parity(dg, gr.grad, torch.float32, "fused dgamma vs autograd")
        assert_parity(db, br.grad, torch.float32, "fused dbeta vs autograd")
    rs, dg2, db2 = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr, g_dev)
    dx2 = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr, rs, C, g_dev)
    assert torch.equal(dx, dx2)
    assert torch.equal(dg, dg2) and torch.equal(db, db2)


@pytest.mark.parametrize("shape", [(40, 512), (700, 3072), (3, 9216), (5, 20480)])
def test_ln3d_two_pass_with_peer(shape):
    """3D flavour on one rank of a depth-2 output group: mean exchange, then
    the centred second moment (parallel_3d/_operation.py:273-276). The wide shapes take the statistics
    kernel that splits a row over wavefronts (several trips; one 16-wavefront group) and the looping one."""
    import oracle
    from cubework_amd import ops
    from cubework_amd._lib import CW_LN_TWO_PASS

    R, C = shape
    H, eps = 2 * C, 1e-12
    x, dy, gamma, beta = _inputs(R, C, torch.float32, 21)
    x_peer = randn((R, C), torch.float32, 99)
    xd, xpd = x.double(), x_peer.double()
    s_local = ops.ln_partial_stats(x.to(DEV), CW_LN_TWO_PASS, None)
    assert_parity(s_local[:, 0].cpu(), xd.sum(-1), torch.float32, "sum x")
    assert torch.count_nonzero(s_local[:, 1]) == 0
    mean = ((xd.sum(-1) + xpd.sum(-1)) / H).float()  # what the first exchange hands back
    s2 = ops.ln_partial_stats(x.to(DEV), CW_LN_TWO_PASS, mean.to(DEV))
    want_sq = ((xd - mean.double()[:, None]) ** 2).sum(-1)
    assert_parity(s2[:, 1].cpu(), want_sq, torch.float32, "centred second moment")
    peer_sq = ((xpd - mean.double()[:, None]) ** 2).sum(-1)
    stats_global = torch.stack([mean, (want_sq + peer_sq).float()], dim=-1)
    y, mr = ops.ln_normalize(x.to(DEV), stats_global.to(DEV), H, eps, gamma.to(DEV), beta.to(DEV), mode=CW_LN_TWO_PASS)
    with oracle.precision(torch.float64):
        # the oracle forms the mean and the centred sum itself; hand it the peers' parts that give the same global statistics
        y_want, mu, sigma = oracle.ln3d_forward(x, gamma, beta, H, eps, peer_sum=mean.double() * H - xd.sum(-1),
                                                peer_sqdev=stats_global[:, 1].double() - want_sq)
    assert_parity(y, y_want, torch.float32, "3D forward")
    assert_parity(mr[:, 1].cpu(), 1.0 / sigma[:, 0], torch.float32, "rstd")


def test_ln3d_backward_formula_matches():
    """The dx kernel's closed form equals _Layernorm3D.backward's three-term
    form (parallel_3d/_operation.py:303-311) at tensor-parallel size 1."""
    import oracle
    from cubework_amd import ops
    from cubework_amd._lib import CW_LN_TWO_PASS

    R, C, eps = 24, 768, 1e-12
    x, dy, gamma, beta = _inputs(R, C, torch.float32, 31)
    with oracle.precision(torch.float64):
        y_want, mu, sigma = oracle.ln3d_forward(x, gamma, beta, C, eps)
        dx_want, dg_want, db_want = oracle.ln3d_backward(dy, mu, sigma, gamma, C)
    y, mr = ops.ln_forward_fused(x.to(DEV), eps, gamma.to(DEV), beta.to(DEV), mode=CW_LN_TWO_PASS)
    rs, dg, db = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr, gamma.to(DEV))
    dx = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr, rs, C, gamma.to(DEV))
    assert_parity(y, y_want, torch.float32, "3D fwd")
    assert_parity(dx, dx_want, torch.float32, "3D dx")
    assert_parity(dg, dg_want, torch.float32, "3D dgamma")
    assert_parity(db, db_want, torch.float32, "3D dbeta")


def test_ln_baseline_shape_properties():
    """The benchmark's LayerNorm2D workload (16384 x 1024 bf16, H = 2048) at full size, through size-independent properties:
    per-row mean(x_hat) = 0, mean(x_hat^2) = var/(var+eps) over the whole H,
    sum_c dx = 0 and sum_c dx*x_hat = 0 over the whole H, split invariance."""
    from cubework_amd import ops

    R, C, H, eps = 16384, 1024, 2048, 1e-5
    xa = randn((R, C), torch.bfloat16, 0, device=DEV)
    xb = randn((R, C), torch.bfloat16, 1, device=DEV)
    dya = randn((R, C), torch.bfloat16, 2, device=DEV)
    dyb = randn((R, C), torch.bfloat16, 3, device=DEV)
    sa, sb = ops.ln_partial_stats(xa), ops.ln_partial_stats(xb)
    # split invariance: partials of the halves add up to the stats of the whole
    whole = ops.ln_partial_stats(torch.cat([xa, xb], dim=1))
    assert_parity(sa + sb, whole, torch.float32, "split invariance")
    stats = sa + sb
    ya, mra = ops.ln_normalize(xa, stats, H, eps)
    yb, mrb = ops.ln_normalize(xb, stats, H, eps)
    assert torch.equal(mra, mrb)
    xh = torch.cat([ya, yb], dim=1).float()
    assert xh.mean(dim=1).abs().max().item() < 5e-3  # bf16 rounding of x_hat
    var = (stats[:, 1] / H - (stats[:, 0] / H) ** 2)
    # x_hat was rounded to bf16. The inputs are bf16 values and x_hat = (x - mean) * rstd lies within half a bf16
    # step of x itself whenever |1 - rstd| < 2^-9, so the rounding snaps a whole row back to x: a coherent error of
    # up to 2 |1 - rstd| in the mean square, not an average of independent roundings. The bf16 bar applies.
    assert_parity((xh * xh).mean(dim=1), var / (var + eps), torch.bfloat16, "unit variance")
    rsa = ops.ln_bwd_partials(dya, xa, mra, None, want_param_grads=False)[0]
    rsb = ops.ln_bwd_partials(dyb, xb, mrb, None, want_param_grads=False)[0]
    rs = rsa + rsb
    dxa = ops.ln_bwd_dx(dya, xa, mra, rs, H)
    dxb = ops.ln_bwd_dx(dyb, xb, mrb, rs, H)
    dx = torch.cat([dxa, dxb], dim=1).float()
    scale = dx.abs().sum(dim=1)
    assert (dx.sum(dim=1).abs() / scale).max().item() < 1e-2
    assert ((dx * xh).sum(dim=1).abs() / scale).max().item() < 1e-2


def test_ln_baseline_shape_sampled_rows_against_the_float64_oracle():
    """The benchmark's LayerNorm2D shard at exactly its size (16384 x 1024 bf16 of H = 2048, gamma ~ U(0.9, 1.1),
    beta ~ N(0, 0.02), peer statistics from a second seeded half): 64 sampled rows of cw_ln_normalize's output and
    saved (mean, rstd) and of cw_ln_bwd_dx_close's dx against the oracle's formulas in float64, evaluated from the
    same inputs the kernels were given (the global statistics / row sums the GPU run produced, as a rank receives
    them after the all-reduce); dgamma / dbeta of the open/close pair in full (16384 rows reduced)."""
    import oracle
    from cubework_amd import ops

    R, C, H, eps = 16384, 1024, 2048, 1e-5
    x, dy, gamma, beta = _inputs(R, C, torch.bfloat16, 0)
    peer = randn((R, C), torch.bfloat16, 7)
    xd, dyd, gd, bd, pd = (t.to(DEV) for t in (x, dy, gamma, beta, peer))
    stats = ops.ln_partial_stats(xd) + ops.ln_partial_stats(pd)
    y, mr = ops.ln_normalize(xd, stats, H, eps, gd, bd)
    rs_local, pending = ops.ln_bwd_partials_open(dyd, xd, mr, gd)
    rs = rs_local * 1.75          # stands in for the all-reduced row sums: any values exercise the dx formula
    dx, dgamma, dbeta = ops.ln_bwd_dx_close(dyd, xd, mr, rs, H, pending, gd)
    g = torch.Generator().manual_seed(3)
    rows = torch.cat([torch.tensor([0, 1, 63, 64, R - 1]), torch.randint(0, R, (59,), generator=g)])
    with oracle.precision(torch.float64):
        st = stats.cpu()[rows]
        want_y, want_mr = oracle.ln2d_normalize(x[rows], st, H, eps, gamma, beta)
        assert_parity(mr.cpu()[rows], want_mr, torch.float32, "mean / rstd, 64 rows of 16384 x 1024")
        assert_parity(y.cpu()[rows], _rounded(want_y, torch.bfloat16), torch.bfloat16, "ln_normalize, 64 rows of 16384 x 1024")
        want_rs, want_dg, want_db = oracle.ln2d_backward_partials(dy, x, mr.cpu(), gamma)
        assert_parity(rs_local, want_rs, torch.float32, "row sums (all 16384 rows)")
        assert_parity(dgamma, want_dg, torch.float32, "dgamma (16384 rows reduced)")
        assert_parity(dbeta, want_db, torch.float32, "dbeta (16384 rows reduced)")
        want_dx = oracle.ln2d_backward_dx(dy[rows], x[rows], mr.cpu()[rows], rs.cpu()[rows], H, gamma)
        assert_parity(dx.cpu()[rows], _rounded(want_dx, torch.bfloat16), torch.bfloat16, "ln_bwd_dx_close, 64 rows of 16384 x 1024")


def test_ln_empty_and_errors():
    from cubework_amd import ops, _lib

    x = torch.zeros((0, 64), dtype=torch.bfloat16, device=DEV)
    assert ops.ln_partial_stats(x).shape == (0, 2)
    lib = _lib.load()
    rc = lib.cw_ln_normalize(4, 8, None, 8, None, 0, 4, 1e-5, None, None, None, 8, None, 0, None)
    assert rc < 0 and b"hidden size" in lib.cw_last_error()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("case", [(50, 1024, 0, 3072), (600, 2560, 512, 4096), (40, 4096, 4096, 12288),
                                  (9, 9216, 8, 9232), (33, 3072, 3, 3080)])
def test_ln_strided_rows(case, dtype):
    """Inputs that are column slices of a wider buffer (row stride larger than the row, as the q/k/v
    slices of a fused projection are): bit-identical to the same call on contiguous copies for the
    whole-row tiles and the kernels that split a row over wavefronts; the last case, a slice that starts
    off a 16-byte boundary, takes the looping kernels and is compared within the tolerance."""
    from cubework_amd import ops

    R, C, off, W = case
    wide_x = randn((R, W), dtype, 41).to(DEV)
    wide_dy = randn((R, W), dtype, 42).to(DEV)
    gamma = rand_uniform((C,), dtype, 43, 0.9, 1.1).to(DEV)
    beta = randn((C,), dtype, 44, std=0.02).to(DEV)
    xs, dys = wide_x[:, off:off + C], wide_dy[:, off:off + C]
    xc, dyc = xs.contiguous(), dys.contiguous()
    assert xs.stride(0) == W and not xs.is_contiguous()
    got, want = [], []
    for x, dy, out in ((xs, dys, got), (xc, dyc, want)):
        y, mr = ops.ln_forward_fused(x, 1e-5, gamma, beta)
        dx, dg, db = ops.ln_backward_fused(dy, x, mr, gamma)
        stats = ops.ln_partial_stats(x)
        y2, mr2 = ops.ln_normalize(x, stats, C, 1e-5, gamma, beta)
        rs, dg2, db2 = ops.ln_bwd_partials(dy, x, mr, gamma)
        dx2 = ops.ln_bwd_dx(dy, x, mr, rs, C, gamma)
        out.extend([y, mr, dx, dg, db, stats, y2, mr2, rs, dg2, db2, dx2])
    same_kernels = (off * xs.element_size()) % 16 == 0 and (W * xs.element_size()) % 16 == 0
    names = ["y", "mean_rstd", "dx", "dgamma", "dbeta", "stats", "y2", "mean_rstd2", "row_sums", "dgamma2", "dbeta2", "dx2"]
    if same_kernels:
        for name, a, b in zip(names, got, want):
            assert torch.equal(a, b), name
    # against float64 (the looping kernels of the unaligned case add in another order than the vector kernels,
    # so there the strided results are checked against the exact values, not against the contiguous call)
    import oracle
    with oracle.precision(torch.float64):
        y_w, mr_w = oracle.ln_forward_full(xc, gamma, beta, 1e-5)
        dx_w, dg_w, db_w = oracle.ln_backward_full(dyc, xc, got[1].cpu(), gamma)
        st_w = oracle.ln2d_partial_stats(xc)
        rs_w = oracle.ln2d_backward_partials(dyc, xc, got[1].cpu(), gamma)[0]
    f32 = torch.float32
    exp = [(y_w, dtype), (mr_w, f32), (dx_w, dtype), (dg_w, f32), (db_w, f32), (st_w, f32), (y_w, dtype), (mr_w, f32),
           (rs_w, f32), (dg_w, f32), (db_w, f32), (dx_w, dtype)]
    for name, a, (w, dt) in zip(names, got, exp):
        assert_parity(a, w.reshape(a.shape), dt, "strided " + name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(16384, 1024), (8192, 2048), (4096, 4096), (300, 1000), (5, 24), (1, 8), (2048, 8200),
                                   (777, 520)])
def test_backward_with_the_column_finalize_in_the_dx_launch(dtype, shape):
    """cw_ln_bwd_partials_open + cw_ln_bwd_dx_close against cw_ln_bwd_partials + cw_ln_bwd_dx on every kernel
    family (whole-row tiles, exact tiles, rows split over wavefronts, looping kernels, ragged rows): row sums
    and dx to the bit (the same kernels compute them), the column sums to fp32 rounding of a sum over the
    partial rows (they are added in another fixed order) and against float64; twice in a row to the bit."""
    import oracle
    from cubework_amd import ops

    R, C = shape
    x = randn((R, C), dtype, 61).to(DEV)
    dy = randn((R, C), dtype, 62).to(DEV)
    gamma = rand_uniform((C,), dtype, 63, 0.9, 1.1).to(DEV)
    _, mr = ops.ln_forward_fused(x, 1e-5, gamma, torch.zeros_like(gamma))
    rs, dg, db = ops.ln_bwd_partials(dy, x, mr, gamma)
    dx = ops.ln_bwd_dx(dy, x, mr, rs, C, gamma)
    rs2, pending = ops.ln_bwd_partials_open(dy, x, mr, gamma)
    dx2, dg2, db2 = ops.ln_bwd_dx_close(dy, x, mr, rs2, C, pending, gamma)
    rs3, pending3 = ops.ln_bwd_partials_open(dy, x, mr, gamma)
    dx3, dg3, db3 = ops.ln_bwd_dx_close(dy, x, mr, rs3, C, pending3, gamma)
    torch.cuda.synchronize()
    assert torch.equal(rs, rs2) and torch.equal(dx, dx2)
    assert torch.equal(dg2, dg3) and torch.equal(db2, db3) and torch.equal(dx2, dx3)
    with oracle.precision(torch.float64):
        _, dg_w, db_w = oracle.ln_backward_full(dy.cpu(), x.cpu(), mr.cpu(), gamma.cpu())
    assert_parity(dg2, dg_w, torch.float32, "dgamma from the dx launch")
    assert_parity(db2, db_w, torch.float32, "dbeta from the dx launch")
    assert_parity(dg2, dg.double().cpu(), torch.float32, "dgamma against the two-launch path")
    assert_parity(db2, db.double().cpu(), torch.float32, "dbeta against the two-launch path")


def test_dx_close_argument_checks_and_no_rows():
    import ctypes as C
    from cubework_amd import _lib

    lib = _lib.load()
    n = C.c_int64(-1)
    out = torch.full((2, 8), float("nan"), dtype=torch.float32, device=DEV)
    assert lib.cw_ln_bwd_partials_open(4, 8, None, 8, None, 8, None, None, None, None, 0, None, 0, None) == -1     # n_parts NULL
    assert lib.cw_ln_bwd_partials_open(4, 8, None, 8, None, 8, None, None, None, None, 0, C.cast(C.byref(n), C.c_void_p), 0, None) == -1
    assert n.value == 0
    assert lib.cw_ln_bwd_dx_close(4, 8, None, 8, None, 8, None, None, None, 8, None, 8, None, 0, None, None, 1, 0, None) == -1   # no dgamma
    assert lib.cw_ln_bwd_dx_close(4, 8, None, 8, None, 8, None, None, None, 8, None, 8, None, 3, out[0].data_ptr(),
                                  out[1].data_ptr(), 1, 0, None) == -1                                                        # partials without workspace
    assert lib.cw_ln_bwd_dx_close(4, 8, None, 8, None, 8, None, None, None, 4, None, 8, None, 0, out[0].data_ptr(),
                                  out[1].data_ptr(), 1, 0, None) == -1                                                        # H < C
    # no rows: zero column sums, nothing else touched
    assert lib.cw_ln_bwd_dx_close(0, 8, None, 8, None, 8, None, None, None, 8, None, 8, None, 0, out[0].data_ptr(),
                                  out[1].data_ptr(), 1, 0, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, torch.zeros_like(out))


def test_partial_stats_into_a_result_buffer_that_is_only_8_byte_aligned():
    """The one-tile-per-wavefront statistics kernel writes two rows' results as one 16-byte piece when the
    result buffer allows it; a buffer that is 8-byte but not 16-byte aligned takes per-row stores. Same bits."""
    import ctypes
    from cubework_amd import _lib, ops

    lib = _lib.load()
    for R, C in ((64, 1024), (37, 512), (1001, 2048)):
        x = randn((R, C), torch.bfloat16, R).to(DEV)
        want = ops.ln_partial_stats(x)
        buf = torch.full((2 * R + 2,), float("nan"), dtype=torch.float32, device=DEV)
        view = buf[2:]
        assert view.data_ptr() % 16 == 8
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        _lib.check(lib.cw_ln_partial_stats(R, C, x.data_ptr(), C, _lib.CW_LN_ONE_PASS, None, view.data_ptr(), _lib.CW_BF16, stream),
                   "cw_ln_partial_stats")
        torch.cuda.synchronize()
        assert torch.equal(view.view(R, 2), want)
        assert torch.isnan(buf[:2]).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(64, 1024), (300, 2048), (33, 4096), (17, 200), (5, 1001), (70, 8192), (9, 12288)])
def test_ln_backward_fused_with_the_residual_branch_gradient(shape, dtype):
    """cw_ln_backward_fused with dx_addend: dx = LayerNorm backward + the gradient arriving along the residual
    branch, rounded once (expected: the oracle's dx in float64 plus the addend); dgamma / dbeta / row sums are
    the same bits as without it. Shapes cover the whole-row kernel, the split kernel for wide rows, and the
    two-kernel path (ragged / unaligned rows), where the wrapper adds separately."""
    import oracle
    from cubework_amd import ops

    R, C = shape
    x, dy, gamma, _ = _inputs(R, C, dtype, 11)
    add = randn((R, C), dtype, 15)
    xd, dyd, gd, ad = (t.to(DEV) for t in (x, dy, gamma, add))
    _, mr = ops.ln_forward_fused(xd, 1e-5, gd, None)
    dx0, dg0, db0 = ops.ln_backward_fused(dyd, xd, mr, gd)
    dx1, dg1, db1 = ops.ln_backward_fused(dyd, xd, mr, gd, dx_addend=ad)
    assert torch.equal(dg0, dg1) and torch.equal(db0, db1)
    with oracle.precision(torch.float64):
        want, _, _ = oracle.ln_backward_full(dy, x, mr.cpu(), gamma)
        want = want.double() + add.double()
    assert_parity(dx1, _rounded(want, dtype), dtype, "fused backward + residual gradient %s" % (shape,))


def test_layernorm2d_fork_residual_option():
    """LayerNorm2D(x, fork_residual=True) returns (LN(x), x): a block y = x + f(LN(x)) built on it has the same
    output and the same gradients as the plain composition, the sum of the two branches' gradients being formed
    in the layer's backward kernel."""
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_2d import LayerNorm2D

    initialize("2d", 1)
    norm = LayerNorm2D(1024).to(torch.bfloat16).to(DEV)
    with torch.no_grad():
        norm.weight.copy_(rand_uniform((1024,), torch.bfloat16, 1, 0.9, 1.1))
        norm.bias.copy_(randn((1024,), torch.bfloat16, 2, 0.02))
    w = randn((1024, 1024), torch.bfloat16, 3, 0.03).to(DEV)
    dy = randn((6, 50, 1024), torch.bfloat16, 4).to(DEV)
    outs = []
    for fork in (False, True):
        x = randn((6, 50, 1024), torch.bfloat16, 5).to(DEV).requires_grad_(True)
        norm.zero_grad(set_to_none=True)
        if fork:
            h, res = norm(x, fork_residual=True)
        else:
            h, res = norm(x), x
        y = res + torch.tanh(h @ w)
        y.backward(dy)
        outs.append((y.detach(), x.grad, norm.weight.grad.clone(), norm.bias.grad.clone()))
    assert torch.equal(outs[0][0], outs[1][0])
    assert torch.equal(outs[0][2], outs[1][2]) and torch.equal(outs[0][3], outs[1][3])
    # one rounding instead of two: equal up to a bf16 step
    assert_parity(outs[1][1], outs[0][1].double(), torch.bfloat16, "x.grad with the branches summed in the kernel")
