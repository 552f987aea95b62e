"""GPU parity of the LayerNorm entry points (through the C ABI) against the
CPU oracle: 2D flavour (one-pass statistics, peers' partial sums added
between the kernels) and 3D flavour (two-pass), forward and backward.
"""
import pytest
import torch

from tests.util import assert_parity, rand_uniform, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
SHAPES = [(64, 1024), (33, 520), (16, 100), (5, 7), (300, 2048), (9, 4096), (3, 8200), (7, 512), (1, 256), (2050, 264),
          (1500, 3072), (5, 16384), (2, 16392)]


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

    # forward: local partials -> (+ peer) -> normalise
    st_want = oracle.ln2d_partial_stats(x)
    st_got = ops.ln_partial_stats(x.to(DEV))
    assert_parity(st_got, st_want, torch.float32, "partial stats", scale=10)
    stats_global = st_want + oracle.ln2d_partial_stats(x_peer)
    y_want, mr_want = oracle.ln2d_normalize(x, stats_global, H, eps, gamma, beta)
    y_got, mr_got = ops.ln_normalize(x.to(DEV), stats_global.to(DEV), H, eps, gamma.to(DEV), beta.to(DEV))
    assert_parity(mr_got, mr_want, torch.float32, "mean/rstd", scale=10)
    assert_parity(y_got, y_want, dtype, "normalise", scale=4 if dtype == torch.float32 else 1)

    # backward: local partials -> (+ peer) -> dx
    rs_want, dg_want, db_want = oracle.ln2d_backward_partials(dy, x, mr_want, gamma)
    rs_got, dg_got, db_got = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr_want.to(DEV), gamma.to(DEV))
    assert_parity(rs_got, rs_want, torch.float32, "row sums", scale=20)
    assert_parity(dg_got, dg_want, torch.float32, "dgamma", scale=20)
    assert_parity(db_got, db_want, torch.float32, "dbeta", scale=20)
    peer_mr = oracle.ln2d_mean_rstd(stats_global, H, eps)
    rs_global = rs_want + oracle.ln2d_backward_partials(dy_peer, x_peer, peer_mr, gamma_peer)[0]
    dx_want = oracle.ln2d_backward_dx(dy, x, mr_want, rs_global, H, gamma)
    dx_got = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr_want.to(DEV), rs_global.to(DEV), H, gamma.to(DEV))
    assert_parity(dx_got, dx_want, dtype, "dx", scale=4 if dtype == torch.float32 else 1)


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
    xr = x.float().requires_grad_(True)
    gr = gamma.float().requires_grad_(True)
    br = beta.float().requires_grad_(True)
    y_ref = torch.nn.functional.layer_norm(xr, (C,), gr, br, eps)
    y_ref.backward(dy.float())
    code = CW_LN_ONE_PASS if mode == "one_pass" else CW_LN_TWO_PASS
    y, mr = ops.ln_forward_fused(x.to(DEV), eps, gamma.to(DEV), beta.to(DEV), mode=code)
    assert_parity(y, y_ref.detach().to(dtype), dtype, "fused forward", scale=10 if dtype == torch.float32 else 1)
    rs, dg, db = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr, gamma.to(DEV))
    dx = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr, rs, C, gamma.to(DEV))
    s = 10 if dtype == torch.float32 else 1
    assert_parity(dx, xr.grad.to(dtype), dtype, "dx vs autograd", scale=s)
    assert_parity(dg, gr.grad, torch.float32, "dgamma vs autograd", scale=50)
    assert_parity(db, br.grad, torch.float32, "dbeta vs autograd", scale=50)


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
    xr = x.float().requires_grad_(True)
    gr = gamma.float().requires_grad_(True)
    br = beta.float().requires_grad_(True)
    y_ref = torch.nn.functional.layer_norm(xr, (C,), gr if affine else None, br if affine else None, eps)
    y_ref.backward(dy.float())
    g_dev = gamma.to(DEV) if affine else None
    _, mr = ops.ln_forward_fused(x.to(DEV), eps, g_dev, beta.to(DEV) if affine else None)
    dx, dg, db = ops.ln_backward_fused(dy.to(DEV), x.to(DEV), mr, g_dev)
    s = 10 if dtype == torch.float32 else 1
    assert_parity(dx, xr.grad.to(dtype), dtype, "fused dx vs autograd", scale=s)
    if affine:
        assert_parity(dg, gr.grad, torch.float32, "fused dgamma vs autograd", scale=50)
        assert_parity(db, br.grad, torch.float32, "fused dbeta vs autograd", scale=50)
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
    s_local = ops.ln_partial_stats(x.to(DEV), CW_LN_TWO_PASS, None)
    assert_parity(s_local[:, 0].cpu(), x.sum(-1), torch.float32, "sum x", scale=10)
    assert torch.count_nonzero(s_local[:, 1]) == 0
    mean = (x.sum(-1) + x_peer.sum(-1)) / H
    s2 = ops.ln_partial_stats(x.to(DEV), CW_LN_TWO_PASS, mean.to(DEV))
    want_sq = ((x - mean[:, None]) ** 2).sum(-1)
    assert_parity(s2[:, 1].cpu(), want_sq, torch.float32, "centred second moment", scale=10)
    peer_sq = ((x_peer - mean[:, None]) ** 2).sum(-1)
    stats_global = torch.stack([mean, want_sq + peer_sq], dim=-1)
    y, mr = ops.ln_normalize(x.to(DEV), stats_global.to(DEV), H, eps, gamma.to(DEV), beta.to(DEV), mode=CW_LN_TWO_PASS)
    y_want, mu, sigma = oracle.ln3d_forward(x, gamma, beta, H, eps, peer_sum=x_peer.sum(-1), peer_sqdev=peer_sq)
    assert_parity(y, y_want, torch.float32, "3D forward", scale=4)
    assert_parity(mr[:, 1].cpu(), 1.0 / sigma[:, 0], torch.float32, "rstd", scale=10)


def test_ln3d_backward_formula_matches():
    """The dx kernel's closed form equals _Layernorm3D.backward's three-term
    form (parallel_3d/_operation.py:303-311) at tensor-parallel size 1."""
    import oracle
    from cubework_amd import ops
    from cubework_amd._lib import CW_LN_TWO_PASS

    R, C, eps = 24, 768, 1e-12
    x, dy, gamma, beta = _inputs(R, C, torch.float32, 31)
    y_want, mu, sigma = oracle.ln3d_forward(x, gamma, beta, C, eps)
    dx_want, dg_want, db_want = oracle.ln3d_backward(dy, mu, sigma, gamma, C)
    y, mr = ops.ln_forward_fused(x.to(DEV), eps, gamma.to(DEV), beta.to(DEV), mode=CW_LN_TWO_PASS)
    rs, dg, db = ops.ln_bwd_partials(dy.to(DEV), x.to(DEV), mr, gamma.to(DEV))
    dx = ops.ln_bwd_dx(dy.to(DEV), x.to(DEV), mr, rs, C, gamma.to(DEV))
    assert_parity(y, y_want, torch.float32, "3D fwd", scale=4)
    assert_parity(dx, dx_want, torch.float32, "3D dx", scale=10)
    assert_parity(dg, dg_want, torch.float32, "3D dgamma", scale=20)
    assert_parity(db, db_want, torch.float32, "3D dbeta", scale=20)


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
    assert_parity(sa + sb, whole, torch.float32, "split invariance", scale=10)
    stats = sa + sb
    ya, mra = ops.ln_normalize(xa, stats, H, eps)
    yb, mrb = ops.ln_normalize(xb, stats, H, eps)
    assert torch.equal(mra, mrb)
    xh = torch.cat([ya, yb], dim=1).float()
    assert xh.mean(dim=1).abs().max().item() < 5e-3  # bf16 rounding of x_hat
    var = (stats[:, 1] / H - (stats[:, 0] / H) ** 2)
    assert_parity((xh * xh).mean(dim=1), var / (var + eps), torch.float32, "unit variance", scale=1e3)
    rsa = ops.ln_bwd_partials(dya, xa, mra, None, want_param_grads=False)[0]
    rsb = ops.ln_bwd_partials(dyb, xb, mrb, None, want_param_grads=False)[0]
    rs = rsa + rsb
    dxa = ops.ln_bwd_dx(dya, xa, mra, rs, H)
    dxb = ops.ln_bwd_dx(dyb, xb, mrb, rs, H)
    dx = torch.cat([dxa, dxb], dim=1).float()
    scale = dx.abs().sum(dim=1)
    assert (dx.sum(dim=1).abs() / scale).max().item() < 1e-2
    assert ((dx * xh).sum(dim=1).abs() / scale).max().item() < 1e-2


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
    for name, a, b in zip(names, got, want):
        if same_kernels:
            assert torch.equal(a, b), name
        else:  # the looping kernels add in another order than the vector kernels the contiguous copy takes
            assert_parity(a, b, a.dtype, "strided " + name, scale=100 if a.dtype == torch.float32 else 2)
    y_ref = torch.nn.functional.layer_norm(xc.float(), (C,), gamma.float(), beta.float(), 1e-5)
    assert_parity(got[0], y_ref.to(dtype), dtype, "strided forward", scale=10 if dtype == torch.float32 else 1)
