"""The CPU oracle against the routines the reference's own tests use as their
oracle (plain single-device torch on the master tensors) and against
invariants of the mathematics. Runs without a GPU."""
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import grid
from tests.util import randn


def close(a, b, tol=1e-5):
    a, b = a.double(), b.double()
    assert a.shape == b.shape
    assert (a - b).abs().max().item() <= tol * max(b.abs().max().item(), 1.0)


@pytest.mark.parametrize("q", [1, 2, 3])
def test_grid_linear2d_composes_to_master(q):
    """tests/test_2d/check_2d_modules.py:31-110 without processes: every rank's
    forward output and gradients are the master's shards."""
    B, S, IN, OUT = 2 * q, 3, 4 * q * q, 2 * q * q
    A = randn((B, S, IN), torch.float32, 0)
    W = randn((IN, OUT), torch.float32, 1)
    b = randn((OUT,), torch.float32, 2)
    dC = randn((B, S, OUT), torch.float32, 3)
    A2, dC2 = A.reshape(-1, IN), dC.reshape(-1, OUT)
    C = A2 @ W + b
    out = grid.linear2d_forward(A, W, b, q)
    dA, dW, db = grid.linear2d_backward(A, W, dC, q)
    for i in range(q):
        for j in range(q):
            close(out[(i, j)], grid.shard(C, q, i, j))
            close(dA[(i, j)], grid.shard(dC2 @ W.t(), q, i, j))
            close(dW[(i, j)], grid.shard(A2.t() @ dC2, q, i, j))
            close(db[(i, j)], grid.bias_shard(dC2.sum(0), q, i, j))


def test_kstep_sum_equals_concatenated_gemm():
    A = [randn((7, 5), torch.float32, s) for s in range(3)]
    B = [randn((5, 6), torch.float32, 10 + s) for s in range(3)]
    close(oracle.gemm_ksteps("NN", A, B), torch.cat(A, 1) @ torch.cat(B, 0))
    close(oracle.gemm_ksteps("NT", A, [b.t().contiguous() for b in B]), torch.cat(A, 1) @ torch.cat(B, 0))
    close(oracle.gemm_ksteps("TN", [a.t().contiguous() for a in A], B), torch.cat(A, 1) @ torch.cat(B, 0))


def test_linear1d_col_and_row_formulas():
    """tests/test_1d/check_1d_modules.py:74,144: A @ W^T + b."""
    x, W, b = randn((6, 8), torch.float32, 0), randn((10, 8), torch.float32, 1), randn((10,), torch.float32, 2)
    close(oracle.gemm_ksteps("NT", [x], [W], b), F.linear(x, W, b))


def test_bf16_oracle_rounds_once():
    A = [randn((16, 32), torch.bfloat16, s) for s in range(2)]
    B = [randn((32, 8), torch.bfloat16, 5 + s) for s in range(2)]
    want = sum(a.float() @ b.float() for a, b in zip(A, B)).to(torch.bfloat16)
    assert torch.equal(oracle.gemm_ksteps("NN", A, B), want)
    # the reference's eager bf16 path rounds after every step: allowed to differ by bf16 rounding only
    eager = oracle.summa_ab_reference_dtype(A, B)
    close(eager.float(), want.float(), 2e-2)


@pytest.mark.parametrize("q", [1, 2])
def test_grid_layernorm2d_matches_reference_test_formula(q):
    """tests/test_2d/check_2d_modules.py:137-143 (no affine) and nn.LayerNorm
    with affine (tests/test_3d/check_3d_modules.py:132)."""
    R, H, eps = 4 * q, 8 * q, 1e-5
    A = randn((R, H), torch.float32, 0)
    dY = randn((R, H), torch.float32, 1)
    Ar = A.clone().requires_grad_(True)
    E = Ar.sum(-1, keepdim=True) / H
    V = (Ar * Ar).sum(-1, keepdim=True) / H - E * E
    C = (Ar - E) * (1.0 / torch.sqrt(V + eps))
    C.backward(dY)
    fwd = grid.layernorm2d_forward(A, q, eps)
    dx = grid.layernorm2d_backward(A, dY, q, eps)
    for i in range(q):
        for j in range(q):
            close(fwd[(i, j)][0], grid.shard(C.detach(), q, i, j))
            close(dx[(i, j)], grid.shard(Ar.grad, q, i, j), 1e-4)
    gamma, beta = torch.rand(H) + 0.5, randn((H,), torch.float32, 2)
    fwd = grid.layernorm2d_forward(A, q, eps, gamma, beta)
    ref = F.layer_norm(A, (H,), gamma, beta, eps)
    for i in range(q):
        for j in range(q):
            close(fwd[(i, j)][0], grid.shard(ref, q, i, j))


def test_layernorm_invariants():
    R, H, eps = 5, 64, 1e-5
    x, dy = randn((R, H), torch.float32, 0), randn((R, H), torch.float32, 1)
    y, mr = oracle.ln_forward_full(x, None, None, eps)
    assert y.mean(-1).abs().max() < 1e-6
    var = x.var(-1, unbiased=False)
    close((y * y).mean(-1), var / (var + eps))
    dx, _, _ = oracle.ln_backward_full(dy, x, mr, None)
    assert dx.sum(-1).abs().max() < 1e-5
    # sum_c dx*x_hat = rstd * sum(g*x_hat) * eps/(var+eps): zero up to the eps term
    want = mr[:, 1] * (dy * y).sum(-1) * eps / (var + eps)
    close((dx * y).sum(-1), want, 1e-4)
    # split invariance of the partial statistics
    close(oracle.ln2d_partial_stats(x[:, :20]) + oracle.ln2d_partial_stats(x[:, 20:]), oracle.ln2d_partial_stats(x))


def test_layernorm3d_matches_nn_layernorm_and_2d_closed_form():
    R, H, eps = 6, 48, 1e-12
    x = randn((R, H), torch.float32, 0).requires_grad_(True)
    g, b = (torch.rand(H) + 0.5).requires_grad_(True), randn((H,), torch.float32, 1).requires_grad_(True)
    dy = randn((R, H), torch.float32, 2)
    ref = F.layer_norm(x, (H,), g, b, eps)
    ref.backward(dy)
    y, mu, sigma = oracle.ln3d_forward(x, g, b, H, eps)
    dx, dg, db = oracle.ln3d_backward(dy, mu, sigma, g, H)
    close(y, ref.detach())
    close(dx, x.grad, 1e-4)
    close(dg, g.grad, 1e-4)
    close(db, b.grad)
    # the three-term 3D backward equals the 2D closed form
    _, mr = oracle.ln_forward_full(x, g, b, eps, two_pass=True)
    dx2, dg2, db2 = oracle.ln_backward_full(dy, x, mr, g)
    close(dx2, dx, 1e-4)
    close(dg2, dg, 1e-4)


@pytest.mark.parametrize("p", [1, 2, 4])
def test_vocab_parallel_ce_matches_cross_entropy(p):
    """tests/test_1d/check_1d_modules.py:499-523 with [tokens, vocab] logits."""
    T, V = 12, 8 * p
    logits = randn((T, V), torch.float32, 0, std=2.0)
    t = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(1))
    lr = logits.clone().requires_grad_(True)
    ref = F.cross_entropy(lr, t, reduction="none")
    dl = torch.linspace(0.5, 2.0, T)
    ref.backward(dl)
    loss, grads = grid.vocab_parallel_ce(logits, t, p, dl)
    close(loss, ref.detach())
    close(torch.cat(grads, 1), lr.grad)
    close(loss, torch.logsumexp(logits, -1) - logits[torch.arange(T), t])
    assert torch.cat(grads, 1).sum(-1).abs().max() < 1e-5  # rows of d(loss)/d(logits) sum to zero


def test_vocab_parallel_ce_edge_targets_and_masked_rows():
    V, p = 5, 3
    logits = randn((6, V * p), torch.float32, 3)
    t = torch.tensor([0, V - 1, V, 2 * V - 1, 2 * V, V * p - 1])
    for r, s in enumerate(torch.chunk(logits, p, -1)):
        m, se, pred, mask = oracle.vpce_fwd_local(s, t, r * V)
        want_mask = [0 if r * V <= int(x) < (r + 1) * V else 1 for x in t]
        assert mask.tolist() == want_mask
        for k in range(6):
            assert pred[k].item() == (0.0 if want_mask[k] else s[k, int(t[k]) - r * V].item())


def test_colsum_and_activation_backward():
    dy, pre = randn((9, 7), torch.float32, 0), randn((9, 7), torch.float32, 1)
    close(oracle.colsum(dy.reshape(3, 3, 7)), dy.sum(0))
    for kind, fn in (("gelu_tanh", lambda v: F.gelu(v, approximate="tanh")), ("gelu", F.gelu), ("relu", F.relu)):
        p = pre.clone().requires_grad_(True)
        fn(p).backward(dy)
        g, s = oracle.act_bwd_colsum(kind, dy, pre)
        close(g, p.grad)
        close(s, p.grad.sum(0))


def test_cpu_path_restatement_matches_torch_library_routines():
    """oracle/cpu_path.py (what bench.py times as the reference's CPU path) against the library routines the
    reference's tests use as their oracle: F.linear, F.layer_norm and F.cross_entropy with autograd."""
    import torch.nn.functional as F
    from oracle import cpu_path

    g = torch.Generator().manual_seed(0)
    x = torch.randn((24, 64), generator=g)
    w = torch.randn((48, 64), generator=g) * 0.1
    b = torch.randn((48,), generator=g)
    dy = torch.randn((24, 48), generator=g)
    y, dx, dw, db = cpu_path.linear1d_col_fwd_bwd(x, w, b, dy)
    xr, wr, br = (t.clone().requires_grad_(True) for t in (x, w, b))
    F.linear(xr, wr, br).backward(dy)
    assert torch.allclose(y, F.linear(x, w, b)) and torch.allclose(dx, xr.grad) and torch.allclose(dw, wr.grad)
    assert torch.allclose(db, br.grad)
    # LayerNorm2D with the whole hidden size on the rank
    xl = torch.randn((16, 96), generator=g)
    gamma, beta = torch.rand((96,), generator=g) + 0.5, torch.randn((96,), generator=g)
    dyl = torch.randn((16, 96), generator=g)
    y, dx, dgam, dbet = cpu_path.layernorm2d_fwd_bwd(xl, gamma, beta, dyl, 96, 1e-5, False)
    xr, gr, br = (t.clone().requires_grad_(True) for t in (xl, gamma, beta))
    ref = F.layer_norm(xr, (96,), gr, br, 1e-5)
    ref.backward(dyl)
    for got, want in ((y, ref.detach()), (dx, xr.grad), (dgam, gr.grad), (dbet, br.grad)):
        assert torch.allclose(got, want, atol=2e-5, rtol=1e-4)
    # cross-entropy over two vocabulary slices: the slices' losses and gradients assemble F.cross_entropy's
    logits = torch.randn((12, 40), generator=g) * 2
    t = torch.randint(0, 40, (12,), generator=g)
    dl = torch.rand((12,), generator=g) + 0.5
    lr = logits.clone().requires_grad_(True)
    ref = F.cross_entropy(lr, t, reduction="none")
    ref.backward(dl)
    loss, grad = cpu_path.vpce1d_fwd_bwd(logits, t, 0, dl, False)   # one slice holding the whole vocabulary
    assert torch.allclose(loss, ref.detach(), atol=1e-5) and torch.allclose(grad, lr.grad, atol=1e-6)
