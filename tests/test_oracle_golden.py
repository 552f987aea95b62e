"""The CPU oracle against the committed golden vectors (tests/golden/
golden_small.json, brute force in float64 with finite-difference gradients;
see make_golden.py). Runs without a GPU."""
import json
import os

import pytest
import torch

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "golden_small.json")) as f:
    GOLDEN = json.load(f)


def T64(v):
    return torch.tensor(v, dtype=torch.float64)


def close(got, want, tol):
    got = got.double()
    want = want.double() if torch.is_tensor(want) else T64(want)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = (got - want).abs().max().item()
    assert err <= tol * max(want.abs().max().item(), 1.0), err


@pytest.mark.parametrize("case", GOLDEN["gemm"], ids=lambda c: c["layout"] + "-" + c["act"])
def test_gemm_ksteps(case):
    A = [T64(a) for a in case["A"]]
    B = [T64(b) for b in case["B"]]
    adds = [T64(case["addend"])] if case["addend"] is not None else []
    act = None if case["act"] == "none" else case["act"]
    out, pre = oracle.gemm_ksteps(case["layout"], A, B, T64(case["bias"]), act, adds, compute_dtype=torch.float64,
                                  return_preact=True)
    close(pre, case["preact"], 1e-12)
    close(out, case["out"], 1e-12)
    # the fp32 evaluation the parity tests use stays within fp32 rounding of it
    out32 = oracle.gemm_ksteps(case["layout"], [a.float() for a in A], [b.float() for b in B],
                               T64(case["bias"]).float(), act, [t.float() for t in adds])
    close(out32, case["out"], 2e-6)


def test_activation_grad_matches_finite_differences():
    x = torch.linspace(-4, 4, 41, dtype=torch.float64)
    h = 1e-6
    for kind in ("gelu_tanh", "gelu_erf", "relu"):
        fd = (oracle.activation(x + h, kind) - oracle.activation(x - h, kind)) / (2 * h)
        got = oracle.activation_grad(x, kind)
        keep = x.abs() > 1e-3 if kind == "relu" else torch.ones_like(x, dtype=torch.bool)
        close(got[keep], fd[keep], 1e-6)


@pytest.mark.parametrize("case", GOLDEN["layernorm"], ids=["eps1e-5", "eps1e-12"])
def test_layernorm_2d_and_3d(case):
    x, dy = T64(case["x"]).float(), T64(case["dy"]).float()
    gamma, beta, eps = T64(case["gamma"]).float(), T64(case["beta"]).float(), case["eps"]
    H = x.shape[1]
    half = H // 2
    # 2D flavour as a q = 2 row group: partials of each half, summed, normalise per half
    st_a, st_b = oracle.ln2d_partial_stats(x[:, :half]), oracle.ln2d_partial_stats(x[:, half:])
    close(st_a, case["stats_local"], 1e-6)
    close(st_b, case["stats_peer"], 1e-6)
    stats = st_a + st_b
    ya, mr = oracle.ln2d_normalize(x[:, :half], stats, H, eps, gamma[:half], beta[:half])
    yb, _ = oracle.ln2d_normalize(x[:, half:], stats, H, eps, gamma[half:], beta[half:])
    close(torch.cat([ya, yb], dim=1), case["y"], 2e-5)
    rs_a, dg_a, db_a = oracle.ln2d_backward_partials(dy[:, :half], x[:, :half], mr, gamma[:half])
    rs_b, dg_b, db_b = oracle.ln2d_backward_partials(dy[:, half:], x[:, half:], mr, gamma[half:])
    rs = rs_a + rs_b
    dxa = oracle.ln2d_backward_dx(dy[:, :half], x[:, :half], mr, rs, H, gamma[:half])
    dxb = oracle.ln2d_backward_dx(dy[:, half:], x[:, half:], mr, rs, H, gamma[half:])
    close(torch.cat([dxa, dxb], dim=1), case["dx"], 2e-4)
    close(torch.cat([dg_a, dg_b]), case["dgamma"], 2e-4)
    close(torch.cat([db_a, db_b]), case["dbeta"], 1e-5)
    # 3D flavour (two-pass), whole row on one rank
    y3, mu, sigma = oracle.ln3d_forward(x, gamma, beta, H, eps)
    close(y3, case["y"], 2e-5)
    dx3, dg3, db3 = oracle.ln3d_backward(dy, mu, sigma, gamma, H)
    close(dx3, case["dx"], 2e-4)
    close(dg3, case["dgamma"], 2e-4)
    close(db3, case["dbeta"], 1e-5)
    # 3D flavour split over a depth-2 output group
    peer_sum = x[:, half:].sum(-1)
    mean = x.sum(-1) / H
    peer_sq = ((x[:, half:] - mean[:, None]) ** 2).sum(-1)
    y3a, _, _ = oracle.ln3d_forward(x[:, :half], gamma[:half], beta[:half], H, eps, peer_sum, peer_sq)
    close(y3a, T64(case["y"])[:, :half], 2e-5)


@pytest.mark.parametrize("case", GOLDEN["cross_entropy"], ids=["3slices", "2slices"])
def test_vocab_parallel_cross_entropy(case):
    logits, targets = T64(case["logits"]).float(), torch.tensor(case["targets"])
    p = case["slices"]
    V = logits.shape[1] // p
    dloss = T64(case["dloss"]).float()
    stats = []
    for r, s in enumerate(torch.chunk(logits, p, dim=-1)):
        m, se, pred, mask = oracle.vpce_fwd_local(s, targets, r * V)
        # integer / gather part: exact
        assert mask.tolist() == case["mask"][r]
        assert torch.equal(pred, T64(case["pred"][r]).float())
        assert torch.equal(m, T64(case["max"][r]).float())
        shifted = [(t - r * V) if not mk else 0 for t, mk in zip(case["targets"], case["mask"][r])]
        assert shifted == case["shifted"][r]
        stats.append((m, se, pred, mask))
    loss, gmax, gsum = oracle.vpce_finalize(*(torch.stack([s[k] for s in stats]) for k in range(4)))
    close(loss, case["loss"], 2e-6)
    grads = [oracle.vpce_bwd(s, targets, r * V, gmax, gsum, dloss)
             for r, s in enumerate(torch.chunk(logits, p, dim=-1))]
    close(torch.cat(grads, dim=1), case["grad"], 2e-5)
    # the line-by-line restatement of the reference agrees too
    loss2, grads2 = oracle.vpce_reference_full(list(torch.chunk(logits, p, dim=-1)), targets, dloss)
    close(loss2, case["loss"], 2e-6)
    close(torch.cat(grads2, dim=1), case["grad"], 2e-5)
