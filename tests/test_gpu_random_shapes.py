"""Seeded random shapes through the C ABI against the CPU oracle: the block GEMM across its three code
paths (register-staged, LDS-DMA, split-k), the attention core, LayerNorm and the cross-entropy slice.
Shapes are drawn once from fixed seeds, so the cases are the same in every run."""
import random

import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _gemm_cases():
    rng = random.Random(1234)
    cases = []
    for _ in range(10):  # ragged: register-staged kernel with guards
        cases.append((rng.choice(["NN", "NT", "TN"]), rng.randint(1, 700), rng.randint(1, 700), rng.randint(1, 300),
                      rng.randint(1, 3)))
    for _ in range(6):   # tile-aligned with many tiles: LDS-DMA kernel
        cases.append((rng.choice(["NN", "NT", "TN"]), 256 * rng.randint(8, 12), 256 * rng.randint(8, 16),
                      64 * rng.randint(1, 5), rng.randint(1, 4)))
    for _ in range(6):   # few tiles, long reduction: split-k
        cases.append((rng.choice(["NN", "NT", "TN"]), 256 * rng.randint(1, 3), 256 * rng.randint(1, 4),
                      512 * rng.randint(2, 5), rng.randint(1, 4)))
    return cases


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", _gemm_cases())
def test_random_gemm(case, dtype):
    import oracle
    from cubework_amd import ops

    layout, M, N, K, steps = case
    a_shape = (K, M) if layout == "TN" else (M, K)
    b_shape = (N, K) if layout == "NT" else (K, N)
    A = [randn(a_shape, dtype, 7 * s + M) for s in range(steps)]
    B = [randn(b_shape, dtype, 7 * s + N + 1, std=0.05) for s in range(steps)]
    bias = randn((N,), dtype, K, std=0.3)
    act = ["relu", "gelu_tanh", None][(M + N + K) % 3]
    want = oracle.gemm_ksteps(layout, A, B, bias, act)
    got = ops.gemm_ksteps(layout, [a.to(DEV) for a in A], [b.to(DEV) for b in B], bias.to(DEV), act)
    torch.cuda.synchronize()
    assert_parity(got, want, dtype, "gemm %s %s" % (case, dtype))


def _attn_cases():
    rng = random.Random(99)
    return [(rng.randint(1, 3), rng.randint(1, 900), rng.randint(1, 5), rng.random() < 0.7) for _ in range(12)]


@pytest.mark.parametrize("case", _attn_cases())
def test_random_attention(case):
    import oracle
    from cubework_amd import ops

    b, s, h, causal = case
    d = 64
    qkv = randn((b, s, h * 3 * d), torch.bfloat16, s + 3 * h, std=1.3)
    d_out = randn((b, s, h * d), torch.bfloat16, s + 5)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    want = oracle.attention_core(qc, kc, vc, causal=causal)
    dq, dk, dv = oracle.attention_core_backward(qc, kc, vc, d_out, causal=causal)
    t = qkv.to(DEV).view(b, s, h, 3 * d)
    q, k, v = t[..., :d], t[..., d:2 * d], t[..., 2 * d:]
    out, lse = ops.attn_fwd(q, k, v, causal=causal, want_lse=True)
    g = torch.empty_like(t)
    ops.attn_bwd(q, k, v, out, d_out.to(DEV), lse, g[..., :d], g[..., d:2 * d], g[..., 2 * d:], causal=causal)
    torch.cuda.synchronize()
    assert_parity(out, want, torch.bfloat16, "attention out %s" % (case,))
    if s == 1:
        assert_parity(g.permute(0, 2, 1, 3), torch.cat([dq, dk, dv], dim=-1), torch.bfloat16, "attention grads %s" % (case,))
        return
    for name, got, ref in (("dq", g[..., :d], dq), ("dk", g[..., d:2 * d], dk), ("dv", g[..., 2 * d:], dv)):
        assert_parity(got.permute(0, 2, 1, 3), ref, torch.bfloat16, "attention %s %s" % (name, case))


def _ln_cases():
    rng = random.Random(5)
    return [(rng.randint(1, 600), 8 * rng.randint(1, 520)) for _ in range(8)] + [(rng.randint(1, 50), rng.randint(1, 3000)) for _ in range(4)]


@pytest.mark.parametrize("shape", _ln_cases())
def test_random_layernorm(shape):
    import oracle
    from cubework_amd import ops

    R, C = shape
    x = randn((R, C), torch.bfloat16, R + C)
    dy = randn((R, C), torch.bfloat16, R + C + 1)
    gamma = (1 + 0.1 * randn((C,), torch.float32, 3)).to(torch.bfloat16)
    beta = randn((C,), torch.bfloat16, 4, std=0.05)
    with oracle.precision(torch.float64):
        y_ref, mr_ref = oracle.ln_forward_full(x, gamma, beta, 1e-5)
        dx_ref, dg_ref, db_ref = oracle.ln_backward_full(dy, x, mr_ref, gamma)
    xd, dyd, gd, bd = (t.to(DEV) for t in (x, dy, gamma, beta))
    y, mr = ops.ln_forward_fused(xd, 1e-5, gd, bd)
    rs, dgam, dbet = ops.ln_bwd_partials(dyd, xd, mr, gd)
    dx = ops.ln_bwd_dx(dyd, xd, mr, rs, C, gd)
    torch.cuda.synchronize()
    assert_parity(y, y_ref, torch.bfloat16, "ln y %s" % (shape,))
    assert_parity(dx, dx_ref, torch.bfloat16, "ln dx %s" % (shape,))
    assert_parity(dgam, dg_ref, torch.float32, "ln dgamma %s" % (shape,))
    assert_parity(dbet, db_ref, torch.float32, "ln dbeta %s" % (shape,))


def _embedding_cases():
    rng = random.Random(4242)
    cases = []
    for _ in range(14):
        dtype_i = rng.randint(0, 2)
        vec = 4 if dtype_i == 1 else 8
        cases.append((rng.choice([1, 2, 31, 64, 65, 500, 2049, 8192, 16384]) if rng.random() < 0.5 else rng.randint(1, 16384),
                      vec * rng.randint(1, 520), rng.randint(1, 3000), rng.randint(0, 5000), dtype_i,
                      rng.choice(["uniform", "hot", "one_id", "zipf"]), rng.random() < 0.5))
    return cases


@pytest.mark.parametrize("case", _embedding_cases())
def test_random_embedding_backward_from_ids(case):
    """cw_embed_bwd_ids on drawn shapes and id distributions (uniform over a vocabulary wider than the slice, one hot
    id for every third token, a single id for all tokens, Zipf-like frequencies), with and without a skipped row:
    float64 sums within the dtype's bar, rows without tokens exactly zero, two calls bit-identical, and equal bit
    for bit to the token-order path wherever no row has more than one token (where neither path adds anything)."""
    from cubework_amd import ops

    T, E, rows, start, dtype_i, dist, with_skip = case
    dtype = [torch.bfloat16, torch.float32, torch.float16][dtype_i]
    g = torch.Generator().manual_seed(T * 31 + E)
    vocab = start + rows + 200
    if dist == "one_id":
        ids = torch.full((T,), start + rows // 2, dtype=torch.int64)
    elif dist == "zipf":
        u = torch.rand((T,), generator=g)
        ids = (start - 50 + ((rows + 100) * u ** 3)).long().clamp(0, vocab - 1)
    else:
        ids = torch.randint(max(0, start - 100), vocab, (T,), generator=g)
        if dist == "hot":
            ids[::3] = start + min(7, rows - 1)
    skip = min(3, rows - 1) if with_skip else -1
    d_out = randn((T, E), dtype, T + 5)
    got = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, start, skip, via_token_order=False)
    again = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, start, skip, via_token_order=False)
    torch.cuda.synchronize()
    assert torch.equal(got, again), "fixed summation order: bit-reproducible"
    local = ids - start
    live = (local >= 0) & (local < rows) & (local != skip)
    want = torch.zeros((rows, E), dtype=torch.float64).index_add_(0, local[live], d_out.double()[live])
    assert_parity(got, want, dtype, "embedding d_weight from ids %s" % (case,))
    untouched = torch.ones(rows, dtype=torch.bool)
    untouched[local[live]] = False
    assert (got.cpu()[untouched] == 0).all(), "rows without tokens (and the skipped row) are exactly zero"
    counts = torch.bincount(local[live], minlength=rows)
    if int(counts.max()) <= 1:
        via = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, start, skip, via_token_order=True)
        assert torch.equal(got, via)
