"""Pins oracle/attention.py without the GPU: pure-Python float64 loops on tiny inputs, torch's own
scaled_dot_product_attention and its autograd (the closed-form backward shares no code with autograd), and
invariants of the softmax chain."""
import torch
import torch.nn.functional as F

import oracle
from tests.util import randn


def _qkv(b, s, h, d, seed):
    return randn((b, s, h * 3 * d), torch.float32, seed)


def test_forward_against_brute_force():
    for causal in (True, False):
        q, k, v = oracle.split_qkv(_qkv(1, 5, 2, 4, 1), 2)
        got = oracle.attention_core(q, k, v, causal=causal)
        want = oracle.attention_brute_force(q, k, v, 4 ** -0.5, causal)
        assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-6)


def test_split_qkv_layout():
    # heads own 3*d consecutive columns: q, k, v side by side (benchmark/opt/opt.py:72-76)
    b, s, h, d = 1, 2, 3, 2
    x = torch.arange(b * s * h * 3 * d, dtype=torch.float32).view(b, s, h * 3 * d)
    q, k, v = oracle.split_qkv(x, h)
    assert q.shape == (b, h, s, d)
    assert q[0, 1, 0].tolist() == [6.0, 7.0] and k[0, 1, 0].tolist() == [8.0, 9.0] and v[0, 1, 0].tolist() == [10.0, 11.0]


def test_forward_and_lse_against_torch_sdpa():
    q, k, v = oracle.split_qkv(_qkv(2, 37, 3, 8, 2), 3)
    for causal in (True, False):
        got, lse = oracle.attention_core(q, k, v, causal=causal, return_lse=True)
        want = F.scaled_dot_product_attention(q, k, v, is_causal=causal).transpose(1, 2).reshape(2, 37, 24)
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)
        w = torch.matmul(q, k.transpose(-1, -2)) * 8 ** -0.5
        if causal:
            w = w.masked_fill(torch.ones(37, 37, dtype=torch.bool).triu(1), float("-inf"))
        assert torch.allclose(lse, torch.logsumexp(w, -1), rtol=1e-6, atol=1e-6)


def test_backward_against_autograd():
    q, k, v = [t.clone().requires_grad_(True) for t in oracle.split_qkv(_qkv(2, 19, 2, 8, 3), 2)]
    d_out = randn((2, 19, 16), torch.float32, 4)
    for causal in (True, False):
        out = F.scaled_dot_product_attention(q, k, v, is_causal=causal).transpose(1, 2).reshape(2, 19, 16)
        want = torch.autograd.grad(out, (q, k, v), d_out)
        got = oracle.attention_core_backward(q, k, v, d_out, causal=causal)
        for g, w in zip(got, want):
            assert torch.allclose(g, w, rtol=1e-4, atol=1e-5)


def test_invariants():
    q, k, v = oracle.split_qkv(_qkv(1, 23, 2, 8, 5), 2)
    ones = torch.ones_like(v)
    assert torch.allclose(oracle.attention_core(q, k, ones), torch.ones(1, 23, 16), atol=1e-6)
    # first causal row attends to key 0 only
    assert torch.allclose(oracle.attention_core(q, k, v)[0, 0].view(2, 8), v[0, :, 0], atol=1e-6)
    # a constant added to every score of a row (k -> k + c along q's direction is not constant, so shift v
    # instead): dV sums the probabilities, whose rows sum to one
    d_out = randn((1, 23, 16), torch.float32, 6)
    _, _, dv = oracle.attention_core_backward(q, k, v, d_out, causal=False)
    assert torch.allclose(dv.sum(dim=2), d_out.view(1, 23, 2, 8).transpose(1, 2).sum(dim=2), rtol=1e-4, atol=1e-5)
