"""Pins oracle/embedding.py without the GPU: the vocabulary slices' outputs sum to torch's own
F.embedding on the whole table, the slices' gradients are the row blocks of its autograd gradient, and
the masked / edge ids behave as the reference's statements say."""
import torch
import torch.nn.functional as F

import oracle
from tests.util import randn


def test_slices_reassemble_f_embedding_and_its_gradient():
    vocab, e, p = 48, 6, 4
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, vocab, (3, 17), generator=g)
    table = randn((vocab, e), torch.float32, 1).requires_grad_(True)
    d_out = randn((3, 17, e), torch.float32, 2)
    ref = F.embedding(ids, table)
    (ref_grad,) = torch.autograd.grad(ref, table, d_out)
    total = torch.zeros_like(ref)
    for r in range(p):
        lo, hi = r * vocab // p, (r + 1) * vocab // p
        total += oracle.vocab_embedding_fwd(ids, table[lo:hi], lo)
        dw = oracle.vocab_embedding_bwd(ids, d_out, hi - lo, lo)
        assert torch.allclose(dw, ref_grad[lo:hi], rtol=1e-6, atol=1e-6)
    assert torch.equal(total, ref.detach())


def test_edge_ids_and_padding_row():
    w = torch.arange(12, dtype=torch.float32).view(4, 3) + 1
    ids = torch.tensor([9, 10, 13, 14, 0, 11])  # slice [10, 14)
    out = oracle.vocab_embedding_fwd(ids, w, 10)
    assert out.tolist() == [[0, 0, 0], [1, 2, 3], [10, 11, 12], [0, 0, 0], [0, 0, 0], [4, 5, 6]]
    d_out = torch.ones((6, 3))
    dw = oracle.vocab_embedding_bwd(ids, d_out, 4, 10)
    assert dw[:, 0].tolist() == [1, 1, 0, 1]
    # F.embedding(shifted ids, weight, padding_idx) blocks the gradient of row `padding_idx` of the slice
    ref_w = w.clone().requires_grad_(True)
    shifted = (ids - 10).clamp(0, 3)
    live = ((ids >= 10) & (ids < 14)).float().unsqueeze(-1)
    (ref,) = torch.autograd.grad(F.embedding(shifted, ref_w, padding_idx=1) * live, ref_w, d_out)
    assert torch.equal(oracle.vocab_embedding_bwd(ids, d_out, 4, 10, padding_idx=1), ref)


def test_clip_grad_oracle_against_torch_and_by_hand():
    """oracle.clip_grad_norm equals torch.nn.utils.clip_grad_norm_ for untagged parameters (the function the
    reference adapts, cubework/utils/clip_grad.py:1-4), and a parameter tagged with n partitions counts n times."""
    shapes = [(13, 5), (7,), (1,), (4, 4, 4)]
    for norm_type in (2.0, 1.0, 3.0, float("inf")):
        for max_norm in (0.3, 1e6):
            ps = [torch.nn.Parameter(torch.zeros(s)) for s in shapes]
            for i, p in enumerate(ps):
                p.grad = randn(s if False else shapes[i], torch.float32, 20 + i)
            grads = [p.grad.clone() for p in ps]
            want = torch.nn.utils.clip_grad_norm_(ps, max_norm, norm_type)
            total, clipped = oracle.clip_grad_norm(grads, [0] * len(ps), max_norm, norm_type)
            assert torch.allclose(total.float(), want, rtol=1e-5)
            for c, p in zip(clipped, ps):
                assert torch.allclose(c.float(), p.grad, rtol=1e-5, atol=1e-7)
    g = [torch.tensor([3.0]), torch.tensor([2.0, 2.0])]
    total, clipped = oracle.clip_grad_norm(g, [0, 2], 1.0)  # sqrt(9 + 2 * 8) = 5
    assert abs(total.item() - 5.0) < 1e-12 and torch.allclose(clipped[0], torch.tensor([3.0 / (5 + 1e-6)], dtype=torch.float64))
