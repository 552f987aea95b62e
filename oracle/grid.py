"""Single-process emulator of a q x q SUMMA grid built from the per-rank oracle
functions: loops over the ranks, Python lists stand in for broadcasts and
sums for reduces. It shows that one rank's kernels compose to the master
result, with the shard layout of the reference's own test
(tests/test_2d/check_2d_modules.py:38-63: i = row index = PARALLEL_2D_COL rank,
j = column index = PARALLEL_2D_ROW rank; activations chunk(dim 0)[i],
chunk(-1)[j]; weight the same; bias chunk(-1)[j] then [i]).
Test infrastructure only (see oracle/__init__.py).
"""
from typing import Callable, Dict, Tuple

import torch

from . import layernorm as _ln
from . import summa as _summa
from . import vpce as _vpce

Rank = Tuple[int, int]


def shard(t: torch.Tensor, q: int, i: int, j: int) -> torch.Tensor:
    return torch.chunk(torch.chunk(t, q, dim=0)[i], q, dim=-1)[j].contiguous()


def bias_shard(b: torch.Tensor, q: int, i: int, j: int) -> torch.Tensor:
    return torch.chunk(torch.chunk(b, q, dim=-1)[j], q, dim=-1)[i].contiguous()


def gathered_bias(b: torch.Tensor, q: int, j: int) -> torch.Tensor:
    """all_gather over the column group of the [out/q^2] shards = feature chunk j
    (parallel_2d/_operation.py:264)."""
    return torch.cat([bias_shard(b, q, i, j) for i in range(q)], dim=-1)


def linear2d_forward(A_master, W_master, b_master, q: int, act=None,
                     rank_fn: Callable = _summa.gemm_ksteps) -> Dict[Rank, torch.Tensor]:
    """Linear2D.forward on every rank. rank_fn(layout, A_steps, B_steps, bias, act)
    is the per-rank kernel (the oracle by default; tests pass the HIP operator)."""
    A2 = A_master.reshape(-1, A_master.shape[-1])
    out = {}
    for i in range(q):
        for j in range(q):
            A_steps = [shard(A2, q, i, k) for k in range(q)]        # row broadcast of step k
            B_steps = [shard(W_master, q, k, j) for k in range(q)]  # column broadcast of step k
            bias = None if b_master is None else gathered_bias(b_master, q, j)
            out[(i, j)] = rank_fn("NN", A_steps, B_steps, bias, act)
    return out


def linear2d_backward(A_master, W_master, dC_master, q: int, rank_fn: Callable = _summa.gemm_ksteps):
    """dA, dW, dbias shards on every rank via summa_ABT / summa_ATB
    (parallel_2d/_operation.py:61-80,119-125,199-204,285-287)."""
    A2 = A_master.reshape(-1, A_master.shape[-1])
    dC2 = dC_master.reshape(-1, dC_master.shape[-1])
    # partial products every rank computes for its peers
    abt = {}  # abt[(i, j, k)] = dC(i,j) W(k,j)^T, destined for rank (i,k)
    atb = {}  # atb[(i, j, k)] = A(i,k)^T dC(i,j), destined for rank (k,j)
    for i in range(q):
        for j in range(q):
            dC = shard(dC2, q, i, j)
            for k in range(q):
                abt[(i, j, k)] = rank_fn("NT", [dC], [shard(W_master, q, k, j)], None, None)
                atb[(i, j, k)] = rank_fn("TN", [shard(A2, q, i, k)], [dC], None, None)
    dA, dW, db = {}, {}, {}
    for i in range(q):
        for j in range(q):
            dC = shard(dC2, q, i, j)
            peers = [abt[(i, jp, j)] for jp in range(q) if jp != j]
            dA[(i, j)] = rank_fn("NT", [dC], [shard(W_master, q, j, j)], None, None, peers)
            peers = [atb[(ip, j, i)] for ip in range(q) if ip != i]
            dW[(i, j)] = rank_fn("TN", [shard(A2, q, i, i)], [dC], None, None, peers)
            # column sum, then reduce_scatter over the column group: rank (i,j) keeps piece i
            total = sum(_summa.colsum(shard(dC2, q, ip, j)) for ip in range(q))
            db[(i, j)] = torch.chunk(total, q, dim=-1)[i]
    return dA, dW, db


def layernorm2d_forward(A_master, q: int, eps: float, gamma_master=None, beta_master=None):
    """LayerNorm2D.forward on every rank; returns {rank: (y, mean_rstd)}."""
    A2 = A_master.reshape(-1, A_master.shape[-1])
    H = A2.shape[-1]
    out = {}
    for i in range(q):
        stats = sum(_ln.ln2d_partial_stats(shard(A2, q, i, j)) for j in range(q))  # all_reduce over the row group
        for j in range(q):
            g = None if gamma_master is None else torch.chunk(gamma_master, q, dim=-1)[j]
            b = None if beta_master is None else torch.chunk(beta_master, q, dim=-1)[j]
            out[(i, j)] = _ln.ln2d_normalize(shard(A2, q, i, j), stats, H, eps, g, b)
    return out


def layernorm2d_backward(A_master, dY_master, q: int, eps: float, gamma_master=None):
    A2 = A_master.reshape(-1, A_master.shape[-1])
    dY2 = dY_master.reshape(-1, dY_master.shape[-1])
    H = A2.shape[-1]
    fwd = layernorm2d_forward(A_master, q, eps)
    dx = {}
    for i in range(q):
        parts = []
        for j in range(q):
            g = None if gamma_master is None else torch.chunk(gamma_master, q, dim=-1)[j]
            parts.append(_ln.ln2d_backward_partials(shard(dY2, q, i, j), shard(A2, q, i, j), fwd[(i, j)][1], g)[0])
        row_sums = sum(parts)
        for j in range(q):
            g = None if gamma_master is None else torch.chunk(gamma_master, q, dim=-1)[j]
            dx[(i, j)] = _ln.ln2d_backward_dx(shard(dY2, q, i, j), shard(A2, q, i, j), fwd[(i, j)][1], row_sums, H, g)
    return dx


def vocab_parallel_ce(logits_master, targets, p: int, dloss=None):
    """Vocab-parallel CE over p vocabulary slices; returns (loss, [grad_r])."""
    slices = list(torch.chunk(logits_master, p, dim=-1))
    V = slices[0].shape[-1]
    stats = [_vpce.vpce_fwd_local(s, targets, r * V) for r, s in enumerate(slices)]
    loss, gmax, gsum = _vpce.vpce_finalize(*(torch.stack([st[k] for st in stats]) for k in range(4)))
    dl = torch.ones_like(loss) if dloss is None else dloss
    grads = [_vpce.vpce_bwd(s, targets, r * V, gmax, gsum, dl) for r, s in enumerate(slices)]
    return loss, grads
