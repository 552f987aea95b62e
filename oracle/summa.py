"""Oracle for the SUMMA block GEMMs, the bias add and the activation that
follows the linear layer. Test infrastructure only (see oracle/__init__.py).

Reference statements followed (paths relative to the reference tree):
  cubework/module/parallel_2d/_operation.py:41-47    C = 0; for i: C = addmm(C, A_i, B_i)
  cubework/module/parallel_2d/_operation.py:119-125  C_temp = A @ B_i^T, reduced to rank i
  cubework/module/parallel_2d/_operation.py:199-204  C_temp = A_i^T @ B, reduced to rank i
  cubework/module/parallel_2d/_operation.py:264-274  output = input_ + all_gather(bias)
  cubework/module/parallel_2d/_operation.py:285-287  dbias = sum over rows of the output grad
  cubework/module/parallel_1d/module.py:269,338      F.linear(x, W, b)
  cubework/module/parallel_3d/_operation.py:34,39,53,59,65
  benchmark/gpt2/gpt2.py:116-117 (gelu after the linear), benchmark/opt/opt.py:200 (ReLU)
"""
from typing import Optional, Sequence

import torch
import torch.nn.functional as F

from . import _precision
from ._precision import round_like


def _f(t: torch.Tensor, dtype) -> torch.Tensor:
    return t.detach().to("cpu").to(dtype)


def activation(x: torch.Tensor, kind: Optional[str]) -> torch.Tensor:
    if kind in (None, "none"):
        return x
    if kind == "gelu_tanh":
        return F.gelu(x, approximate="tanh")
    if kind in ("gelu", "gelu_erf"):
        return F.gelu(x)
    if kind == "relu":
        return F.relu(x)
    raise ValueError(kind)


def activation_grad(x: torch.Tensor, kind: Optional[str]) -> torch.Tensor:
    """d act(x) / dx by autograd of the torch routine."""
    x = x.detach().clone().requires_grad_(True)
    activation(x, kind).sum().backward()
    return x.grad


def gemm_ksteps(layout: str, A_steps: Sequence[torch.Tensor], B_steps: Sequence[torch.Tensor],
                bias: Optional[torch.Tensor] = None, act: Optional[str] = None,
                addends: Sequence[torch.Tensor] = (), compute_dtype=None, return_preact: bool = False):
    """act(sum_i op(A_i) op(B_i) + sum_j addends_j + bias), accumulated in
    compute_dtype (default: the oracle's compute type) on the inputs as given; 16-bit
    inputs give a result rounded once to their type, fp32 inputs one in compute_dtype.

    The k-step loop is parallel_2d/_operation.py:43-47 (NN), :119-125 (NT),
    :199-204 (TN) with the broadcast operands passed in; addends are the
    partial products a `reduce` delivers from the peers.
    """
    if compute_dtype is None:
        compute_dtype = _precision.compute_dtype()
    out_dtype = A_steps[0].dtype if A_steps[0].dtype in (torch.bfloat16, torch.float16) else compute_dtype
    acc = None
    for a, b in zip(A_steps, B_steps):
        a, b = _f(a, compute_dtype), _f(b, compute_dtype)
        a = a.reshape(-1, a.shape[-1])
        b = b.reshape(-1, b.shape[-1])
        if layout == "NN":
            p = a @ b
        elif layout == "NT":
            p = a @ b.t()
        elif layout == "TN":
            p = a.t() @ b
        else:
            raise ValueError(layout)
        acc = p if acc is None else acc + p
    for t in addends:
        acc = acc + _f(t, compute_dtype).reshape(acc.shape)
    if bias is not None:
        acc = acc + _f(bias, compute_dtype)
    pre = acc
    out = activation(acc, act)
    if return_preact:
        return out.to(out_dtype), pre.to(out_dtype)
    return out.to(out_dtype)


def summa_ab_rank(A_steps, B_steps, bias=None, act=None, **kw):
    """One rank's _SUMMA_AB.forward + _SUMMAbias.forward (+ activation)."""
    return gemm_ksteps("NN", A_steps, B_steps, bias, act, **kw)


def summa_abt_rank(A, B_steps, my_index: int, peer_partials=(), **kw):
    """One rank's _SUMMA_ABT.forward: the product for step `my_index` plus the
    partial products the row peers computed for that step
    (parallel_2d/_operation.py:122-125)."""
    return gemm_ksteps("NT", [A], [B_steps[my_index]], addends=peer_partials, **kw)


def summa_atb_rank(A_steps, B, my_index: int, peer_partials=(), **kw):
    """One rank's _SUMMA_ATB.forward (parallel_2d/_operation.py:201-204)."""
    return gemm_ksteps("TN", [A_steps[my_index]], [B], addends=peer_partials, **kw)


def summa_ab_reference_dtype(A_steps, B_steps, bias=None):
    """The reference's eager path in the tensors' own dtype: C is rounded to
    the input dtype after every k-step (parallel_2d/_operation.py:41,47) and
    the bias is added in that dtype (:273). Informational comparison only."""
    a0 = A_steps[0].detach().cpu()
    C = torch.zeros((a0.reshape(-1, a0.shape[-1]).shape[0], B_steps[0].shape[-1]), dtype=a0.dtype)
    for a, b in zip(A_steps, B_steps):
        a = a.detach().cpu().reshape(-1, a.shape[-1])
        C = torch.addmm(C, a, b.detach().cpu())
    if bias is not None:
        C = C + bias.detach().cpu()
    return C


def colsum(dy: torch.Tensor) -> torch.Tensor:
    """Sum over every dimension but the last, in the compute type
    (parallel_2d/_operation.py:285-286, parallel_3d/_operation.py:59)."""
    d = _f(dy, _precision.compute_dtype())
    return d.reshape(-1, d.shape[-1]).sum(dim=0)


def act_bwd_colsum(kind, dy: torch.Tensor, preact: torch.Tensor):
    """Backward of `act(preact)` followed by the bias-gradient column sum."""
    ct = _precision.compute_dtype()
    g = _f(dy, ct) * activation_grad(_f(preact, ct), kind)
    return round_like(g, dy), g.reshape(-1, g.shape[-1]).sum(dim=0)
