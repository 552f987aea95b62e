"""Oracle for LayerNorm2D / LayerNorm3D per-rank math. Test infrastructure only
(see oracle/__init__.py).

Reference statements followed:
  cubework/module/parallel_2d/module.py:143-153   E_x = sum(x)/H; Var_x = sum(x*x)/H - E_x^2;
                                                  rstd = 1/sqrt(Var_x + eps)
  cubework/module/parallel_2d/_operation.py:321-324  x_hat = (x - E_x) * rstd
  cubework/module/parallel_2d/module.py:170       y = addcmul(bias, scale, x_hat)
  cubework/module/parallel_2d/_operation.py:334-345  backward of x_hat w.r.t. x
  cubework/module/parallel_3d/_operation.py:273-281  two-pass mean / var / sigma, y = w*z + b
  cubework/module/parallel_3d/_operation.py:294-311  3D backward
Collectives are replaced by explicit "local partial" / "summed over peers"
arguments. All arithmetic is in the oracle's compute type (fp32 unless oracle.precision says
float64) on the inputs as given.
"""
from typing import Optional

import torch


from ._precision import round_like, to_compute as _f


# ---- 2D: one-pass statistics ----------------------------------------------
def ln2d_partial_stats(x: torch.Tensor) -> torch.Tensor:
    """[rows, 2] = (sum x, sum x*x) over the local columns
    (parallel_2d/module.py:144,148 before the all_reduce)."""
    x = _f(x).reshape(-1, x.shape[-1])
    return torch.stack([x.sum(dim=-1), (x * x).sum(dim=-1)], dim=-1)


def ln2d_mean_rstd(stats_global: torch.Tensor, hidden: int, eps: float) -> torch.Tensor:
    """(mean, rstd) from statistics summed over the row group
    (parallel_2d/module.py:145,149,151,153)."""
    s = _f(stats_global)
    e_x = s[:, 0] / hidden
    var = s[:, 1] / hidden
    var = var - e_x * e_x
    rstd = 1.0 / torch.sqrt(var + eps)
    return torch.stack([e_x, rstd], dim=-1)


def ln2d_normalize(x, stats_global, hidden: int, eps: float, gamma=None, beta=None):
    """Returns (y, mean_rstd). y keeps x's dtype."""
    xf = _f(x).reshape(-1, x.shape[-1])
    mr = ln2d_mean_rstd(stats_global, hidden, eps)
    xh = (xf - mr[:, 0:1]) * mr[:, 1:2]  # _operation.py:321-324
    y = xh
    if gamma is not None:
        y = y * _f(gamma)
    if beta is not None:
        y = y + _f(beta)  # module.py:170
    return round_like(y, x).reshape(x.shape), mr


def ln2d_backward_partials(dy, x, mean_rstd, gamma=None):
    """Local partial sums of the backward. With g = dy*gamma (autograd of
    addcmul, module.py:170) and x_hat = (x-mean)*rstd:
      row_sums = (sum_c g, sum_c g*x_hat)   (_operation.py:334,338 before all_reduce)
      dgamma = sum_r dy*x_hat, dbeta = sum_r dy  (autograd of addcmul + _operation.py:285-286)
    """
    dyf = _f(dy).reshape(-1, dy.shape[-1])
    xf = _f(x).reshape(-1, x.shape[-1])
    mr = _f(mean_rstd)
    xh = (xf - mr[:, 0:1]) * mr[:, 1:2]
    g = dyf if gamma is None else dyf * _f(gamma)
    row_sums = torch.stack([g.sum(dim=-1), (g * xh).sum(dim=-1)], dim=-1)
    return row_sums, (dyf * xh).sum(dim=0), dyf.sum(dim=0)


def ln2d_backward_dx(dy, x, mean_rstd, row_sums_global, hidden: int, gamma=None):
    """dx = (g - x_hat*mean(g*x_hat) - mean(g)) * rstd (_operation.py:336-345)."""
    dyf = _f(dy).reshape(-1, dy.shape[-1])
    xf = _f(x).reshape(-1, x.shape[-1])
    mr = _f(mean_rstd)
    rs = _f(row_sums_global)
    xh = (xf - mr[:, 0:1]) * mr[:, 1:2]
    g = dyf if gamma is None else dyf * _f(gamma)
    grad = g.clone()
    grad -= xh * (rs[:, 1:2] / hidden)
    grad -= rs[:, 0:1] / hidden
    grad *= mr[:, 1:2]
    return round_like(grad, x).reshape(x.shape)


# ---- 3D: two-pass statistics ------------------------------------------------
def ln3d_forward(x, gamma, beta, hidden: int, eps: float, peer_sum=None, peer_sqdev=None):
    """_Layernorm3D.forward on the local columns (parallel_3d/_operation.py:273-281).
    peer_sum / peer_sqdev: what the other ranks of the output group contribute
    to the two all_reduces (None = this rank holds the whole hidden size).
    Returns (y, mu, sigma)."""
    xf = _f(x).reshape(-1, x.shape[-1])
    s = xf.sum(dim=-1, keepdim=True)
    if peer_sum is not None:
        s = s + _f(peer_sum).reshape(-1, 1)
    mean = s / hidden
    mu = xf - mean
    v = (mu ** 2).sum(dim=-1, keepdim=True)
    if peer_sqdev is not None:
        v = v + _f(peer_sqdev).reshape(-1, 1)
    var = v / hidden
    sigma = torch.sqrt(var + eps)
    z = mu / sigma
    y = _f(gamma) * z + _f(beta)
    return round_like(y, x).reshape(x.shape), mu, sigma


def ln3d_backward(dy, mu, sigma, gamma, hidden: int, peer_dvar=None, peer_dmean_fn=None):
    """_Layernorm3D.backward (parallel_3d/_operation.py:294-311) for a rank that
    holds the whole hidden size when the peer terms are None.
    Returns (dx, dgamma, dbeta)."""
    dyf = _f(dy).reshape(-1, dy.shape[-1])
    w = _f(gamma)
    dbeta = dyf.sum(dim=0)
    dgamma = (dyf * mu / sigma).sum(dim=0)
    dz = dyf * w
    dvar = (dz * mu * (-0.5) * sigma ** (-3)).sum(dim=-1, keepdim=True)
    if peer_dvar is not None:
        dvar = dvar + peer_dvar
    dmean = (dz * (-1 / sigma) + dvar * -2 * mu / hidden).sum(dim=-1, keepdim=True)
    if peer_dmean_fn is not None:
        dmean = dmean + peer_dmean_fn(dvar)
    dx = dz / sigma + dvar * 2 * mu / hidden + dmean / hidden
    return round_like(dx, dy).reshape(dy.shape), dgamma, dbeta


# ---- whole-row helpers (tensor-parallel size 1) -----------------------------
def ln_forward_full(x, gamma, beta, eps: float, two_pass: bool = False):
    """LayerNorm over the whole last dimension, 2D (one-pass) or 3D (two-pass) flavour."""
    H = x.shape[-1]
    if two_pass:
        y, mu, sigma = ln3d_forward(x, gamma if gamma is not None else torch.ones(H),
                                    beta if beta is not None else torch.zeros(H), H, eps)
        mean = (_f(x).reshape(-1, H) - mu)[:, 0]
        return y, torch.stack([mean, 1.0 / sigma[:, 0]], dim=-1)
    return ln2d_normalize(x, ln2d_partial_stats(x), H, eps, gamma, beta)


def ln_backward_full(dy, x, mean_rstd, gamma: Optional[torch.Tensor]):
    H = x.shape[-1]
    row_sums, dgamma, dbeta = ln2d_backward_partials(dy, x, mean_rstd, gamma)
    dx = ln2d_backward_dx(dy, x, mean_rstd, row_sums, H, gamma)
    return dx, dgamma, dbeta
