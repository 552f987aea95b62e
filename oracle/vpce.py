"""Oracle for vocab-parallel cross-entropy, one rank's slice. Test
infrastructure only (see oracle/__init__.py).

Reference statements followed (cubework/module/loss/):
  loss_1d.py:17      logits_max = max over the local vocab slice      (2D :39, 3D :43)
  loss_1d.py:20      logits - global max                              (2D :43, 3D :46)
  loss_1d.py:23-31   vocab_start/end, target_mask, masked_target      (2D :45-53, 3D :48-56)
  loss_1d.py:36-42   predicted = logits[arange, masked_target]; [mask] = 0
  loss_1d.py:47-49   sum_exp = exp(logits - max).sum(-1)
  loss_1d.py:53      loss = log(sum_exp) - predicted
  loss_1d.py:55-56   softmax = exp / sum_exp
  loss_1d.py:74,77   grad = softmax; grad[arange, masked_target] -= 1 - mask; grad *= dloss
The three all_reduces (:18 MAX, :44 SUM, :50 SUM) are replaced by explicit
per-rank statistics that `vpce_finalize` combines. 2D/3D use an inclusive
vocab_end with `>` (loss_2d.py:48-50): the same set of targets.
"""
import torch


from ._precision import compute_dtype, to_compute as _f


def vpce_fwd_local(logits: torch.Tensor, targets: torch.Tensor, vocab_start: int):
    """(max, sumexp relative to the LOCAL max, pred, mask) for one slice."""
    x = _f(logits).reshape(-1, logits.shape[-1])
    t = targets.detach().to("cpu").reshape(-1).to(torch.int64)
    V = x.shape[-1]
    vocab_end = vocab_start + V
    m = torch.max(x, dim=-1)[0]
    sumexp = torch.exp(x - m.unsqueeze(-1)).sum(dim=-1)
    mask = (t < vocab_start) | (t >= vocab_end)
    masked_target = t.clone() - vocab_start
    masked_target[mask] = 0
    ar = torch.arange(x.shape[0])
    pred = x[ar, masked_target].clone()
    pred[mask] = 0.0
    return m, sumexp, pred, mask.to(torch.uint8)


def vpce_finalize(max_all, sumexp_all, pred_all, mask_all):
    """Combine [n_ranks, T] statistics: global max, global sum of
    exponentials, loss = log(S) - sum_r (mask_r ? 0 : pred_r - max)."""
    max_all, sumexp_all, pred_all = _f(max_all), _f(sumexp_all), _f(pred_all)
    mask_all = mask_all.detach().to("cpu").to(torch.bool)
    gmax = max_all.max(dim=0)[0]
    gsum = (sumexp_all * torch.exp(max_all - gmax)).sum(dim=0)
    predicted = torch.where(mask_all, torch.zeros_like(pred_all), pred_all - gmax).sum(dim=0)
    loss = torch.log(gsum) - predicted
    return loss, gmax, gsum


def vpce_bwd(logits, targets, vocab_start: int, gmax, gsum, dloss):
    """Gradient w.r.t. this rank's logits slice; dloss is [T] or a scalar.
    Returned in the compute type."""
    x = _f(logits).reshape(-1, logits.shape[-1])
    t = targets.detach().to("cpu").reshape(-1).to(torch.int64)
    V = x.shape[-1]
    mask = (t < vocab_start) | (t >= vocab_start + V)
    masked_target = t.clone() - vocab_start
    masked_target[mask] = 0
    softmax = torch.exp(x - _f(gmax).unsqueeze(-1)) / _f(gsum).unsqueeze(-1)
    grad = softmax
    ar = torch.arange(x.shape[0])
    grad[ar, masked_target] -= 1.0 - mask.to(grad.dtype)
    dl = dloss if torch.is_tensor(dloss) else torch.tensor(float(dloss))
    dl = _f(dl)
    grad = grad * (dl.unsqueeze(-1) if dl.dim() == 1 else dl)
    return grad.reshape(logits.shape)


def vpce_reference_full(slices, targets, dloss=None):
    """All ranks at once, written as the reference writes it for one rank
    (loss_1d.py:14-57,61-79) with the all_reduces done by hand. slices: list of
    [T, V_r] tensors, equal widths. Returns (loss [T], [grad_r])."""
    xs = [_f(s).reshape(-1, s.shape[-1]) for s in slices]
    t = targets.detach().to("cpu").reshape(-1).to(torch.int64)
    V = xs[0].shape[-1]
    logits_max = torch.stack([torch.max(x, dim=-1)[0] for x in xs]).max(dim=0)[0]      # :17-18
    xs = [x - logits_max.unsqueeze(-1) for x in xs]                                     # :20
    predicted = torch.zeros(xs[0].shape[0], dtype=compute_dtype())
    masks, mts = [], []
    ar = torch.arange(xs[0].shape[0])
    for r, x in enumerate(xs):
        start, end = V * r, V * r + V                                                   # :23-26
        mask = (t < start) | (t >= end)                                                 # :29
        mt = t.clone() - start
        mt[mask] = 0                                                                    # :30-31
        p = x[ar, mt].clone()
        p[mask] = 0.0                                                                   # :39-42
        predicted = predicted + p                                                       # :44
        masks.append(mask)
        mts.append(mt)
    exps = [torch.exp(x) for x in xs]                                                   # :47-48
    sum_exp = sum(e.sum(dim=-1) for e in exps)                                          # :49-50
    loss = torch.log(sum_exp) - predicted                                               # :53
    grads = []
    dl = torch.ones_like(loss) if dloss is None else _f(dloss if torch.is_tensor(dloss) else torch.tensor(float(dloss)))
    for e, mask, mt in zip(exps, masks, mts):
        g = e / sum_exp.unsqueeze(-1)                                                   # :55
        g[ar, mt] -= 1.0 - mask.to(g.dtype)                                                # :74
        g = g * (dl.unsqueeze(-1) if dl.dim() == 1 else dl)                             # :77
        grads.append(g)
    return loss, grads
