"""Oracle for tensor-parallel-aware gradient-norm clipping. Test infrastructure only
(see oracle/__init__.py).

Reference statements followed (cubework/utils/clip_grad.py):
  :31-35   infinity norm: max over parameters of max |g|
  :39-46   else: per parameter norm(g, p) ** p, times NUM_PARTITIONS for tagged parameters
  :47-54   std_norm + all_reduce(tp_norm) / world_size, then ** (1 / p)
  :63-68   clip_coef = max_norm / (total_norm + 1e-6), clamped at 1, g *= clip_coef
At tensor-parallel size 1 the all-reduce is the identity.
"""
import torch


def clip_grad_norm(grads, partitions, max_norm, norm_type=2.0):
    """grads: list of tensors; partitions: NUM_PARTITIONS of each (0 = untagged). Returns
    (total_norm, clipped gradients) in float64."""
    gs = [g.detach().to("cpu").to(torch.float64) for g in grads]
    if norm_type == float("inf"):
        total = max(g.abs().max() for g in gs)
    else:
        std = sum(g.abs().pow(norm_type).sum() for g, n in zip(gs, partitions) if n <= 0)
        tp = sum(g.abs().pow(norm_type).sum() * n for g, n in zip(gs, partitions) if n > 0)
        total = (std + tp) ** (1.0 / norm_type)
    coef = min(1.0, float(max_norm) / (float(total) + 1e-6))
    return torch.as_tensor(total), [g * coef for g in gs]
