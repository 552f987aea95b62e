"""The reference's CPU path for the benchmark workloads, statement by statement, for timing.

The reference runs on CPU tensors as plain torch with the gloo backend at world size 1
(cubework/initialize.py:33-35). At world size 1 its own collective wrappers return their input
(cubework/distributed/collective.py:8-10 and following), but the raw torch.distributed.all_reduce calls
inside the loss and inside _Layernorm_2D.backward still run on the group; they are kept here (`group` is the
default process group of a gloo world of one, or None to skip them when no group could be formed).

bench.py's cpu_baseline leg times these functions on the GPU host's cores. Test infrastructure only (see
oracle/__init__.py): nothing in cubework_amd imports this module.
"""
import torch
import torch.distributed as dist
import torch.nn.functional as F


def _all_reduce(t, group_ok, op=None):
    if group_ok:
        if op is None:
            dist.all_reduce(t)
        else:
            dist.all_reduce(t, op=op)
    return t


def linear1d_col_fwd_bwd(x, weight, bias, dy):
    """Linear1D_Col at world size 1: F.linear forward (parallel_1d/module.py:263-278) and its autograd
    backward (dX, dW, db). x [..., in], weight [out, in]; returns (y, dx, dw, db)."""
    x = x.detach().requires_grad_(True)
    w = weight.detach().requires_grad_(True)
    b = bias.detach().requires_grad_(True)
    y = F.linear(x, w, b)
    y.backward(dy)
    return y.detach(), x.grad, w.grad, b.grad


def layernorm2d_fwd_bwd(x, gamma, beta, dy, hidden, eps, group_ok):
    """LayerNorm2D forward (parallel_2d/module.py:142-171, _operation.py:321-324) and backward
    (_operation.py:330-347, autograd of addcmul) on one rank's [rows, hidden/q] shard, in the tensors' own
    dtype as the reference's eager path runs it. The two forward all-reduces go through the reference's
    wrapper, which is the identity at world size 1; the two in the backward are raw calls and run."""
    E_x = torch.sum(x, dim=-1, keepdim=True) / hidden                    # module.py:144-145
    Var_x = torch.sum(x * x, dim=-1, keepdim=True) / hidden              # :148-149
    Var_x = Var_x - E_x * E_x                                            # :151
    Var_x = 1.0 / torch.sqrt(Var_x + eps)                                # :153
    xh = (x - E_x) * Var_x                                               # _operation.py:321-324
    y = torch.addcmul(beta, gamma, xh)                                   # module.py:170
    # backward: autograd of addcmul, then _Layernorm_2D.backward
    dbeta = dy.reshape(-1, dy.shape[-1]).sum(0)
    dgamma = (dy * xh).reshape(-1, dy.shape[-1]).sum(0)
    g = dy * gamma
    g_sum = torch.sum(g, dim=-1, keepdim=True)                           # _operation.py:334
    _all_reduce(g_sum, group_ok)                                         # :335
    g_sum /= hidden
    gx_sum = torch.sum(g * xh, dim=-1, keepdim=True)                     # :338
    _all_reduce(gx_sum, group_ok)                                        # :339
    gx_sum /= hidden
    dx = g.clone()                                                       # :342-345
    dx -= xh * gx_sum
    dx -= g_sum
    dx *= Var_x
    return y, dx, dgamma, dbeta


def vpce1d_fwd_bwd(logits, targets, vocab_start, dloss, group_ok):
    """_VocabParallelCrossEntropy1D forward and backward (loss/loss_1d.py:14-79) on one rank's vocabulary
    slice, with its three all-reduces. The reference casts the logits to fp32 (custom_fwd(cast_inputs=
    torch.float32) applies under autocast; its training scripts run under autocast) and then works in place
    on that copy; so does this."""
    x = logits.float()                                                   # the cast copy the Function receives
    logits_max = torch.max(x, dim=-1)[0]                                 # :17
    _all_reduce(logits_max, group_ok, dist.ReduceOp.MAX)                 # :18
    x.sub_(logits_max.unsqueeze(dim=-1))                                 # :20
    V = x.size()[-1]
    vocab_end = vocab_start + V
    target_mask = (targets < vocab_start) | (targets >= vocab_end)       # :29
    masked_target = targets.clone() - vocab_start
    masked_target[target_mask] = 0                                       # :30-31
    x2 = x.view(-1, V)
    arange = torch.arange(start=0, end=x2.size()[0])
    predicted = x2[arange, masked_target.view(-1)].clone().contiguous()  # :36-40
    predicted[target_mask.view(-1)] = 0.0                                # :42
    _all_reduce(predicted, group_ok)                                     # :44
    torch.exp(x, out=x)                                                  # :47-48
    sum_exp = x.sum(dim=-1)                                              # :49
    _all_reduce(sum_exp, group_ok)                                       # :50
    loss = torch.log(sum_exp) - predicted                                # :53
    x.div_(sum_exp.unsqueeze(dim=-1))                                    # :55
    # backward (:61-79)
    grad = x
    g2 = grad.view(-1, V)
    g2[arange, masked_target.view(-1)] -= 1.0 - target_mask.view(-1).float()   # :74
    grad.mul_(dloss.unsqueeze(dim=-1))                                   # :77
    return loss, grad
