"""Vocab-parallel cross-entropy operator: one rank's share of
_VocabParallelCrossEntropy1D/2D/3D (cubework/module/loss/loss_1d.py:11-79,
loss_2d.py:30-93, loss_3d.py:36-91).

forward: one online pass over the local logits slice gives (max, sum-exp,
target logit, mask); the MAX / SUM / SUM all-reduces of the reference
(loss_1d.py:18,44,50) become one exchange of those four per-row values, which
cw_vpce_finalize combines. backward recomputes the softmax from the saved
logits and the global (max, sum) instead of keeping a softmax-sized buffer,
and never writes into the caller's logits (the reference's 1D variant does,
loss_1d.py:20,47-48).
"""
import torch

from ... import ops
from .._amp import bwd, loss_fwd


class _VocabParallelCrossEntropy(torch.autograd.Function):

    @staticmethod
    @loss_fwd()
    def forward(ctx, logits, targets, parallel_mode):
        vocab = logits.size(-1)
        vocab_start = parallel_mode.local_rank * vocab
        logits_2d = logits.reshape(-1, vocab)
        local = ops.vpce_fwd_local(logits_2d, targets.reshape(-1), vocab_start)
        if parallel_mode.world_size == 1:
            stacked = [s.unsqueeze(0) for s in local]
        else:
            # peers' (max, sumexp, pred, mask), each [world_size - 1, tokens]
            peers = parallel_mode.take("vpce_stats")
            stacked = [torch.cat([s.unsqueeze(0), p.to(s.dtype).reshape(-1, s.numel())]) for s, p in zip(local, peers)]
        loss, gmax, gsum = ops.vpce_finalize(*stacked)
        ctx.save_for_backward(logits_2d, targets.reshape(-1), gmax, gsum)
        ctx.meta = (vocab_start, logits.shape)
        return loss.reshape(targets.shape)

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        logits_2d, targets, gmax, gsum = ctx.saved_tensors
        vocab_start, shape = ctx.meta
        grad = ops.vpce_bwd(logits_2d, targets, vocab_start, gmax, gsum, output_grad.reshape(-1).float(), 1.0)
        return grad.reshape(shape), None, None


def vocab_parallel_cross_entropy(logits, targets, parallel_mode):
    """Per-token loss [targets.shape] for this rank's vocabulary slice."""
    return _VocabParallelCrossEntropy.apply(logits, targets, parallel_mode)
