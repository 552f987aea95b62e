"""Loss modules with the reference's names and signatures
(cubework/module/loss/loss_1d.py:82-91, loss_2d.py:13-27,96-110,
loss_3d.py:12-33,94-110, losses.py:21-35)."""
import torch.nn as nn
from torch.nn.functional import cross_entropy

from ...distributed import ParallelManager as pm
from ...global_vars import env
from ..parallel_2d._utils import assert_summa_initialization, reduce_by_batch_2d, split_batch_2d
from ..parallel_3d._utils import (get_input_parallel_mode, get_output_parallel_mode, get_weight_parallel_mode,
                                  reduce_by_batch_3d, split_batch_3d)
from ..utils import get_tensor_parallel_mode
from ._operation import vocab_parallel_cross_entropy


class VocabParallelCrossEntropyLoss1D(nn.Module):
    def __init__(self, reduction=True):
        super().__init__()
        self.reduction_mean = reduction

    def forward(self, logits, targets):
        loss = vocab_parallel_cross_entropy(logits, targets, pm.PARALLEL_1D)
        return loss.mean() if self.reduction_mean else loss


class VocabParallelCrossEntropyLoss2D(nn.Module):
    """The class axis is split over the grid columns (the ROW group,
    loss_2d.py:45-48); logits must be [tokens, vocab/q] and targets [tokens]."""

    def __init__(self, reduction=True):
        super().__init__()
        self.reduction_mean = reduction

    def forward(self, logits, targets):
        targets = split_batch_2d(targets)
        loss = vocab_parallel_cross_entropy(logits, targets, pm.PARALLEL_2D_ROW)
        if self.reduction_mean:
            loss = reduce_by_batch_2d(loss.mean(), True)
        return loss


class VocabParallelCrossEntropyLoss3D(nn.Module):
    def __init__(self, reduction=True):
        super().__init__()
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.reduction_mean = reduction

    def forward(self, logits, targets):
        targets = split_batch_3d(targets, input_parallel_mode=self.input_parallel_mode,
                                 weight_parallel_mode=self.weight_parallel_mode)
        loss = vocab_parallel_cross_entropy(logits, targets, self.output_parallel_mode)
        if self.reduction_mean:
            loss = reduce_by_batch_3d(loss.mean(), self.input_parallel_mode, self.weight_parallel_mode, True)
        return loss


class CrossEntropyLoss2D(nn.Module):
    """Not vocab-parallel: stock F.cross_entropy plus the batch reduction."""

    def __init__(self, reduction=True, *args, **kwargs):
        super().__init__()
        assert_summa_initialization()
        self.reduction_mean = reduction
        self.loss_args = args
        self.loss_kwargs = kwargs

    def forward(self, logits, targets):
        targets = split_batch_2d(targets)
        loss = cross_entropy(logits, targets, reduction="none", *self.loss_args, **self.loss_kwargs)
        if self.reduction_mean:
            loss = reduce_by_batch_2d(loss.mean(), True)
        return loss


class CrossEntropyLoss3D(nn.Module):
    def __init__(self, reduction=True, *args, **kwargs):
        super().__init__()
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.reduction_mean = reduction
        self.loss_args = args
        self.loss_kwargs = kwargs

    def forward(self, logits, targets):
        targets = split_batch_3d(targets, input_parallel_mode=self.input_parallel_mode,
                                 weight_parallel_mode=self.weight_parallel_mode)
        loss = cross_entropy(logits, targets, reduction="none", *self.loss_args, **self.loss_kwargs)
        if self.reduction_mean:
            loss = reduce_by_batch_3d(loss.mean(), self.input_parallel_mode, self.weight_parallel_mode, True)
        return loss


_parallel_cross_entropy = {"2d": CrossEntropyLoss2D, "3d": CrossEntropyLoss3D}
_vocab_parallel_cross_entropy = {"1d": VocabParallelCrossEntropyLoss1D, "2d": VocabParallelCrossEntropyLoss2D,
                                 "3d": VocabParallelCrossEntropyLoss3D}


class CrossEntropyLoss(nn.Module):
    """Facade: vocab-parallel when a vocab-parallel classifier/embedding was
    built before it (env.vocab_parallel), else the mode's plain loss."""

    def __init__(self, reduction: bool = True, *args, **kwargs):
        super().__init__()
        tensor_parallel = get_tensor_parallel_mode()
        if tensor_parallel is not None and env.vocab_parallel:
            self.loss = _vocab_parallel_cross_entropy[tensor_parallel](reduction=reduction, *args, **kwargs)
        elif tensor_parallel is None or tensor_parallel == "1d":
            self.loss = nn.CrossEntropyLoss(reduction="mean" if reduction else "none", *args, **kwargs)
        else:
            self.loss = _parallel_cross_entropy[tensor_parallel](reduction=reduction, *args, **kwargs)

    def forward(self, *args, **kwargs):
        return self.loss(*args, **kwargs)
