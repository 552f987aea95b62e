"""Mode-dispatching facade (cubework/module/modules.py:83-188): Linear,
LayerNorm and Classifier pick the 1d/2d/3d implementation from `env.mode`
(and `env.vocab_parallel`), move it to `dtype` and expose .weight / .bias.
With no tensor parallelism they are the stock torch layers, as in the
reference."""
import math
from typing import Callable

from torch import nn

from ..global_vars import env
from . import init
from .parallel_1d import Classifier1D, LayerNorm1D, Linear1D, VocabParallelClassifier1D
from .parallel_2d import Classifier2D, LayerNorm2D, Linear2D, VocabParallelClassifier2D, split_batch_2d
from .parallel_3d import Classifier3D, LayerNorm3D, Linear3D, VocabParallelClassifier3D, split_batch_3d
from .utils import get_tensor_parallel_mode

_parallel_layernorm = {"1d": LayerNorm1D, "2d": LayerNorm2D, "3d": LayerNorm3D}
_parallel_linear = {"1d": Linear1D, "2d": Linear2D, "3d": Linear3D}
_parallel_classifier = {"1d": Classifier1D, "2d": Classifier2D, "3d": Classifier3D}
_vocab_parallel_classifier = {"1d": VocabParallelClassifier1D, "2d": VocabParallelClassifier2D,
                              "3d": VocabParallelClassifier3D}
_parallel_split_batch = {"2d": split_batch_2d, "3d": split_batch_3d}


def partition_batch(input_):
    mode = get_tensor_parallel_mode()
    if mode not in _parallel_split_batch:
        return input_
    split = _parallel_split_batch[mode]
    if isinstance(input_, dict):
        return {k: split(v) for k, v in input_.items()}
    if isinstance(input_, (tuple, list)):
        return type(input_)(split(x) for x in input_)
    return split(input_)


class _Wrapped(nn.Module):
    _inner = "linear"

    def forward(self, *args, **kwargs):
        return getattr(self, self._inner)(*args, **kwargs)

    @property
    def weight(self):
        return getattr(self, self._inner).weight

    @property
    def bias(self):
        return getattr(self, self._inner).bias


class LayerNorm(_Wrapped):
    _inner = "norm"

    def __init__(self, normalized_shape: int, eps=1e-05, dtype=None):
        super().__init__()
        mode = get_tensor_parallel_mode()
        norm = nn.LayerNorm(normalized_shape, eps=eps) if mode is None else _parallel_layernorm[mode](normalized_shape, eps=eps)
        self.norm = norm.to(dtype)


class Linear(_Wrapped):

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype=None,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1), **kwargs):
        super().__init__()
        mode = get_tensor_parallel_mode()
        if mode is None:
            linear = nn.Linear(in_features, out_features, bias=bias)
            weight_initializer(linear.weight, fan_in=in_features, fan_out=out_features)
            if linear.bias is not None:
                bias_initializer(linear.bias, fan_in=in_features)
        else:
            linear = _parallel_linear[mode](in_features, out_features, bias=bias, weight_initializer=weight_initializer,
                                            bias_initializer=bias_initializer, **kwargs)
        self.linear = linear.to(dtype)


class _ClassifierSTD(nn.Module):
    """No tensor parallelism: F.linear with an optionally shared weight
    (cubework/module/module_std.py ClassifierSTD)."""

    def __init__(self, in_features, num_classes, weight=None, bias=True, weight_initializer=None,
                 bias_initializer=None):
        super().__init__()
        import torch
        if weight is not None:
            self.weight, self.has_weight = weight, False
        else:
            self.weight, self.has_weight = nn.Parameter(torch.empty(num_classes, in_features)), True
            weight_initializer(self.weight, fan_in=in_features, fan_out=num_classes)
        self.bias = nn.Parameter(torch.zeros(num_classes)) if bias else None
        if self.bias is not None:
            bias_initializer(self.bias, fan_in=in_features)

    def forward(self, input_):
        return nn.functional.linear(input_, self.weight, self.bias)


class Classifier(_Wrapped):

    def __init__(self, in_features: int, num_classes: int, weight: nn.Parameter = None, bias: bool = True, dtype=None,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        mode = get_tensor_parallel_mode()
        if env.vocab_parallel:
            cls = _vocab_parallel_classifier[mode]
        else:
            cls = _ClassifierSTD if mode is None else _parallel_classifier[mode]
        self.linear = cls(in_features, num_classes, weight=weight, bias=bias, weight_initializer=weight_initializer,
                          bias_initializer=bias_initializer).to(dtype)
