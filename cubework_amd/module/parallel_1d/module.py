"""1D (Megatron) layers with the reference's signatures and shard shapes
(cubework/module/parallel_1d/module.py):

  Linear1D_Col  weight [out/p, in]  bias [out/p]   (:213-278)
  Linear1D_Row  weight [out, in/p]  bias [out]     (:281-346)
  Linear1D      picks Col, then Row, from env.parallel_input_1d (:25-69)
  Classifier1D  weight [classes, in/p] bias [classes]          (:90-151)
  VocabParallelClassifier1D weight [classes/p, in] bias [classes/p] (:154-210)
  LayerNorm1D   a plain nn.LayerNorm (:72-87)
"""
import math
from typing import Callable, Optional

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn.parameter import Parameter

from ... import ops
from ...distributed import ParallelManager as pm
from ...distributed import seed
from ...global_vars import env
from .. import init
from ..utils import set_tensor_parallel_attribute_by_partition
from ._operation import (gather_forward_split_backward, get_parallel_input, linear_nt, reduce_grad, reduce_input,
                         set_parallel_input, split_forward_gather_backward)


class Linear1D_Col(nn.Module):

    def __init__(self, in_features: int, out_features: int, bias: bool = True, gather_output: bool = False,
                 skip_bias_add: bool = False, weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1), activation: Optional[str] = None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.gather_output = gather_output
        self.skip_bias_add = skip_bias_add
        self.activation = activation
        if skip_bias_add and not bias:
            raise ValueError("cannot skip bias addition if bias is None")
        if activation is not None and skip_bias_add:
            raise ValueError("a fused activation needs the bias added inside the layer (skip_bias_add=False)")
        self.out_features_per_partition = out_features // pm.PARALLEL_1D.world_size
        self.weight = Parameter(torch.empty(self.out_features_per_partition, in_features))
        self.bias = Parameter(torch.empty(self.out_features_per_partition)) if bias else None
        with seed(pm.PARALLEL_1D):
            weight_initializer(self.weight, fan_in=in_features, fan_out=out_features)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        num_partition = pm.PARALLEL_1D.world_size
        set_tensor_parallel_attribute_by_partition(self.weight, num_partition)
        if self.bias is not None:
            set_tensor_parallel_attribute_by_partition(self.bias, num_partition)
        set_parallel_input(True)

    def forward(self, input_: Tensor):
        input_parallel = reduce_grad(input_, pm.PARALLEL_1D)
        bias = self.bias if not self.skip_bias_add else None
        output = linear_nt(input_parallel, self.weight, bias, self.activation)
        if self.gather_output:
            output = gather_forward_split_backward(output, pm.PARALLEL_1D, dim=-1)
        return (output, self.bias) if self.skip_bias_add else output


class Linear1D_Row(nn.Module):

    def __init__(self, in_features: int, out_features: int, bias: bool = True, parallel_input: bool = True,
                 skip_bias_add: bool = False, weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.parallel_input = parallel_input
        self.skip_bias_add = skip_bias_add
        if skip_bias_add and not bias:
            raise ValueError("cannot skip bias addition if bias is None")
        self.input_size_per_partition = in_features // pm.PARALLEL_1D.world_size
        self.weight = Parameter(torch.empty(out_features, self.input_size_per_partition))
        self.bias = Parameter(torch.empty(out_features)) if bias else None
        with seed(pm.PARALLEL_1D):
            weight_initializer(self.weight, fan_in=in_features, fan_out=out_features)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        set_tensor_parallel_attribute_by_partition(self.weight, pm.PARALLEL_1D.world_size)
        set_parallel_input(False)

    def forward(self, input_: Tensor):
        if not self.parallel_input:
            input_ = split_forward_gather_backward(input_, pm.PARALLEL_1D, dim=-1)
        add_here = self.bias is not None and not self.skip_bias_add
        if pm.PARALLEL_1D.world_size == 1:
            # no peers' partial products to add: the bias goes into the GEMM epilogue
            output = linear_nt(input_, self.weight, self.bias if add_here else None)
        else:
            output = reduce_input(linear_nt(input_, self.weight), pm.PARALLEL_1D)
            if add_here:
                output = _BiasAdd.apply(output, self.bias)
        return (output, self.bias) if self.skip_bias_add else output


class _BiasAdd(torch.autograd.Function):
    """output + bias after the all-reduce of a row-parallel product."""

    @staticmethod
    def forward(ctx, input_, bias):
        ctx.bias_dtype = bias.dtype
        return ops.bias_act(input_, bias, None)

    @staticmethod
    def backward(ctx, grad):
        return grad, ops.colsum(grad.reshape(-1, grad.shape[-1]), out_dtype=ctx.bias_dtype)


class Linear1D(nn.Module):

    def __init__(self, in_features: int, out_features: int, bias: bool = True, gather_output: bool = False,
                 skip_bias_add: bool = False, weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        parallel_input = get_parallel_input()
        if not parallel_input:
            self.linear = Linear1D_Col(in_features, out_features, bias=bias, gather_output=gather_output,
                                       skip_bias_add=skip_bias_add, weight_initializer=weight_initializer,
                                       bias_initializer=bias_initializer)
        else:
            self.linear = Linear1D_Row(in_features, out_features, bias=bias, parallel_input=parallel_input,
                                       skip_bias_add=skip_bias_add, weight_initializer=weight_initializer,
                                       bias_initializer=bias_initializer)

    def forward(self, *args, **kwargs):
        return self.linear(*args, **kwargs)

    @property
    def weight(self):
        return self.linear.weight

    @property
    def bias(self):
        return self.linear.bias


class LayerNorm1D(nn.Module):

    def __init__(self, normalized_shape: int, eps=1e-05):
        super().__init__()
        self.norm = nn.LayerNorm(normalized_shape, eps=eps)

    def forward(self, *args, **kwargs):
        return self.norm(*args, **kwargs)

    @property
    def weight(self):
        return self.norm.weight

    @property
    def bias(self):
        return self.norm.bias


class Classifier1D(nn.Module):

    def __init__(self, in_features: int, num_classes: int, weight: Parameter = None, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.num_classes = num_classes
        self.parallel_input = get_parallel_input()
        self.input_size_per_partition = in_features // pm.PARALLEL_1D.world_size
        if weight is not None:
            self.weight = weight
            self.has_weight = False
        else:
            self.weight = Parameter(torch.empty(num_classes, self.input_size_per_partition))
            self.has_weight = True
        self.bias = Parameter(torch.empty(num_classes)) if bias else None
        with seed(pm.PARALLEL_1D):
            if self.has_weight:
                weight_initializer(self.weight, fan_in=in_features, fan_out=num_classes)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        if self.has_weight:
            set_tensor_parallel_attribute_by_partition(self.weight, pm.TENSOR.world_size)
        set_parallel_input(False)
        env.vocab_parallel = False

    def forward(self, input_: Tensor) -> Tensor:
        if not self.parallel_input:
            input_ = split_forward_gather_backward(input_, pm.PARALLEL_1D, dim=-1)
        if pm.PARALLEL_1D.world_size == 1:
            return linear_nt(input_, self.weight, self.bias)
        output = reduce_input(linear_nt(input_, self.weight), pm.PARALLEL_1D)
        return _BiasAdd.apply(output, self.bias) if self.bias is not None else output


class VocabParallelClassifier1D(nn.Module):

    def __init__(self, in_features: int, num_classes: int, weight: Parameter = None, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.num_classes = num_classes
        self.parallel_input = get_parallel_input()
        self.num_classes_per_partition = num_classes // pm.PARALLEL_1D.world_size
        if weight is not None:
            self.weight = weight
            self.has_weight = False
        else:
            self.weight = Parameter(torch.empty(self.num_classes_per_partition, in_features))
            self.has_weight = True
        self.bias = Parameter(torch.empty(self.num_classes_per_partition)) if bias else None
        with seed(pm.PARALLEL_1D):
            if self.has_weight:
                weight_initializer(self.weight, fan_in=in_features, fan_out=num_classes)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        num_partition = pm.PARALLEL_1D.world_size
        if self.has_weight:
            set_tensor_parallel_attribute_by_partition(self.weight, num_partition)
        if self.bias is not None:
            set_tensor_parallel_attribute_by_partition(self.bias, num_partition)
        set_parallel_input(False)
        env.vocab_parallel = True

    def forward(self, input_: Tensor) -> Tensor:
        return linear_nt(reduce_grad(input_, pm.PARALLEL_1D), self.weight, self.bias)
