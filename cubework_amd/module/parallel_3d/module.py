"""3D layers with the reference's signatures and shard shapes
(cubework/module/parallel_3d/module.py):

  LayerNorm3D  weight, bias [hidden/d], default eps 1e-12        (:22-62)
  Linear3D     weight [in/d, out/d^2]   bias [out/d]             (:65-126)
  Classifier3D weight [classes, in/d]   bias [classes]           (:129-190)
  VocabParallelClassifier3D weight [classes/d^2, in/d] bias [classes/d] (:193-261)
"""
import math
from typing import Callable, Optional

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn import Parameter

from ...distributed import ParallelManager as pm
from ...distributed import seed
from ...global_vars import env
from .. import init
from ..utils import set_tensor_parallel_attribute_by_partition
from ._operation import classifier_3d, layernorm_3d, linear_3d, vocab_parallel_classifier_3d
from ._utils import (get_depth_from_env, get_input_parallel_mode, get_input_x_weight_parallel_mode,
                     get_output_parallel_mode, get_output_x_weight_parallel_mode, get_weight_parallel_mode,
                     swap_in_out_group)


class LayerNorm3D(nn.Module):

    def __init__(self, normalized_shape: int, eps: float = 1e-12):
        super().__init__()
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.input_x_weight_parallel_mode = get_input_x_weight_parallel_mode()
        self.depth = get_depth_from_env()
        self.normalized_shape = normalized_shape
        self.normalized_shape_per_partition = normalized_shape // self.depth
        self.weight = Parameter(torch.ones(self.normalized_shape_per_partition))
        self.bias = Parameter(torch.zeros(self.normalized_shape_per_partition))
        self.variance_epsilon = eps
        set_tensor_parallel_attribute_by_partition(self.weight, self.depth)
        set_tensor_parallel_attribute_by_partition(self.bias, self.depth)

    def forward(self, input_: Tensor) -> Tensor:
        return layernorm_3d(input_, self.weight, self.bias, self.normalized_shape, self.variance_epsilon,
                            self.input_parallel_mode, self.weight_parallel_mode, self.output_parallel_mode,
                            self.input_x_weight_parallel_mode)


class Linear3D(nn.Module):

    def __init__(self, in_features: int, out_features: int, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1),
                 activation: Optional[str] = None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.activation = activation
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.output_x_weight_parallel_mode = get_output_x_weight_parallel_mode()
        self.depth = get_depth_from_env()
        self.in_features_per_partition = in_features // self.depth
        self.out_features_per_partition = out_features // self.depth ** 2
        self.bias_features_per_partition = out_features // self.depth
        self.weight = Parameter(torch.empty(self.in_features_per_partition, self.out_features_per_partition))
        self.bias = Parameter(torch.zeros(self.bias_features_per_partition)) if bias else None
        with seed(pm.TENSOR):
            weight_initializer(self.weight, fan_in=in_features, fan_out=out_features)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        set_tensor_parallel_attribute_by_partition(self.weight, self.depth ** 3)
        if self.bias is not None:
            set_tensor_parallel_attribute_by_partition(self.bias, self.depth)
        swap_in_out_group()

    def forward(self, input_: Tensor) -> Tensor:
        return linear_3d(input_, self.weight, self.bias, self.input_parallel_mode, self.weight_parallel_mode,
                         self.output_parallel_mode, self.activation)


class Classifier3D(nn.Module):

    def __init__(self, in_features: int, num_classes: int, weight: Parameter = None, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.num_classes = num_classes
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.depth = get_depth_from_env()
        self.in_features_per_partition = in_features // self.depth
        if weight is not None:
            self.weight = weight
            self.has_weight = False
        else:
            self.weight = Parameter(torch.empty(num_classes, self.in_features_per_partition))
            self.has_weight = True
        self.bias = Parameter(torch.zeros(num_classes)) if bias else None
        with seed(pm.TENSOR):
            if self.has_weight:
                weight_initializer(self.weight, fan_in=in_features, fan_out=num_classes)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        if self.has_weight:
            set_tensor_parallel_attribute_by_partition(self.weight, self.depth)

    def forward(self, input_: Tensor) -> Tensor:
        return classifier_3d(input_, self.weight, self.bias, self.input_parallel_mode, self.weight_parallel_mode,
                             self.output_parallel_mode)


class VocabParallelClassifier3D(nn.Module):

    def __init__(self, in_features: int, num_classes: int, weight: Parameter = None, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.num_classes = num_classes
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.output_x_weight_parallel_mode = get_output_x_weight_parallel_mode()
        self.depth = get_depth_from_env()
        self.in_features_per_partition = in_features // self.depth
        self.out_features_per_partition = num_classes // self.depth ** 2
        self.bias_features_per_partition = num_classes // self.depth
        if weight is not None:
            self.weight = weight
            self.has_weight = False
        else:
            self.weight = Parameter(torch.empty(self.out_features_per_partition, self.in_features_per_partition))
            self.has_weight = True
        self.bias = Parameter(torch.zeros(self.bias_features_per_partition)) if bias else None
        with seed(pm.TENSOR):
            if self.has_weight:
                weight_initializer(self.weight, fan_in=in_features, fan_out=num_classes)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        if self.has_weight:
            set_tensor_parallel_attribute_by_partition(self.weight, self.depth ** 3)
        if self.bias is not None:
            set_tensor_parallel_attribute_by_partition(self.bias, self.depth)
        swap_in_out_group()
        env.vocab_parallel = True

    def forward(self, input_: Tensor) -> Tensor:
        return vocab_parallel_classifier_3d(input_, self.weight, self.bias, self.input_parallel_mode,
                                            self.weight_parallel_mode, self.output_parallel_mode)
