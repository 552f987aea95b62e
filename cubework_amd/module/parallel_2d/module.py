"""2D (SUMMA) layers with the reference's constructor / forward signatures,
parameter names and shard shapes (cubework/module/parallel_2d/module.py):

  Linear2D                  weight [in/q, out/q]      bias [out/q^2]     (:25-111)
  LayerNorm2D               weight, bias [hidden/q^2]                    (:114-171)
  Classifier2D              weight [classes, in/q^2]  bias [classes]     (:358-423)
  VocabParallelClassifier2D weight [classes/q, in/q]  bias [classes/q^2] (:426-506)

The arithmetic runs in the HIP library (see _operation.py); `activation` on
Linear2D is an additive option (default off) that fuses the activation which
follows the layer in the models (benchmark/gpt2/gpt2.py:116-117).
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
from ._operation import add_bias_2d, classifier_2d, layernorm_2d, summa_AB, summa_AB_bias_act, summa_ABT
from ._utils import assert_summa_initialization, get_summa_dim_from_env


class Linear2D(nn.Module):

    def __init__(self, in_features: int, out_features: int, bias: bool = True, skip_bias_add: bool = False,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1),
                 activation: Optional[str] = None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.skip_bias_add = skip_bias_add
        self.activation = activation
        if activation is not None and skip_bias_add:
            raise ValueError("a fused activation needs the bias added inside the layer (skip_bias_add=False)")

        assert_summa_initialization()
        self.row_rank = pm.PARALLEL_2D_COL.local_rank
        self.col_rank = pm.PARALLEL_2D_ROW.local_rank
        self.summa_dim = get_summa_dim_from_env()
        self.input_size_per_partition = in_features // self.summa_dim
        self.hidden_size_per_partition = out_features // self.summa_dim

        self.weight = Parameter(torch.empty(self.input_size_per_partition, self.hidden_size_per_partition))
        if bias:
            self.bias = Parameter(torch.empty(out_features // self.summa_dim ** 2))
        else:
            self.register_parameter("bias", None)
        with seed(pm.TENSOR):
            self.reset_parameters(weight_initializer, bias_initializer)
        self._set_tensor_parallel_attributes()

    def _set_tensor_parallel_attributes(self):
        set_tensor_parallel_attribute_by_partition(self.weight, self.summa_dim ** 2)
        if self.bias is not None:
            set_tensor_parallel_attribute_by_partition(self.bias, self.summa_dim ** 2)

    def reset_parameters(self, weight_initializer, bias_initializer) -> None:
        weight_initializer(self.weight, fan_in=self.in_features, fan_out=self.out_features)
        if self.bias is not None:
            bias_initializer(self.bias, fan_in=self.in_features)

    def forward(self, x: Tensor, residual: Optional[Tensor] = None):
        """residual (additive option, default off): a tensor of the output's shape that is added to the
        result in the GEMM's epilogue - the `x + layer(...)` that follows the layer in the models
        (benchmark/opt/opt.py:181,207) without a pass of its own."""
        out_shape = x.shape[:-1] + (self.hidden_size_per_partition,)
        row, col = pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL
        if self.bias is not None and self.skip_bias_add:
            if residual is not None:
                raise ValueError("a residual addend needs the bias added inside the layer (skip_bias_add=False)")
            output = summa_AB(x, self.weight, self.summa_dim, out_shape, row, col)
            return output, add_bias_2d(None, self.bias, row, col, True)
        if residual is not None:
            assert residual.shape == out_shape, "residual {} does not match the output {}".format(
                tuple(residual.shape), tuple(out_shape))
        return summa_AB_bias_act(x, self.weight, self.bias, self.summa_dim, out_shape, row, col, self.activation,
                                 residual)


class LayerNorm2D(nn.Module):

    def __init__(self, normalized_shape: int, eps: float = 1e-05):
        super().__init__()
        self.normalized_shape = normalized_shape
        self.variance_epsilon = eps
        assert_summa_initialization()
        self.row_rank = pm.PARALLEL_2D_COL.local_rank
        self.col_rank = pm.PARALLEL_2D_ROW.local_rank
        self.summa_dim = get_summa_dim_from_env()
        self.partitioned_partition = normalized_shape // self.summa_dim ** 2
        self.weight = Parameter(torch.ones(self.partitioned_partition))
        self.bias = Parameter(torch.zeros(self.partitioned_partition))
        set_tensor_parallel_attribute_by_partition(self.weight, self.summa_dim ** 2)
        set_tensor_parallel_attribute_by_partition(self.bias, self.summa_dim ** 2)

    def forward(self, x: Tensor, fork_residual: bool = False):
        """fork_residual (additive option, default off): returns (normalised x, x) for a pre-LayerNorm block whose
        residual branch starts at this layer's input (benchmark/opt/opt.py:170-174, 193-197): take the residual from
        the second result, and the gradients of both branches are summed inside this layer's backward kernel."""
        return layernorm_2d(x, self.weight, self.bias, self.normalized_shape, self.variance_epsilon,
                            pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL, fork_residual)


class Classifier2D(nn.Module):

    def __init__(self, in_features: int, num_classes: int, weight: Parameter = None, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.num_classes = num_classes
        assert_summa_initialization()
        self.row_rank = pm.PARALLEL_2D_COL.local_rank
        self.col_rank = pm.PARALLEL_2D_ROW.local_rank
        self.summa_dim = get_summa_dim_from_env()
        self.input_size_per_partition = in_features // self.summa_dim ** 2
        if weight is not None:
            self.weight = weight
            self.has_weight = False
        else:
            self.weight = Parameter(torch.empty(num_classes, self.input_size_per_partition))
            self.has_weight = True
        self.bias = Parameter(torch.zeros(num_classes)) if bias else None
        self.reset_parameters(weight_initializer, bias_initializer)
        if self.has_weight:
            set_tensor_parallel_attribute_by_partition(self.weight, self.summa_dim ** 2)

    def reset_parameters(self, weight_initializer, bias_initializer) -> None:
        with seed(pm.TENSOR):
            if self.has_weight:
                weight_initializer(self.weight, fan_in=self.in_features, fan_out=self.num_classes)
            if self.bias is not None:
                # the reference then broadcasts the bias from rank 0 of both groups
                # (module.py:403-405): a no-op for the single rank computed here
                bias_initializer(self.bias, fan_in=self.in_features)

    def forward(self, input_: Tensor) -> Tensor:
        out_shape = input_.shape[:-1] + (self.num_classes,)
        return classifier_2d(input_, self.weight, self.bias, self.summa_dim, out_shape, pm.PARALLEL_2D_ROW,
                             pm.PARALLEL_2D_COL)


class VocabParallelClassifier2D(nn.Module):

    def __init__(self, in_features: int, num_classes: int, weight: Parameter = None, bias: bool = True,
                 weight_initializer: Callable = init.kaiming_uniform_(a=math.sqrt(5)),
                 bias_initializer: Callable = init.xavier_uniform_(a=1, scale=1)):
        super().__init__()
        self.in_features = in_features
        self.num_classes = num_classes
        assert_summa_initialization()
        self.row_rank = pm.PARALLEL_2D_COL.local_rank
        self.col_rank = pm.PARALLEL_2D_ROW.local_rank
        self.summa_dim = get_summa_dim_from_env()
        self.input_size_per_partition = in_features // self.summa_dim
        self.output_size_per_partition = num_classes // self.summa_dim
        if weight is not None:
            self.weight = weight
            self.has_weight = False
        else:
            self.weight = Parameter(torch.empty(self.output_size_per_partition, self.input_size_per_partition))
            self.has_weight = True
        self.bias = Parameter(torch.empty(num_classes // self.summa_dim ** 2)) if bias else None
        with seed(pm.TENSOR):
            if self.has_weight:
                weight_initializer(self.weight, fan_in=in_features, fan_out=num_classes)
            if self.bias is not None:
                bias_initializer(self.bias, fan_in=in_features)
        if self.has_weight:
            set_tensor_parallel_attribute_by_partition(self.weight, self.summa_dim ** 2)
        if self.bias is not None:
            set_tensor_parallel_attribute_by_partition(self.bias, self.summa_dim ** 2)
        env.vocab_parallel = True

    def forward(self, x: Tensor) -> Tensor:
        out_shape = x.shape[:-1] + (self.output_size_per_partition,)
        row, col = pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL
        output = summa_ABT(x, self.weight, self.summa_dim, out_shape, row, col)
        if self.bias is not None:
            output = add_bias_2d(output, self.bias, row, col, False)
        return output
