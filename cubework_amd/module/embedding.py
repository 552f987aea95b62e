"""Embedding layers of `cubework.module`, on the HIP lookup / scatter kernels.

Mirrors, with the same constructor signatures, parameter names and shard shapes:
  Embedding1D / VocabParallelEmbedding1D   cubework/module/parallel_1d/module.py:349-455
  Embedding2D / VocabParallelEmbedding2D   cubework/module/parallel_2d/module.py:248-355
  Embedding3D / VocabParallelEmbedding3D   cubework/module/parallel_3d/module.py:344-468
  Embedding (mode-dispatching facade)      cubework/module/modules.py:191-236
The lookup is cw_embed_fwd / cw_embed_bwd (ops.vocab_embedding); the collectives
around it (all-gather of the embedding columns, reduce / reduce-scatter of the
vocabulary slices' outputs) go through the single-process stand-ins of
cubework_amd.distributed, identity at tensor-parallel size 1.

F.embedding's extra positional / keyword arguments (max_norm, scale_grad_by_freq,
sparse) are accepted and must be left at their defaults: the kernels do not
implement them and the constructor says so instead of ignoring them.
"""
from typing import Callable, Optional

import torch
from torch import Tensor, nn
from torch.nn import Parameter

from .. import ops
from ..distributed import all_gather, all_reduce, broadcast, reduce_scatter, seed
from ..distributed import ParallelManager as pm
from ..global_vars import env
from . import init
from .parallel_1d._operation import gather_forward_split_backward, reduce_input, set_parallel_input
from .parallel_2d._utils import assert_summa_initialization, get_summa_dim_from_env, split_batch_2d
from .parallel_3d._utils import (get_depth_from_env, get_input_parallel_mode, get_input_x_weight_parallel_mode,
                                 get_output_parallel_mode, get_weight_parallel_mode, split_batch_3d)
from .utils import get_tensor_parallel_mode, set_tensor_parallel_attribute_by_partition, split_tensor


def _check_embed_args(args, kwargs):
    defaults = {"max_norm": None, "norm_type": 2.0, "scale_grad_by_freq": False, "sparse": False}
    names = list(defaults)
    given = dict(zip(names, args))
    given.update(kwargs)
    for k, v in given.items():
        if k not in defaults or v != defaults[k]:
            raise NotImplementedError("F.embedding option %s=%r is not provided by the HIP lookup" % (k, v))


class _AllGatherTensor(torch.autograd.Function):
    """all-gather along `dim` forward, reduce-scatter backward
    (all_gather_tensor_2d, parallel_2d/_operation.py:760-790; all_gather_weight_3d, parallel_3d/_operation.py)."""

    @staticmethod
    def forward(ctx, tensor, dim, mode):
        ctx.dim, ctx.mode = dim, mode
        return all_gather(tensor, dim, mode)

    @staticmethod
    def backward(ctx, grad):
        return reduce_scatter(grad, ctx.dim, ctx.mode), None, None


class _ReduceScatterTensor(torch.autograd.Function):
    """reduce-scatter along `dim` forward, all-gather backward
    (reduce_scatter_tensor_2d, parallel_2d/_operation.py:799-830; reduce_scatter_tensor_3d)."""

    @staticmethod
    def forward(ctx, tensor, dim, mode):
        ctx.dim, ctx.mode = dim, mode
        return reduce_scatter(tensor, dim, mode)

    @staticmethod
    def backward(ctx, grad):
        return all_gather(grad, ctx.dim, ctx.mode), None, None


class _EmbeddingBase(nn.Module):
    """Shared bookkeeping: arguments, padding row, slice bounds."""

    vocab_start_index = 0

    def _setup(self, num_embeddings, embedding_dim, padding_idx, args, kwargs):
        _check_embed_args(args, kwargs)
        self.num_embeddings = num_embeddings
        self.embed_dim = embedding_dim
        self.padding_idx = padding_idx
        self.embed_args = args
        self.embed_kwargs = kwargs

    def _lookup(self, input_: Tensor, weight: Tensor) -> Tensor:
        # F.embedding(shifted ids, weight, padding_idx): padding_idx names a row of the tensor it is handed
        pad = self.padding_idx if (self.padding_idx is not None and 0 <= self.padding_idx < weight.shape[0]) else None
        return ops.vocab_embedding(input_, weight, self.vocab_start_index, pad)


# --------------------------------------------------------------------------------------------- 1D
class Embedding1D(_EmbeddingBase):
    """weight [num_embeddings, embedding_dim / p]; output columns gathered (parallel_1d/module.py:349-394)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int = None,
                 weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        self.weight = Parameter(torch.empty((num_embeddings, embedding_dim // pm.PARALLEL_1D.world_size)))
        with seed(pm.PARALLEL_1D):
            weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
            if padding_idx is not None:
                with torch.no_grad():
                    self.weight[padding_idx].fill_(0)
        set_tensor_parallel_attribute_by_partition(self.weight, pm.PARALLEL_1D.world_size)
        set_parallel_input(False)

    def forward(self, input_: Tensor) -> Tensor:
        return gather_forward_split_backward(self._lookup(input_, self.weight), pm.PARALLEL_1D, dim=-1)


class VocabParallelEmbedding1D(_EmbeddingBase):
    """weight [num_embeddings / p, embedding_dim]; outputs summed over the ranks (parallel_1d/module.py:397-455)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int = None,
                 weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        self.num_embeddings_per_partition = num_embeddings // pm.PARALLEL_1D.world_size
        self.vocab_start_index = pm.PARALLEL_1D.local_rank * self.num_embeddings_per_partition
        self.vocab_end_index = self.vocab_start_index + self.num_embeddings_per_partition
        self.weight = Parameter(torch.empty((self.num_embeddings_per_partition, embedding_dim)))
        with seed(pm.PARALLEL_1D):
            weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
            _zero_padding_row(self)
        set_tensor_parallel_attribute_by_partition(self.weight, pm.PARALLEL_1D.world_size)
        set_parallel_input(False)
        env.vocab_parallel = True

    def forward(self, input_: Tensor) -> Tensor:
        return reduce_input(self._lookup(input_, self.weight), pm.PARALLEL_1D)


def _zero_padding_row(layer):
    p = layer.padding_idx
    if p is not None and layer.vocab_start_index <= p < layer.vocab_end_index:
        with torch.no_grad():
            layer.weight[p - layer.vocab_start_index].fill_(0)


# --------------------------------------------------------------------------------------------- 2D
class Embedding2D(_EmbeddingBase):
    """weight [num_embeddings, embedding_dim / q^2], gathered along the columns of the grid
    (parallel_2d/module.py:248-293)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int = None,
                 weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        assert_summa_initialization()
        self.summa_dim = get_summa_dim_from_env()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        self.weight = Parameter(torch.empty((num_embeddings, embedding_dim // self.summa_dim ** 2)))
        with seed(pm.TENSOR):
            weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
            if padding_idx is not None:
                with torch.no_grad():
                    self.weight[padding_idx].fill_(0)
        set_tensor_parallel_attribute_by_partition(self.weight, self.summa_dim ** 2)

    def forward(self, input_: Tensor) -> Tensor:
        input_ = split_batch_2d(input_)
        weight = _AllGatherTensor.apply(self.weight, -1, pm.PARALLEL_2D_COL)
        return self._lookup(input_, weight)


class VocabParallelEmbedding2D(_EmbeddingBase):
    """weight [num_embeddings / q, embedding_dim / q]; outputs reduce-scattered over the column group
    (parallel_2d/module.py:296-355)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int = None,
                 weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        assert_summa_initialization()
        self.summa_dim = get_summa_dim_from_env()
        self.num_embeddings_per_partition = num_embeddings // self.summa_dim
        self.embed_dim_per_partition = embedding_dim // self.summa_dim
        self.vocab_start_index = pm.PARALLEL_2D_COL.local_rank * self.num_embeddings_per_partition
        self.vocab_end_index = self.vocab_start_index + self.num_embeddings_per_partition
        self.weight = Parameter(torch.empty((self.num_embeddings_per_partition, self.embed_dim_per_partition)))
        with seed(pm.TENSOR):
            weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
            _zero_padding_row(self)
        set_tensor_parallel_attribute_by_partition(self.weight, self.summa_dim ** 2)
        env.vocab_parallel = True

    def forward(self, input_: Tensor) -> Tensor:
        return _ReduceScatterTensor.apply(self._lookup(input_, self.weight), 0, pm.PARALLEL_2D_COL)


# --------------------------------------------------------------------------------------------- 3D
class Embedding3D(_EmbeddingBase):
    """weight [num_embeddings, embedding_dim / depth], replicated over the input x weight group
    (parallel_3d/module.py:344-398)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int = None,
                 weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        self.depth = get_depth_from_env()
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.input_x_weight_parallel_mode = get_input_x_weight_parallel_mode()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        self.weight = Parameter(torch.empty((num_embeddings, embedding_dim // self.depth)))
        with seed(pm.TENSOR):
            weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
            if padding_idx is not None:
                with torch.no_grad():
                    self.weight[padding_idx].fill_(0)
        mode = self.input_x_weight_parallel_mode
        with torch.no_grad():
            self.weight.copy_(broadcast(self.weight.detach(), mode.rank_by_idx(0), mode))
        self.weight.register_hook(lambda grad: all_reduce(grad.clone(), self.input_x_weight_parallel_mode))
        set_tensor_parallel_attribute_by_partition(self.weight, self.depth)

    def forward(self, input_: Tensor) -> Tensor:
        input_ = split_batch_3d(input_, input_parallel_mode=self.input_parallel_mode,
                                weight_parallel_mode=self.weight_parallel_mode)
        return self._lookup(input_, self.weight)


class VocabParallelEmbedding3D(_EmbeddingBase):
    """weight [num_embeddings / depth^2, embedding_dim / depth] (parallel_3d/module.py:401-468)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int = None,
                 weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        self.depth = get_depth_from_env()
        self.input_parallel_mode = get_input_parallel_mode()
        self.weight_parallel_mode = get_weight_parallel_mode()
        self.output_parallel_mode = get_output_parallel_mode()
        self.num_embeddings_per_partition = num_embeddings // self.depth ** 2
        self.embed_dim_per_partition = embedding_dim // self.depth
        span = self.num_embeddings_per_partition * self.depth
        self.vocab_start_index = self.input_parallel_mode.local_rank * span
        self.vocab_end_index = self.vocab_start_index + span
        self.weight = Parameter(torch.empty((self.num_embeddings_per_partition, self.embed_dim_per_partition)))
        with seed(pm.TENSOR):
            weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
            _zero_padding_row(self)
        set_tensor_parallel_attribute_by_partition(self.weight, self.depth ** 3)
        env.vocab_parallel = True

    def forward(self, input_: Tensor) -> Tensor:
        input_ = split_tensor(input_, 0, self.weight_parallel_mode) if self.weight_parallel_mode.world_size > 1 else input_
        weight = _AllGatherTensor.apply(self.weight, 0, self.weight_parallel_mode)
        return _ReduceScatterTensor.apply(self._lookup(input_, weight), 0, self.input_parallel_mode)


# ------------------------------------------------------------------------------------------ facade
_parallel_embedding = {"1d": Embedding1D, "2d": Embedding2D, "3d": Embedding3D}
_vocab_parallel_embedding = {"1d": VocabParallelEmbedding1D, "2d": VocabParallelEmbedding2D,
                             "3d": VocabParallelEmbedding3D}


class _EmbeddingSTD(_EmbeddingBase):
    """No tensor parallelism: the reference wraps nn.Embedding (modules.py:204-206); here the same
    parameter goes through the HIP lookup."""

    def __init__(self, num_embeddings, embedding_dim, padding_idx=None, weight_initializer=init.normal_(), *args,
                 **kwargs):
        super().__init__()
        self._setup(num_embeddings, embedding_dim, padding_idx, args, kwargs)
        self.weight = Parameter(torch.empty((num_embeddings, embedding_dim)))
        weight_initializer(self.weight, fan_in=num_embeddings, fan_out=embedding_dim)
        if padding_idx is not None:
            with torch.no_grad():
                self.weight[padding_idx].fill_(0)

    def forward(self, input_: Tensor) -> Tensor:
        return self._lookup(input_, self.weight)


class Embedding(nn.Module):
    """cubework/module/modules.py:191-236."""

    def __init__(self, num_embeddings: int, embedding_dim: int, vocab_parallel: bool = False, padding_idx: int = None,
                 dtype=None, weight_initializer: Callable = init.normal_(), *args, **kwargs):
        super().__init__()
        mode = get_tensor_parallel_mode()
        if mode is None:
            cls = _EmbeddingSTD
        else:
            cls = (_vocab_parallel_embedding if vocab_parallel else _parallel_embedding)[mode]
        self.embed = cls(num_embeddings, embedding_dim, *args, padding_idx=padding_idx,
                         weight_initializer=weight_initializer, **kwargs).to(dtype)

    def forward(self, *args, **kwargs):
        return self.embed(*args, **kwargs)

    @property
    def weight(self):
        return self.embed.weight
