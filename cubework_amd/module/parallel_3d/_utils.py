"""3D helpers (cubework/module/parallel_3d/_utils.py:12-137): the group
getters read the names held in `env`, which every Linear3D /
VocabParallelClassifier3D construction swaps (input <-> output)."""
import torch
from torch import Tensor

from ...distributed import ParallelManager as pm
from ...distributed import ParallelMode, all_reduce
from ...global_vars import env
from .._amp import bwd, fp32_fwd


def get_depth_from_env() -> int:
    return env.depth_3d


def get_input_parallel_mode() -> ParallelMode:
    return getattr(pm, env.input_group_3d)


def get_weight_parallel_mode() -> ParallelMode:
    return getattr(pm, env.weight_group_3d)


def get_output_parallel_mode() -> ParallelMode:
    return getattr(pm, env.output_group_3d)


def get_input_x_weight_parallel_mode() -> ParallelMode:
    return getattr(pm, env.input_x_weight_group_3d)


def get_output_x_weight_parallel_mode() -> ParallelMode:
    return getattr(pm, env.output_x_weight_group_3d)


def swap_in_out_group():
    env.input_group_3d, env.output_group_3d = env.output_group_3d, env.input_group_3d
    env.input_x_weight_group_3d, env.output_x_weight_group_3d = (env.output_x_weight_group_3d,
                                                                 env.input_x_weight_group_3d)


def split_batch_3d(input_: Tensor, dim: int = 0, input_parallel_mode: ParallelMode = None,
                   weight_parallel_mode: ParallelMode = None) -> Tensor:
    if input_.size(dim) <= 1:
        return input_
    weight_parallel_mode = get_weight_parallel_mode()
    input_parallel_mode = get_input_parallel_mode()
    out = input_
    for mode in (weight_parallel_mode, input_parallel_mode):
        if mode.world_size > 1:
            out = torch.chunk(out, mode.world_size, dim=dim)[mode.local_rank].contiguous()
    return out


class _ReduceByBatch3D(torch.autograd.Function):
    @staticmethod
    @fp32_fwd()
    def forward(ctx, input_, input_parallel_mode, weight_parallel_mode, reduce_mean=False):
        output = all_reduce(all_reduce(input_, input_parallel_mode), weight_parallel_mode)
        ctx.reduce_size = input_parallel_mode.world_size * weight_parallel_mode.world_size if reduce_mean else 1
        return output.clone() / ctx.reduce_size if reduce_mean else output.clone()

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        return output_grad / ctx.reduce_size, None, None, None


def reduce_by_batch_3d(tensor: Tensor, input_parallel_mode: ParallelMode, weight_parallel_mode: ParallelMode,
                       reduce_mean: bool = False) -> Tensor:
    return _ReduceByBatch3D.apply(tensor, input_parallel_mode, weight_parallel_mode, reduce_mean)
