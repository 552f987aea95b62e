"""2D helpers (cubework/module/parallel_2d/_utils.py:12-101)."""
import torch
from torch import Tensor

from ...distributed import ParallelManager as pm
from ...distributed import all_reduce
from ...global_vars import env
from .._amp import bwd, fp32_fwd


def get_summa_dim_from_env() -> int:
    return env.summa_dim


def assert_summa_initialization():
    assert pm.PARALLEL_2D_COL.is_initialized() and pm.PARALLEL_2D_ROW.is_initialized(), \
        "Both TWO_DIMENSION_COL and TWO_DIMENSION_ROW must be initialized by the process group initializer"


def split_batch_2d(input_: Tensor, dim: int = 0) -> Tensor:
    """This rank's batch chunk (identity at world size 1 or for size-1 dims)."""
    if input_.size(dim) <= 1 or pm.PARALLEL_2D_COL.world_size == 1:
        return input_
    return torch.chunk(input_, pm.PARALLEL_2D_COL.world_size, dim=dim)[pm.PARALLEL_2D_COL.local_rank].contiguous()


class _ReduceByBatch2D(torch.autograd.Function):
    @staticmethod
    @fp32_fwd()
    def forward(ctx, input_, reduce_mean: bool = False):
        output = all_reduce(input_, pm.PARALLEL_2D_COL)
        ctx.reduce_size = pm.PARALLEL_2D_COL.world_size if reduce_mean else 1
        return output.clone() / ctx.reduce_size if reduce_mean else output.clone()

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        return output_grad / ctx.reduce_size, None


def reduce_by_batch_2d(input_, reduce_mean: bool = False) -> Tensor:
    """All-reduce over the batch-splitting (column) group, optionally averaged."""
    return _ReduceByBatch2D.apply(input_, reduce_mean)
