"""1D (Megatron) operators. The per-rank compute of every 1D layer is
F.linear(x, W[out, in], b) (cubework/module/parallel_1d/module.py:147,209,269,338)
and its autograd; here it is the NT block GEMM with the bias in the epilogue,
dX = dY W (NN), dW = dY^T X (TN), db = column sums. The Megatron mapping
Functions (cubework/module/parallel_1d/_utils.py:52-126) keep their
forward/backward pairing and go through the single-process collectives.
"""
from typing import Optional

import torch
from torch import Tensor

from ... import ops
from ...distributed import all_gather, all_reduce
from ...global_vars import env
from .._amp import bwd, gemm_fwd
from ..utils import split_tensor


def set_parallel_input(input_parallel: bool):
    env.parallel_input_1d = input_parallel


def get_parallel_input():
    return env.parallel_input_1d


class _LinearNT(torch.autograd.Function):
    @staticmethod
    @gemm_fwd()
    def forward(ctx, input_, weight, bias, activation):
        x2 = input_.reshape(-1, input_.shape[-1])
        # ReLU needs no separate pre-activation: its derivative [pre > 0] is [out > 0], so the output serves
        need_pre = activation is not None and activation != "relu"
        res = ops.gemm_ksteps("NT", [x2], [weight], bias, activation, want_preact=need_pre)
        out, pre = res if need_pre else (res, None)
        if activation == "relu":
            pre = out
        ctx.save_for_backward(x2, weight, pre)
        ctx.meta = (input_.shape, activation, bias is not None, None if bias is None else bias.dtype)
        return out.reshape(input_.shape[:-1] + (weight.shape[0],))

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        x2, weight, pre = ctx.saved_tensors
        in_shape, activation, has_bias, bias_dtype = ctx.meta
        g = output_grad.reshape(-1, output_grad.shape[-1])
        dbias = None
        with torch.no_grad():
            if activation is not None:
                g, dbias = ops.act_bwd_colsum(activation, g, pre, want_dbias=has_bias, out_dtype=bias_dtype)
            elif has_bias:
                dbias = ops.colsum(g, out_dtype=bias_dtype)   # fp32 sums stored in the parameter's dtype: no cast launch
            dx = ops.gemm_ksteps("NN", [g], [weight]).reshape(in_shape) if ctx.needs_input_grad[0] else None
            dw = ops.gemm_ksteps("TN", [g], [x2]) if ctx.needs_input_grad[1] else None
        return dx, dw, dbias, None


def linear_nt(input_: Tensor, weight: Tensor, bias: Optional[Tensor] = None,
              activation: Optional[str] = None) -> Tensor:
    """F.linear(input_, weight, bias) (+ fused activation) on the HIP path."""
    return _LinearNT.apply(input_, weight, bias, activation)


class _ReduceGrad(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, parallel_mode):
        ctx.mode = parallel_mode
        return input_

    @staticmethod
    def backward(ctx, grad_output):
        return all_reduce(grad_output, ctx.mode), None


class _ReduceInput(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, parallel_mode):
        return all_reduce(input_, parallel_mode)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


class _SplitForwardGatherBackward(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, parallel_mode, dim):
        ctx.mode, ctx.dim = parallel_mode, dim
        return split_tensor(input_, dim, parallel_mode) if parallel_mode.world_size > 1 else input_

    @staticmethod
    def backward(ctx, grad_output):
        return all_gather(grad_output, ctx.dim, ctx.mode), None, None


class _GatherForwardSplitBackward(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, parallel_mode, dim):
        ctx.mode, ctx.dim = parallel_mode, dim
        return all_gather(input_, dim, parallel_mode)

    @staticmethod
    def backward(ctx, grad_output):
        g = split_tensor(grad_output, ctx.dim, ctx.mode) if ctx.mode.world_size > 1 else grad_output
        return g, None, None


def reduce_grad(input_, parallel_mode):
    return _ReduceGrad.apply(input_, parallel_mode)


def reduce_input(input_, parallel_mode):
    return _ReduceInput.apply(input_, parallel_mode)


def split_forward_gather_backward(input_, parallel_mode, dim):
    return _SplitForwardGatherBackward.apply(input_, parallel_mode, dim)


def gather_forward_split_backward(input_, parallel_mode, dim):
    return _GatherForwardSplitBackward.apply(input_, parallel_mode, dim)
