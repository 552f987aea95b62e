"""2D (SUMMA) operators: one rank's math of the reference's autograd Functions
(cubework/module/parallel_2d/_operation.py), each forward/backward being one
or two calls into the HIP library.

Differences from the reference, by design:
  * the q k-steps of SUMMA are ONE kernel launch: the operands the row/column
    broadcasts deliver are collected first (from the mailbox of the
    single-process ParallelMode) and cw_gemm_ksteps accumulates over all of
    them in fp32; C is rounded once, not after every step (_operation.py:41,47);
  * bias add (and, optionally, the activation that follows the layer) are the
    GEMM's epilogue instead of separate elementwise passes (_operation.py:273);
  * partial products a `reduce` would sum (_operation.py:123,202) enter the
    epilogue as addends.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

from ... import ops
from ...distributed import ParallelMode, all_gather, all_reduce, broadcast, reduce_scatter
from .._amp import bwd, fp32_fwd, gemm_fwd
from ..._lib import CW_LN_ONE_PASS


def _flat(t: Tensor) -> Tensor:
    return t.reshape(-1, t.shape[-1])


class _SUMMA_AB(torch.autograd.Function):
    """C = act(sum_i A_i B_i + bias). _SUMMA_AB.forward (_operation.py:18-57)
    fused with _SUMMAbias.forward (:256-274) and the activation."""

    @staticmethod
    @gemm_fwd()
    def forward(ctx, A, B, bias, summa_dim, out_shape, row_parallel_mode, col_parallel_mode, activation, residual=None):
        assert A.shape[-1] == B.shape[-2], "Invalid shapes: A={}, B={} for AB.".format(A.shape, B.shape)
        if residual is not None and activation is not None:
            raise ValueError("a residual addend and a fused activation cannot be combined: the addend would be "
                             "added before the activation")
        A2, B2 = _flat(A), _flat(B)
        A_steps = [broadcast(A2, row_parallel_mode.rank_by_idx(i), row_parallel_mode) for i in range(summa_dim)]
        B_steps = [broadcast(B2, col_parallel_mode.rank_by_idx(i), col_parallel_mode) for i in range(summa_dim)]
        bias_full = None if bias is None else all_gather(bias, -1, col_parallel_mode)
        # ReLU needs no separate pre-activation: its derivative [pre > 0] is [out > 0], so the output serves
        need_pre = activation is not None and activation != "relu"
        addends = () if residual is None else (residual.reshape(-1, out_shape[-1]),)
        res = ops.gemm_ksteps("NN", A_steps, B_steps, bias_full, activation, addends=addends, want_preact=need_pre)
        out, pre = res if need_pre else (res, None)
        if activation == "relu":
            pre = out
        ctx.save_for_backward(A, B, pre)
        ctx.meta = (summa_dim, row_parallel_mode, col_parallel_mode, activation, bias is not None,
                    None if bias is None else bias.dtype, A.shape, B.shape)
        return out.reshape(out_shape)

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        A, B, pre = ctx.saved_tensors
        summa_dim, row_mode, col_mode, activation, has_bias, bias_dtype, A_shape, B_shape = ctx.meta
        g = _flat(output_grad)
        bias_grad = None
        # with nobody to sum the column sums with, they are stored in the parameter's dtype at once (no cast launch);
        # across ranks the fp32 sums are reduced first and rounded once afterwards
        sum_dtype = bias_dtype if has_bias and col_mode.world_size == 1 else None
        with torch.no_grad():
            if activation is not None:
                g, dbias = ops.act_bwd_colsum(activation, g, pre, want_dbias=has_bias, out_dtype=sum_dtype)
            elif has_bias:
                dbias = ops.colsum(g, out_dtype=sum_dtype)
            if has_bias:
                bias_grad = reduce_scatter(dbias, -1, col_mode).to(bias_dtype)
            g = g.reshape(output_grad.shape)
            A_grad = summa_ABT(g, B, summa_dim, A_shape, row_mode, col_mode) if ctx.needs_input_grad[0] else None
            B_grad = summa_ATB(A, g, summa_dim, B_shape, row_mode, col_mode) if ctx.needs_input_grad[1] else None
        residual_grad = output_grad if len(ctx.needs_input_grad) > 8 and ctx.needs_input_grad[8] else None
        return A_grad, B_grad, bias_grad, None, None, None, None, None, residual_grad


def summa_AB(A: Tensor, B: Tensor, summa_dim: int, out_shape: Tuple[int, ...], row_parallel_mode: ParallelMode,
             col_parallel_mode: ParallelMode) -> Tensor:
    """Reference signature (_operation.py:83-91)."""
    return _SUMMA_AB.apply(A, B, None, summa_dim, out_shape, row_parallel_mode, col_parallel_mode, None, None)


def summa_AB_bias_act(A: Tensor, B: Tensor, bias: Optional[Tensor], summa_dim: int, out_shape: Tuple[int, ...],
                      row_parallel_mode: ParallelMode, col_parallel_mode: ParallelMode,
                      activation: Optional[str] = None, residual: Optional[Tensor] = None) -> Tensor:
    """summa_AB + add_bias_2d (+ activation, or + a residual of the output's shape) in one kernel."""
    return _SUMMA_AB.apply(A, B, bias, summa_dim, out_shape, row_parallel_mode, col_parallel_mode, activation, residual)


class _SUMMA_ABT(torch.autograd.Function):
    """C = A B^T (_operation.py:97-136): per step i the rank multiplies by the
    column broadcast B_i; the product of step i == my column is mine (plus the
    row peers' products for it), the others belong to the peers."""

    @staticmethod
    @gemm_fwd()
    def forward(ctx, A, B, summa_dim, out_shape, row_parallel_mode, col_parallel_mode):
        assert A.shape[-1] == B.shape[-1], "Invalid shapes: A={}, B={} for ABT.".format(A.shape, B.shape)
        ctx.save_for_backward(A, B)
        A2, B2 = _flat(A), _flat(B)
        C = None
        for i in range(summa_dim):
            B_i = broadcast(B2, col_parallel_mode.rank_by_idx(i), col_parallel_mode)
            if i == row_parallel_mode.local_rank:
                peers = row_parallel_mode.take("reduce") if row_parallel_mode.world_size > 1 else ()
                C = ops.gemm_ksteps("NT", [A2], [B_i], addends=peers)
            else:
                row_parallel_mode.post("reduce", (i, ops.gemm_ksteps("NT", [A2], [B_i])))
        ctx.meta = (summa_dim, row_parallel_mode, col_parallel_mode, A.shape, B.shape)
        return C.reshape(out_shape)

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        A, B = ctx.saved_tensors
        summa_dim, row_mode, col_mode, A_shape, B_shape = ctx.meta
        with torch.no_grad():
            A_grad = summa_AB(output_grad, B, summa_dim, A_shape, row_mode, col_mode)
            B_grad = summa_ATB(output_grad, A, summa_dim, B_shape, row_mode, col_mode)
        return A_grad, B_grad, None, None, None, None


def summa_ABT(A: Tensor, B: Tensor, summa_dim: int, out_shape: Tuple[int, ...], row_parallel_mode: ParallelMode,
              col_parallel_mode: ParallelMode) -> Tensor:
    return _SUMMA_ABT.apply(A, B, summa_dim, out_shape, row_parallel_mode, col_parallel_mode)


class _SUMMA_ATB(torch.autograd.Function):
    """C = A^T B (_operation.py:177-215): per step i the row broadcast A_i is
    multiplied into this rank's B; step i == my row is mine (plus the column
    peers' products)."""

    @staticmethod
    @gemm_fwd()
    def forward(ctx, A, B, summa_dim, out_shape, row_parallel_mode, col_parallel_mode):
        assert A.shape[-2] == B.shape[-2], "Invalid shapes: A={}, B={} for ATB.".format(A.shape, B.shape)
        ctx.save_for_backward(A, B)
        A2, B2 = _flat(A), _flat(B)
        C = None
        for i in range(summa_dim):
            A_i = broadcast(A2, row_parallel_mode.rank_by_idx(i), row_parallel_mode)
            if i == col_parallel_mode.local_rank:
                peers = col_parallel_mode.take("reduce") if col_parallel_mode.world_size > 1 else ()
                C = ops.gemm_ksteps("TN", [A_i], [B2], addends=peers)
            else:
                col_parallel_mode.post("reduce", (i, ops.gemm_ksteps("TN", [A_i], [B2])))
        ctx.meta = (summa_dim, row_parallel_mode, col_parallel_mode, A.shape, B.shape)
        return C.reshape(out_shape)

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        A, B = ctx.saved_tensors
        summa_dim, row_mode, col_mode, A_shape, B_shape = ctx.meta
        with torch.no_grad():
            A_grad = summa_ABT(B, output_grad, summa_dim, A_shape, row_mode, col_mode)
            B_grad = summa_AB(A, output_grad, summa_dim, B_shape, row_mode, col_mode)
        return A_grad, B_grad, None, None, None, None


def summa_ATB(A: Tensor, B: Tensor, summa_dim: int, out_shape: Tuple[int, ...], row_parallel_mode: ParallelMode,
              col_parallel_mode: ParallelMode) -> Tensor:
    return _SUMMA_ATB.apply(A, B, summa_dim, out_shape, row_parallel_mode, col_parallel_mode)


class _SUMMAbias(torch.autograd.Function):
    """Stand-alone bias op (_operation.py:253-288): gathers the [out/q^2] shards
    over the column group; returns the gathered bias (skip_bias_add) or
    input + bias."""

    @staticmethod
    @gemm_fwd()
    def forward(ctx, input_, bias, row_parallel_mode, col_parallel_mode, skip_bias_add):
        bias_temp = all_gather(bias, -1, col_parallel_mode)
        ctx.meta = (col_parallel_mode, skip_bias_add, bias.dtype)
        if skip_bias_add:
            return bias_temp.clone() if bias_temp is bias else bias_temp
        return ops.bias_act(input_, bias_temp, None)

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        col_mode, skipped, bias_dtype = ctx.meta
        if skipped:
            return None, reduce_scatter(output_grad, -1, col_mode), None, None, None
        dbias = ops.colsum(_flat(output_grad), out_dtype=bias_dtype if col_mode.world_size == 1 else None)
        return output_grad, reduce_scatter(dbias, -1, col_mode).to(bias_dtype), None, None, None


def add_bias_2d(input_: Optional[Tensor], bias: Tensor, row_parallel_mode: ParallelMode,
                col_parallel_mode: ParallelMode, skip_bias_add: bool) -> Tensor:
    return _SUMMAbias.apply(input_, bias, row_parallel_mode, col_parallel_mode, skip_bias_add)


class _Layernorm2D(torch.autograd.Function):
    """LayerNorm2D.forward (parallel_2d/module.py:142-171) and
    _Layernorm_2D.backward (_operation.py:330-347) as one operator:
    partial (sum x, sum x^2) -> [all_reduce over the row group] -> normalise
    with the gathered gamma/beta; backward: partial (sum g, sum g*x_hat) +
    dgamma/dbeta column sums -> [all_reduce] -> dx."""

    @staticmethod
    @fp32_fwd()
    def forward(ctx, input_, weight, bias, hidden_size, eps, row_parallel_mode, col_parallel_mode, fork_residual=False):
        gamma = all_gather(weight, -1, col_parallel_mode)
        beta = all_gather(bias, -1, col_parallel_mode)
        if row_parallel_mode.world_size == 1:
            out, mean_rstd = ops.ln_forward_fused(input_, eps, gamma, beta, mode=CW_LN_ONE_PASS)
        else:
            stats = all_reduce(ops.ln_partial_stats(input_, CW_LN_ONE_PASS), row_parallel_mode)
            out, mean_rstd = ops.ln_normalize(input_, stats, hidden_size, eps, gamma, beta, mode=CW_LN_ONE_PASS)
        ctx.save_for_backward(input_, gamma, mean_rstd)
        ctx.meta = (hidden_size, row_parallel_mode, col_parallel_mode, weight.dtype, bias.dtype)
        if fork_residual:
            # the input goes out again beside the result, for the residual branch around the layers that follow:
            # the gradients of the two branches then meet in this operator's backward, where the kernel that writes
            # dx adds the residual branch's in the same pass, instead of in an accumulation pass of autograd
            return out, input_.view_as(input_)
        return out

    @staticmethod
    @bwd()
    def backward(ctx, output_grad, residual_grad=None):
        x, gamma, mean_rstd = ctx.saved_tensors
        hidden_size, row_mode, col_mode, w_dtype, b_dtype = ctx.meta
        # dgamma / dbeta: fp32 sums, stored in the parameters' dtype at once where no reduce-scatter follows
        pd = w_dtype if col_mode.world_size == 1 and w_dtype == b_dtype else None
        with torch.no_grad():
            if row_mode.world_size == 1:
                input_grad, dgamma, dbeta = ops.ln_backward_fused(output_grad, x, mean_rstd, gamma, param_dtype=pd,
                                                                  dx_addend=residual_grad)
                residual_grad = None
            else:
                # the dx launch also finishes the column sums that the first launch leaves as partial rows
                row_sums, pending = ops.ln_bwd_partials_open(output_grad, x, mean_rstd, gamma)
                row_sums = all_reduce(row_sums, row_mode)
                input_grad, dgamma, dbeta = ops.ln_bwd_dx_close(output_grad, x, mean_rstd, row_sums, hidden_size, pending,
                                                                gamma, param_dtype=pd)
            if residual_grad is not None:
                input_grad = input_grad + residual_grad
            weight_grad = reduce_scatter(dgamma, -1, col_mode).to(w_dtype)
            bias_grad = reduce_scatter(dbeta, -1, col_mode).to(b_dtype)
        return input_grad, weight_grad, bias_grad, None, None, None, None, None


def layernorm_2d(input_: Tensor, weight: Tensor, bias: Tensor, hidden_size: int, eps: float,
                 row_parallel_mode: ParallelMode, col_parallel_mode: ParallelMode, fork_residual: bool = False):
    """fork_residual (additive option, default off): returns (normalised, input) - see _Layernorm2D.forward."""
    return _Layernorm2D.apply(input_, weight, bias, hidden_size, eps, row_parallel_mode, col_parallel_mode, fork_residual)


class _Classifier2D(torch.autograd.Function):
    """C = all_reduce(A W^T) + bias with W gathered over the column group
    (_operation.py:364-419); the peers' products enter as epilogue addends."""

    @staticmethod
    @gemm_fwd()
    def forward(ctx, A, B, bias, summa_dim, out_shape, row_parallel_mode, col_parallel_mode):
        A2 = _flat(A)
        B_temp = all_gather(_flat(B), -1, col_parallel_mode)
        peers = row_parallel_mode.take("all_reduce") if row_parallel_mode.world_size > 1 else ()
        C = ops.gemm_ksteps("NT", [A2], [B_temp], bias, None, addends=peers)
        ctx.save_for_backward(A2, B_temp)
        ctx.meta = (row_parallel_mode, col_parallel_mode, A.shape, B.shape, bias is not None,
                    None if bias is None else bias.dtype)
        return C.reshape(out_shape)

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        A2, B_temp = ctx.saved_tensors
        row_mode, col_mode, A_shape, B_shape, use_bias, bias_dtype = ctx.meta
        g = _flat(output_grad)
        with torch.no_grad():
            A_grad = ops.gemm_ksteps("NN", [g], [B_temp]).reshape(A_shape)
            B_grad = ops.gemm_ksteps("TN", [g], [A2])
            B_grad = reduce_scatter(B_grad, -1, col_mode).reshape(B_shape)
            sum_dtype = bias_dtype if use_bias and col_mode.world_size == 1 else None
            bias_grad = all_reduce(ops.colsum(g, out_dtype=sum_dtype), col_mode).to(bias_dtype) if use_bias else None
        return A_grad, B_grad, bias_grad, None, None, None, None


def classifier_2d(A: Tensor, B: Tensor, bias: Optional[Tensor], summa_dim: int, out_shape: Tuple[int, ...],
                  row_parallel_mode: ParallelMode, col_parallel_mode: ParallelMode) -> Tensor:
    return _Classifier2D.apply(A, B, bias, summa_dim, out_shape, row_parallel_mode, col_parallel_mode)
