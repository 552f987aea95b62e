"""3D operators: one rank's math of cubework/module/parallel_3d/_operation.py.

After the gathers, _Linear3D is X[M,K] W[K,N] + bias with dW = X^T dY,
db = sum dY, dX = dY W^T (:34,39,53,59,65): the NN / TN / NT block GEMMs.
The classifiers use W[classes, in] (NT forward). _Layernorm3D is the two-pass
LayerNorm (:273-281, backward :294-311). The reference's asynchronous
gradient bucket (push_async_grad) has no counterpart: nothing here is
asynchronous, gradients are returned directly.
"""
from typing import Optional

import torch
from torch import Tensor

from ... import ops
from ..._lib import CW_LN_TWO_PASS
from ...distributed import ParallelMode, all_gather, all_reduce, broadcast, reduce, reduce_scatter
from .._amp import bwd, fp32_fwd, gemm_fwd


def _flat(t: Tensor) -> Tensor:
    return t.reshape(-1, t.shape[-1])


class _Linear3D(torch.autograd.Function):

    @staticmethod
    @gemm_fwd()
    def forward(ctx, input_, weight, bias, input_parallel_mode, weight_parallel_mode, output_parallel_mode,
                activation):
        x = all_gather(input_, 0, input_parallel_mode)
        w = all_gather(weight, -1, weight_parallel_mode)
        x2 = _flat(x)
        pre = None
        if output_parallel_mode.world_size == 1:
            # ReLU needs no separate pre-activation: its derivative [pre > 0] is [out > 0], so the output serves
            need_pre = activation is not None and activation != "relu"
            res = ops.gemm_ksteps("NN", [x2], [w], bias, activation, want_preact=need_pre)
            out, pre = res if need_pre else (res, None)
            if activation == "relu":
                pre = out
            out = out.reshape(x.shape[:-1] + (w.shape[-1],))
        else:
            assert activation is None, "a fused activation needs the whole reduction on this rank"
            out = ops.gemm_ksteps("NN", [x2], [w]).reshape(x.shape[:-1] + (w.shape[-1],))
            out = reduce_scatter(out, 0, output_parallel_mode)
            if bias is not None:
                out = ops.bias_act(out, bias, None)
        ctx.save_for_backward(x, w, pre)
        ctx.meta = (input_parallel_mode, weight_parallel_mode, output_parallel_mode, activation, bias is not None,
                    None if bias is None else bias.dtype)
        return out

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        x, w, pre = ctx.saved_tensors
        in_mode, w_mode, out_mode, activation, use_bias, bias_dtype = ctx.meta
        with torch.no_grad():
            g = all_gather(output_grad, 0, out_mode)
            g2 = _flat(g)
            bias_grad = None
            # fp32 column sums, stored in the parameter's dtype at once when nobody else adds to them
            sum_dtype = bias_dtype if use_bias and w_mode.world_size == 1 else None
            if activation is not None:
                g2, dbias = ops.act_bwd_colsum(activation, g2, pre, want_dbias=use_bias, out_dtype=sum_dtype)
            elif use_bias:
                dbias = ops.colsum(g2, out_dtype=sum_dtype)
            if use_bias:
                bias_grad = all_reduce(dbias, w_mode).to(bias_dtype)
            weight_grad = ops.gemm_ksteps("TN", [_flat(x)], [g2])
            weight_grad = reduce_scatter(weight_grad, -1, w_mode)
            input_grad = ops.gemm_ksteps("NT", [g2], [w]).reshape(x.shape)
            input_grad = reduce_scatter(input_grad, 0, in_mode)
        return input_grad, weight_grad, bias_grad, None, None, None, None


def linear_3d(input_: Tensor, weight: Tensor, bias: Optional[Tensor], input_parallel_mode: ParallelMode,
              weight_parallel_mode: ParallelMode, output_parallel_mode: ParallelMode,
              activation: Optional[str] = None) -> Tensor:
    return _Linear3D.apply(input_, weight, bias, input_parallel_mode, weight_parallel_mode, output_parallel_mode,
                           activation)


class _Classifier3D(torch.autograd.Function):

    @staticmethod
    @gemm_fwd()
    def forward(ctx, input_, weight, bias, input_parallel_mode, weight_parallel_mode, output_parallel_mode):
        src_rank = input_parallel_mode.ranks_in_group[output_parallel_mode.local_rank]
        w = broadcast(weight, src_rank, input_parallel_mode)
        x2 = _flat(input_)
        peers = output_parallel_mode.take("all_reduce") if output_parallel_mode.world_size > 1 else ()
        out = ops.gemm_ksteps("NT", [x2], [w], bias, None, addends=peers)
        ctx.save_for_backward(input_, w)
        ctx.meta = (src_rank, input_parallel_mode, weight_parallel_mode, output_parallel_mode, bias is not None,
                    None if bias is None else bias.dtype)
        return out.reshape(input_.shape[:-1] + (w.shape[0],))

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        input_, w = ctx.saved_tensors
        src_rank, in_mode, w_mode, out_mode, use_bias, bias_dtype = ctx.meta
        g2 = _flat(output_grad)
        with torch.no_grad():
            weight_grad = ops.gemm_ksteps("TN", [g2], [_flat(input_)])
            weight_grad = reduce(weight_grad, src_rank, in_mode)
            if in_mode.local_rank == out_mode.local_rank:
                weight_grad = all_reduce(weight_grad, w_mode)
            else:
                weight_grad = None
            bias_grad = None
            if use_bias:
                sum_dtype = bias_dtype if in_mode.world_size == 1 and w_mode.world_size == 1 else None
                bias_grad = all_reduce(all_reduce(ops.colsum(g2, out_dtype=sum_dtype), in_mode), w_mode).to(bias_dtype)
            input_grad = ops.gemm_ksteps("NN", [g2], [w]).reshape(input_.shape)
        return input_grad, weight_grad, bias_grad, None, None, None


def classifier_3d(input_: Tensor, weight: Tensor, bias: Optional[Tensor], input_parallel_mode: ParallelMode,
                  weight_parallel_mode: ParallelMode, output_parallel_mode: ParallelMode) -> Tensor:
    return _Classifier3D.apply(input_, weight, bias, input_parallel_mode, weight_parallel_mode,
                               output_parallel_mode)


class _VocabParallelClassifier3D(torch.autograd.Function):

    @staticmethod
    @gemm_fwd()
    def forward(ctx, input_, weight, bias, input_parallel_mode, weight_parallel_mode, output_parallel_mode):
        x = all_gather(input_, 0, input_parallel_mode)
        x2 = _flat(x)
        if weight_parallel_mode.world_size == 1:
            # weight stays [classes/d^2, in/d]: the NT orientation needs no transpose
            w_t = None
            out = ops.gemm_ksteps("NT", [x2], [weight], bias if output_parallel_mode.world_size == 1 else None)
        else:
            w_t = all_gather(weight.transpose(0, 1), -1, weight_parallel_mode).contiguous()
            out = ops.gemm_ksteps("NN", [x2], [w_t], bias if output_parallel_mode.world_size == 1 else None)
        out = out.reshape(x.shape[:-1] + (out.shape[-1],))
        if output_parallel_mode.world_size > 1:
            out = reduce_scatter(out, 0, output_parallel_mode)
            if bias is not None:
                out = ops.bias_act(out, bias, None)
        ctx.save_for_backward(x, weight if w_t is None else w_t)
        ctx.meta = (input_parallel_mode, weight_parallel_mode, output_parallel_mode, w_t is None, bias is not None,
                    None if bias is None else bias.dtype)
        return out

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        x, w = ctx.saved_tensors
        in_mode, w_mode, out_mode, w_is_nt, use_bias, bias_dtype = ctx.meta
        with torch.no_grad():
            g2 = _flat(all_gather(output_grad, 0, out_mode))
            if w_is_nt:
                weight_grad = ops.gemm_ksteps("TN", [g2], [_flat(x)])             # [classes, in]
                input_grad = ops.gemm_ksteps("NN", [g2], [w]).reshape(x.shape)
            else:
                weight_grad = ops.gemm_ksteps("TN", [_flat(x)], [g2])             # [in, classes]
                weight_grad = reduce_scatter(weight_grad.transpose(0, 1), 0, w_mode)
                input_grad = ops.gemm_ksteps("NT", [g2], [w]).reshape(x.shape)
            sum_dtype = bias_dtype if use_bias and w_mode.world_size == 1 else None
            bias_grad = all_reduce(ops.colsum(g2, out_dtype=sum_dtype), w_mode).to(bias_dtype) if use_bias else None
            input_grad = reduce_scatter(input_grad, 0, in_mode)
        return input_grad, weight_grad, bias_grad, None, None, None


def vocab_parallel_classifier_3d(input_: Tensor, weight: Tensor, bias: Optional[Tensor],
                                 input_parallel_mode: ParallelMode, weight_parallel_mode: ParallelMode,
                                 output_parallel_mode: ParallelMode) -> Tensor:
    return _VocabParallelClassifier3D.apply(input_, weight, bias, input_parallel_mode, weight_parallel_mode,
                                            output_parallel_mode)


class _Layernorm3D(torch.autograd.Function):
    """Two-pass LayerNorm: sum x -> [all_reduce over the output group] -> mean;
    sum (x-mean)^2 -> [all_reduce] -> var; y = gamma (x-mean)/sqrt(var+eps) + beta."""

    @staticmethod
    @fp32_fwd()
    def forward(ctx, input_, weight, bias, normalized_shape, eps, input_parallel_mode, weight_parallel_mode,
                output_parallel_mode, input_x_weight_parallel_mode):
        if output_parallel_mode.world_size == 1:
            out, mean_rstd = ops.ln_forward_fused(input_, eps, weight, bias, mode=CW_LN_TWO_PASS)
        else:
            s = ops.ln_partial_stats(input_, CW_LN_TWO_PASS, None)[:, 0]
            mean = all_reduce(s, output_parallel_mode) / normalized_shape
            sq = ops.ln_partial_stats(input_, CW_LN_TWO_PASS, mean)[:, 1]
            sq = all_reduce(sq, output_parallel_mode)
            stats = torch.stack([mean, sq], dim=-1)
            out, mean_rstd = ops.ln_normalize(input_, stats, normalized_shape, eps, weight, bias, mode=CW_LN_TWO_PASS)
        ctx.save_for_backward(input_, weight, mean_rstd)
        ctx.meta = (normalized_shape, output_parallel_mode, input_x_weight_parallel_mode, weight.dtype, bias.dtype)
        return out

    @staticmethod
    @bwd()
    def backward(ctx, output_grad):
        x, weight, mean_rstd = ctx.saved_tensors
        hidden, out_mode, ixw_mode, w_dtype, b_dtype = ctx.meta
        pd = w_dtype if ixw_mode.world_size == 1 and w_dtype == b_dtype else None
        with torch.no_grad():
            if out_mode.world_size == 1:
                input_grad, dgamma, dbeta = ops.ln_backward_fused(output_grad, x, mean_rstd, weight, param_dtype=pd)
            else:
                # the dx launch also finishes the column sums that the first launch leaves as partial rows
                row_sums, pending = ops.ln_bwd_partials_open(output_grad, x, mean_rstd, weight)
                row_sums = all_reduce(row_sums, out_mode)
                input_grad, dgamma, dbeta = ops.ln_bwd_dx_close(output_grad, x, mean_rstd, row_sums, hidden, pending, weight,
                                                                param_dtype=pd)
            weight_grad = all_reduce(dgamma, ixw_mode).to(w_dtype)
            bias_grad = all_reduce(dbeta, ixw_mode).to(b_dtype)
        return input_grad, weight_grad, bias_grad, None, None, None, None, None, None


def layernorm_3d(input_: Tensor, weight: Tensor, bias: Tensor, normalized_shape: int, eps: float,
                 input_parallel_mode: ParallelMode, weight_parallel_mode: ParallelMode,
                 output_parallel_mode: ParallelMode, input_x_weight_parallel_mode: ParallelMode) -> Tensor:
    return _Layernorm3D.apply(input_, weight, bias, normalized_shape, eps, input_parallel_mode,
                              weight_parallel_mode, output_parallel_mode, input_x_weight_parallel_mode)
