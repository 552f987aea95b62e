"""Tensor-parallel-aware gradient-norm clipping: `cubework.utils.clip_grad_norm`
(cubework/utils/clip_grad.py:16-70 of the reference) on the multi-tensor HIP kernels.

Same signature, same arithmetic: per-parameter |g|^p sums, those of parameters tagged with
NUM_PARTITIONS weighted by their partition count and all-reduced over the tensor-parallel group
(identity at size 1) then divided by its size, the root, the clamped coefficient
max_norm / (norm + 1e-6) applied to every gradient without a host round trip. The reference
launches one norm kernel and one multiply per parameter; here all gradients of one dtype go
through two launches per 48 tensors.
"""
import ctypes
from typing import Iterable, Union

import torch
from torch import Tensor

from . import _lib, ops
from .distributed import ParallelManager as pm
from .distributed import all_reduce
from .global_vars import NUM_PARTITIONS

inf = float("inf")


def _tables(grads):
    n = len(grads)
    ptrs = (ctypes.c_void_p * max(n, 1))()
    numels = (ctypes.c_int64 * max(n, 1))()
    for i, g in enumerate(grads):
        ptrs[i] = g.data_ptr()
        numels[i] = g.numel()
    return ptrs, numels


def _norm_partials(grads, factors, groups, norm_type):
    """(standard, tensor-parallel) partial results of the gradients of one dtype, as a [2] fp32 tensor."""
    lib = _lib.load()
    ptrs, numels = _tables(grads)
    n = len(grads)
    fac = (ctypes.c_float * max(n, 1))(*factors)
    grp = (ctypes.c_ubyte * max(n, 1))(*groups)
    dev = grads[0].device
    out = torch.empty(2, dtype=torch.float32, device=dev)
    ws_bytes = lib.cw_multi_norm_workspace_bytes(n, ctypes.cast(numels, ctypes.c_void_p))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.cw_multi_norm_partials(n, ptrs, ctypes.cast(numels, ctypes.c_void_p), ctypes.cast(fac, ctypes.c_void_p),
                                    ctypes.cast(grp, ctypes.c_void_p), norm_type, out.data_ptr(), ws.data_ptr(),
                                    ws_bytes, ops._dtype_code(grads[0]), ops._stream())
    _lib.check(rc, "cw_multi_norm_partials")
    return out


def _scale(grads, coef):
    lib = _lib.load()
    ptrs, numels = _tables(grads)
    rc = lib.cw_multi_scale(len(grads), ptrs, ctypes.cast(numels, ctypes.c_void_p), coef.data_ptr(),
                            ops._dtype_code(grads[0]), ops._stream())
    _lib.check(rc, "cw_multi_scale")


def clip_grad_norm(parameters: Union[Tensor, Iterable[Tensor]], max_norm: float, norm_type: float = 2.0,
                   error_if_nonfinite: bool = False) -> Tensor:
    if isinstance(parameters, Tensor):
        parameters = [parameters]
    parameters = [p for p in parameters if p.grad is not None]
    max_norm = float(max_norm)
    norm_type = float(norm_type)
    if len(parameters) == 0:
        return torch.tensor(0.0)
    device = parameters[0].grad.device
    by_dtype = {}
    for p in parameters:
        g = p.grad.detach()
        if not g.is_cuda:
            raise RuntimeError("clip_grad_norm: gradients must live on the GPU (there is no CPU path)")
        if not g.is_contiguous():
            raise RuntimeError("clip_grad_norm: gradients must be contiguous")
        parts = getattr(p, NUM_PARTITIONS, 0)
        by_dtype.setdefault(g.dtype, []).append((g, float(parts) if parts > 0 else 1.0, 1 if parts > 0 else 0))
    std = tp = None
    for items in by_dtype.values():
        out = _norm_partials([g for g, _, _ in items], [f for _, f, _ in items], [k for _, _, k in items], norm_type)
        if norm_type == inf:
            std = out[0] if std is None else torch.maximum(std, out[0])
            tp = out[1] if tp is None else torch.maximum(tp, out[1])
        else:
            std = out[0] if std is None else std + out[0]
            tp = out[1] if tp is None else tp + out[1]
    if norm_type == inf:
        total_norm = torch.maximum(std, tp)
        if pm.TENSOR.is_initialized() and pm.TENSOR.world_size > 1:
            total_norm = all_reduce(total_norm, pm.TENSOR, op="max")
    else:
        if pm.TENSOR.is_initialized() and pm.TENSOR.world_size > 1:
            tp = all_reduce(tp, pm.TENSOR) / pm.TENSOR.world_size
        total_norm = (std + tp) ** (1.0 / norm_type)
    if error_if_nonfinite and torch.logical_or(total_norm.isnan(), total_norm.isinf()):
        raise RuntimeError(f"The total norm of order {norm_type} for gradients from `parameters` is non-finite, so it "
                           "cannot be clipped. To disable this error and scale the gradients by the non-finite norm "
                           "anyway, set `error_if_nonfinite=False`")
    clip_coef_clamped = torch.clamp(max_norm / (total_norm + 1e-6), max=1.0).to(torch.float32).reshape(1).contiguous()
    for items in by_dtype.values():
        _scale([g for g, _, _ in items], clip_coef_clamped)
    return total_norm.to(device)
