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


def _norm_partials(grads, factors, groups, norm_type, out):
    """(standard, tensor-parallel) partial results of the gradients of one dtype into the [2] fp32 view `out`."""
    lib = _lib.load()
    ptrs, numels = _tables(grads)
    n = len(grads)
    fac = (ctypes.c_float * max(n, 1))(*factors)
    grp = (ctypes.c_ubyte * max(n, 1))(*groups)
    ws_bytes = lib.cw_multi_norm_workspace_bytes(n, ctypes.cast(numels, ctypes.c_void_p))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=out.device)
    rc = lib.cw_multi_norm_partials(n, ptrs, ctypes.cast(numels, ctypes.c_void_p), ctypes.cast(fac, ctypes.c_void_p),
                                    ctypes.cast(grp, ctypes.c_void_p), norm_type, out.data_ptr(), ws.data_ptr(),
                                    ws_bytes, ops._dtype_code(grads[0]), ops._stream())
    _lib.check(rc, "cw_multi_norm_partials")


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
    sets = torch.empty((len(by_dtype), 2), dtype=torch.float32, device=device)
    for i, items in enumerate(by_dtype.values()):
        _norm_partials([g for g, _, _ in items], [f for _, f, _ in items], [k for _, _, k in items], norm_type, sets[i])
    tp_scale = 1.0
    if pm.TENSOR.is_initialized() and pm.TENSOR.world_size > 1:
        # the peers' share: maximum of everything, or sum of the tensor-parallel column divided by the group size
        if norm_type == inf:
            sets = all_reduce(sets.amax().reshape(1), pm.TENSOR, op="max").expand(2).reshape(1, 2).contiguous()
        else:
            sets = sets.sum(0, keepdim=True)
            sets[0, 1] = all_reduce(sets[0, 1].clone(), pm.TENSOR)
            tp_scale = 1.0 / pm.TENSOR.world_size
    norm_coef = torch.empty(2, dtype=torch.float32, device=device)
    lib = _lib.load()
    rc = lib.cw_clip_coef(sets.shape[0], sets.data_ptr(), tp_scale, norm_type, max_norm, norm_coef.data_ptr(), ops._stream())
    _lib.check(rc, "cw_clip_coef")
    total_norm = norm_coef[0]
    if error_if_nonfinite and torch.logical_or(total_norm.isnan(), total_norm.isinf()):
        raise RuntimeError(f"The total norm of order {norm_type} for gradients from `parameters` is non-finite, so it "
                           "cannot be clipped. To disable this error and scale the gradients by the non-finite norm "
                           "anyway, set `error_if_nonfinite=False`")
    clip_coef_clamped = norm_coef[1:]
    for items in by_dtype.values():
        _scale([g for g, _, _ in items], clip_coef_clamped)
    return total_norm
