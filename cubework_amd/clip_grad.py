"""Tensor-parallel-aware gradient-norm clipping: `cubework.utils.clip_grad_norm`
(cubework/utils/clip_grad.py:16-70 of the reference) on the multi-tensor HIP kernels.

Same signature, same arithmetic: per-parameter |g|^p sums, those of parameters tagged with
NUM_PARTITIONS weighted by their partition count and all-reduced over the tensor-parallel group
(identity at size 1) then divided by its size, the root, the clamped coefficient
max_norm / (norm + 1e-6) applied to every gradient without a host round trip. The reference
launches one norm kernel and one multiply per parameter; here all gradients of one dtype go
through two launches per 48 tensors: the norm stage and the scaling, which works the coefficient
out of the norm stage's results itself.
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


class _DtypeSet:
    """The gradients of one dtype with their host tables, built once per clipping call."""

    def __init__(self, items):
        grads = [g for g, _, _ in items]
        self.n = n = len(grads)
        self.ptrs = (ctypes.c_void_p * n)(*[g.data_ptr() for g in grads])
        self.numels = (ctypes.c_int64 * n)(*[g.numel() for g in grads])
        self.numels_p = ctypes.cast(self.numels, ctypes.c_void_p)
        self._factors = (ctypes.c_float * n)(*[f for _, f, _ in items])
        self._groups = (ctypes.c_ubyte * n)(*[k for _, _, k in items])
        self.factors = ctypes.cast(self._factors, ctypes.c_void_p)
        self.groups = ctypes.cast(self._groups, ctypes.c_void_p)
        self.dtype_code = ops._dtype_code(grads[0])
        self.partials = _lib.load().cw_multi_norm_partial_count(n, self.numels_p)


def _norm_partials(st, norm_type, out_ptr, ws_ptr, ws_bytes, stream):
    """Norm stage of one dtype: block partials into the workspace and, unless out_ptr is None, their
    (standard, tensor-parallel) combination into the [2] fp32 array at out_ptr."""
    rc = _lib.load().cw_multi_norm_partials(st.n, st.ptrs, st.numels_p, st.factors, st.groups, norm_type, out_ptr, ws_ptr,
                                            ws_bytes, st.dtype_code, stream)
    if rc != 0:
        _lib.check(rc, "cw_multi_norm_partials")


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
        g = p.grad
        if not g.is_cuda:
            raise RuntimeError("clip_grad_norm: gradients must live on the GPU (there is no CPU path)")
        if not g.is_contiguous():
            raise RuntimeError("clip_grad_norm: gradients must be contiguous")
        parts = getattr(p, NUM_PARTITIONS, 0)
        item = (g, float(parts), 1) if parts > 0 else (g, 1.0, 0)
        same = by_dtype.get(g.dtype)
        if same is None:
            by_dtype[g.dtype] = [item]
        else:
            same.append(item)
    sets_of = [_DtypeSet(items) for items in by_dtype.values()]
    lib = _lib.load()
    stream = ops._stream()
    norm_coef = torch.empty(2, dtype=torch.float32, device=device)
    n_partials = sum(st.partials for st in sets_of)
    ws = torch.empty(max(n_partials, 1) * 2, dtype=torch.float32, device=device)
    exchange = pm.TENSOR.is_initialized() and pm.TENSOR.world_size > 1
    if not exchange:
        # no peers to ask: the scaling launch finishes the block partials itself (two launches per dtype)
        offset = 0
        for st in sets_of:
            _norm_partials(st, norm_type, None, ws.data_ptr() + 8 * offset, 8 * max(st.partials, 1), stream)
            offset += st.partials
        n_sets, sets_ptr, partials_ptr, tp_scale = 0, None, ws.data_ptr(), 1.0
    else:
        sets = torch.empty((len(sets_of), 2), dtype=torch.float32, device=device)
        for i, st in enumerate(sets_of):
            _norm_partials(st, norm_type, sets[i].data_ptr(), ws.data_ptr(), 8 * max(st.partials, 1), stream)
        # the peers' share: maximum of everything, or sum of the tensor-parallel column divided by the group size
        tp_scale = 1.0
        if norm_type == inf:
            sets = all_reduce(sets.amax().reshape(1), pm.TENSOR, op="max").expand(2).reshape(1, 2).contiguous()
        else:
            sets = sets.sum(0, keepdim=True)
            sets[0, 1] = all_reduce(sets[0, 1].clone(), pm.TENSOR)
            tp_scale = 1.0 / pm.TENSOR.world_size
        n_sets, sets_ptr, partials_ptr, n_partials = sets.shape[0], sets.data_ptr(), None, 0
    if error_if_nonfinite:
        # the check comes before any gradient is touched, so the coefficient needs a launch of its own
        if not exchange:
            sets = torch.empty((len(sets_of), 2), dtype=torch.float32, device=device)
            for i, st in enumerate(sets_of):
                _norm_partials(st, norm_type, sets[i].data_ptr(), ws.data_ptr(), 8 * max(st.partials, 1), stream)
            n_sets, sets_ptr, partials_ptr, n_partials = sets.shape[0], sets.data_ptr(), None, 0
        rc = lib.cw_clip_coef(n_sets, sets_ptr, tp_scale, norm_type, max_norm, norm_coef.data_ptr(), stream)
        _lib.check(rc, "cw_clip_coef")
        total_norm = norm_coef[0]
        if torch.logical_or(total_norm.isnan(), total_norm.isinf()):
            raise RuntimeError(f"The total norm of order {norm_type} for gradients from `parameters` is non-finite, so it "
                               "cannot be clipped. To disable this error and scale the gradients by the non-finite norm "
                               "anyway, set `error_if_nonfinite=False`")
    for st in sets_of:
        rc = lib.cw_clip_scale(st.n, st.ptrs, st.numels_p, st.dtype_code, n_sets, sets_ptr, n_partials, partials_ptr,
                               tp_scale, norm_type, max_norm, norm_coef.data_ptr(), stream)
        if rc != 0:
            _lib.check(rc, "cw_clip_scale")
    return norm_coef[0]
