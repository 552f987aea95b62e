"""Autocast policy of the operators.

The reference wraps its GEMM-type Functions in custom_fwd(cast_inputs=float16)
and its LayerNorm / loss Functions in custom_fwd(cast_inputs=float32)
(cubework/module/parallel_2d/_operation.py:17,96,176,255,309,363;
cubework/module/loss/loss_1d.py:13). Here the GEMM-type operators cast to the
dtype the autocast region was opened with: float16 under a plain
torch.autocast("cuda") / torch.cuda.amp.autocast(), which is what the
reference's training scripts use (benchmark/opt/train.py:85-86) and so gives
the reference's dtype, and bfloat16 under torch.autocast("cuda",
dtype=torch.bfloat16), where the reference would still cast to float16.
Outside autocast nothing is cast, as in the reference. The loss keeps
16-bit logits instead of copying them to float32 (loss_fwd below).
"""
import functools

import torch

_GEMM_CAST_DTYPES = (torch.float16, torch.bfloat16)


def gemm_fwd():
    """custom_fwd whose cast_inputs follows the autocast dtype (float16 unless the region asks for bfloat16)."""
    def decorate(fwd):
        variants = {dt: torch.amp.custom_fwd(fwd, device_type="cuda", cast_inputs=dt) for dt in _GEMM_CAST_DTYPES}

        @functools.wraps(fwd)
        def wrapper(*args, **kwargs):
            dt = torch.float16
            if torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") in variants:
                dt = torch.get_autocast_dtype("cuda")
            return variants[dt](*args, **kwargs)
        return wrapper
    return decorate


fp32_fwd = functools.partial(torch.amp.custom_fwd, device_type="cuda", cast_inputs=torch.float32)


def loss_fwd():
    """The loss Function's policy. The reference casts the logits to float32 under autocast
    (custom_fwd(cast_inputs=torch.float32), cubework/module/loss/loss_1d.py:13), a copy twice the size of
    the 16-bit logits a classifier hands over. The kernels read 16-bit logits and compute in fp32, which is
    the same arithmetic on the same values (the cast is exact), so 16-bit logits stay as they are; autocast
    is switched off inside, as custom_fwd does. Other floating types are cast to float32."""
    def decorate(fwd):
        @functools.wraps(fwd)
        def wrapper(ctx, logits, *args, **kwargs):
            ctx._dtype = torch.get_autocast_dtype("cuda")
            ctx._fwd_used_autocast = False  # the body runs with autocast off; custom_bwd gives backward the same state
            if not torch.is_autocast_enabled("cuda"):
                return fwd(ctx, logits, *args, **kwargs)
            if logits.is_floating_point() and logits.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                logits = logits.to(torch.float32)
            with torch.autocast("cuda", enabled=False):
                return fwd(ctx, logits, *args, **kwargs)
        return wrapper
    return decorate


bwd = functools.partial(torch.amp.custom_bwd, device_type="cuda")
