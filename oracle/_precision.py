"""The floating-point type the oracle evaluates the reference's formulas in.

The reference computes in fp32; that is the default here. Parity tests of fp32 kernels evaluate the same
formulas in float64 instead (`with oracle.precision(torch.float64): ...`), so that the expected value
carries no rounding of its own and the whole 1e-5 bar belongs to the kernel under test. Results whose
inputs are 16-bit are rounded once to the input type in either mode; results of fp32 inputs stay in the
compute type. Test infrastructure only (see oracle/__init__.py).
"""
import contextlib

import torch

_state = {"dtype": torch.float32}


def compute_dtype():
    return _state["dtype"]


@contextlib.contextmanager
def precision(dtype):
    if dtype not in (torch.float32, torch.float64):
        raise ValueError("the oracle computes in float32 or float64")
    saved = _state["dtype"]
    _state["dtype"] = dtype
    try:
        yield
    finally:
        _state["dtype"] = saved


def to_compute(t):
    """Detached CPU copy of t in the compute type (None stays None)."""
    return None if t is None else t.detach().to("cpu").to(_state["dtype"])


def round_like(y, like):
    """y rounded once to `like`'s type when that is a 16-bit type; otherwise y in the compute type."""
    if like.dtype in (torch.bfloat16, torch.float16):
        return y.to(like.dtype)
    return y.to(_state["dtype"])
