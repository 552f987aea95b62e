"""Helpers shared by the parity tests."""
import torch

# Parity bars: relative to the largest magnitude of the expected result.
# float16 carries 11 significand bits (one rounding of an fp32 sum: 2.4e-4 relative to the value).
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-3}

# (what, dtype, achieved error, bar) of every assert_parity call of the session; tests/conftest.py prints the
# largest error-to-bar ratios at the end of the run and writes the whole list to $CW_PARITY_LOG when set.
PARITY_LOG = []


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got = got.detach().to("cpu").to(torch.float64)
    want = want.detach().to("cpu").to(torch.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if want.numel() == 0:
        return 0.0
    denom = max(want.abs().max().item(), 1e-30)
    return (got - want).abs().max().item() / denom


def assert_parity(got, want, dtype, what="", bar=None):
    """Largest |got - want| relative to the largest |want| against the bar of `dtype`, or against `bar`
    when a comparison has a reason, written beside it, for another one. The achieved error is logged."""
    assert torch.isfinite(got.detach().float().cpu()).all(), "%s: non-finite values" % what
    err = rel_err(got, want)
    tol = bar if bar is not None else TOL[dtype]
    PARITY_LOG.append((what, str(dtype).replace("torch.", ""), err, tol))
    assert err <= tol, "%s: relative error %.3e above %.1e" % (what, err, tol)
    return err


def randn(shape, dtype, seed, std=1.0, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype).to(device)


def rand_uniform(shape, dtype, seed, lo, hi, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(shape, generator=g) * (hi - lo) + lo).to(dtype).to(device)
