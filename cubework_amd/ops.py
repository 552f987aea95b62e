"""Tensor-level wrappers of the C ABI: check shapes, allocate outputs with torch
(device memory and streams are torch's; the arithmetic is the HIP library's),
pass raw pointers and the current stream.

Every function requires CUDA (ROCm) tensors of dtype bfloat16 or float32 (the
GEMM, column-sum, attention and cross-entropy wrappers also take float16, the
type autocast hands the GEMM-type operators by default) and raises instead of falling back to torch
arithmetic.
"""
import ctypes
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import (CW_ACT_GELU_ERF, CW_ACT_GELU_TANH, CW_ACT_NONE, CW_ACT_RELU, CW_BF16, CW_F16, CW_EPI_BIAS,
                   CW_EPI_BIAS_GELU_ERF, CW_EPI_BIAS_GELU_TANH, CW_EPI_BIAS_RELU, CW_EPI_NONE, CW_F32, CW_LN_ONE_PASS,
                   CW_LN_TWO_PASS, CW_NN, CW_NT, CW_TN)

ACTIVATIONS = {None: CW_ACT_NONE, "none": CW_ACT_NONE, "gelu_tanh": CW_ACT_GELU_TANH, "gelu": CW_ACT_GELU_ERF,
               "gelu_erf": CW_ACT_GELU_ERF, "relu": CW_ACT_RELU}
LAYOUTS = {"NN": CW_NN, "NT": CW_NT, "TN": CW_TN}


def epilogue_code(has_bias: bool, activation: Optional[str]) -> int:
    act = ACTIVATIONS[activation]
    if act == CW_ACT_NONE:
        return CW_EPI_BIAS if has_bias else CW_EPI_NONE
    return {CW_ACT_GELU_TANH: CW_EPI_BIAS_GELU_TANH, CW_ACT_GELU_ERF: CW_EPI_BIAS_GELU_ERF,
            CW_ACT_RELU: CW_EPI_BIAS_RELU}[act]


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return CW_BF16
    if t.dtype == torch.float32:
        return CW_F32
    if t.dtype == torch.float16:
        return CW_F16
    raise TypeError("the cubework_amd kernels take bfloat16, float16 or float32 tensors, got %s" % t.dtype)


def _require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("cubework_amd operators run on the GPU only (got a %s tensor); "
                               "there is no CPU fallback" % t.device)


def _rows(t: torch.Tensor) -> torch.Tensor:
    """View as [rows, cols] with unit column stride (copy only if unavoidable)."""
    if t.dim() != 2:
        t = t.reshape(-1, t.shape[-1])
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    return t


def _ld(t: torch.Tensor) -> int:
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def _stream() -> ctypes.c_void_p:
    # the raw handle of torch's current stream on the current device; torch.cuda.current_stream() builds a
    # Stream object for the same value and costs ten times as much per call
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _ptr_table(tensors: Sequence[torch.Tensor]):
    arr = (ctypes.c_void_p * max(len(tensors), 1))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


# --------------------------------------------------------------------------
# block GEMM
# --------------------------------------------------------------------------
def gemm_ksteps(layout: str, A_steps: Sequence[torch.Tensor], B_steps: Sequence[torch.Tensor],
                bias: Optional[torch.Tensor] = None, activation: Optional[str] = None,
                addends: Sequence[torch.Tensor] = (), want_preact: bool = False,
                out: Optional[torch.Tensor] = None):
    """C = act(sum_i op(A_i) op(B_i) + sum_j addends_j + bias); see cw_gemm_ksteps.

    layout "NN": A_i [M,K], B_i [K,N];  "NT": A_i [M,K], B_i [N,K];  "TN": A_i [K,M], B_i [K,N].
    Returns C, or (C, preact) when want_preact.
    """
    lib = _lib.load()
    if len(A_steps) != len(B_steps) or len(A_steps) == 0:
        raise ValueError("need the same, non-zero number of A and B step operands")
    A_steps = [_rows(a) for a in A_steps]
    B_steps = [_rows(b) for b in B_steps]
    _require_device(*A_steps, *B_steps, bias, *addends)
    a0, b0 = A_steps[0], B_steps[0]
    dt = _dtype_code(a0)
    if layout == "NN":
        M, K, N, Kb = a0.shape[0], a0.shape[1], b0.shape[1], b0.shape[0]
    elif layout == "NT":
        M, K, N, Kb = a0.shape[0], a0.shape[1], b0.shape[0], b0.shape[1]
    elif layout == "TN":
        M, K, N, Kb = a0.shape[1], a0.shape[0], b0.shape[1], b0.shape[0]
    else:
        raise ValueError("layout must be NN, NT or TN")
    if K != Kb:
        raise ValueError("reduction sizes differ: A %s, B %s for %s" % (tuple(a0.shape), tuple(b0.shape), layout))
    for t in list(A_steps) + list(B_steps):
        if t.dtype != a0.dtype:
            raise TypeError("all GEMM operands must share one dtype")
    lda, ldb = _ld(a0), _ld(b0)
    for a in A_steps:
        if a.shape != a0.shape or _ld(a) != lda:
            raise ValueError("A step operands must share shape and leading dimension")
    for b in B_steps:
        if b.shape != b0.shape or _ld(b) != ldb:
            raise ValueError("B step operands must share shape and leading dimension")
    if bias is not None:
        if bias.numel() != N:
            raise ValueError("bias has %d elements, output width is %d" % (bias.numel(), N))
        bias = bias.to(a0.dtype).contiguous()
    addends = [_rows(t) for t in addends]
    for t in addends:
        if tuple(t.shape) != (M, N) or t.dtype != a0.dtype:
            raise ValueError("addends must be [M,N] of the operand dtype")
    ldadd = _ld(addends[0]) if addends else 0
    # the C ABI takes one leading dimension for all addends: copy those that are laid out differently
    addends = [t if _ld(t) == ldadd else t.contiguous() for t in addends]
    if any(_ld(t) != ldadd for t in addends):
        ldadd = N
        addends = [t.contiguous() for t in addends]
    if out is None:
        out = torch.empty((M, N), dtype=a0.dtype, device=a0.device)
    elif tuple(out.shape) != (M, N) or out.dtype != a0.dtype or out.stride(1) != 1:
        raise ValueError("out must be a row-major [M,N] tensor of the operand dtype")
    preact = torch.empty((M, N), dtype=a0.dtype, device=a0.device) if want_preact else None
    epi = epilogue_code(bias is not None, activation)
    ta, tb, tadd = _ptr_table(A_steps), _ptr_table(B_steps), _ptr_table(addends)
    # scratch for the split-k path (few output tiles, long reduction: the weight-gradient shape)
    ws_bytes = lib.cw_gemm_workspace_bytes(LAYOUTS[layout], M, N, K, len(A_steps), dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a0.device) if ws_bytes > 0 else None
    rc = lib.cw_gemm_ksteps_ws(LAYOUTS[layout], M, N, K, len(A_steps), ta, lda, tb, ldb, _p(bias), epi, _p(out),
                               _ld(out), _p(preact), _ld(preact) if preact is not None else 0, tadd, len(addends),
                               ldadd, _p(ws), ws_bytes, dt, _stream())
    _lib.check(rc, "cw_gemm_ksteps_ws")
    return (out, preact) if want_preact else out


def bias_act(x: torch.Tensor, bias: Optional[torch.Tensor], activation: Optional[str] = None) -> torch.Tensor:
    """act(x + bias) as the GEMM epilogue alone (zero k-steps, x as the addend)."""
    lib = _lib.load()
    shape = x.shape
    x2 = _rows(x)
    _require_device(x2, bias)
    M, N = x2.shape
    if bias is not None:
        if bias.numel() != N:
            raise ValueError("bias has %d elements, width is %d" % (bias.numel(), N))
        bias = bias.to(x2.dtype).contiguous()
    out = torch.empty((M, N), dtype=x2.dtype, device=x2.device)
    tadd = _ptr_table([x2])
    rc = lib.cw_gemm_ksteps(CW_NN, M, N, 0, 0, None, 0, None, 0, _p(bias), epilogue_code(bias is not None, activation),
                            _p(out), _ld(out), None, 0, tadd, 1, _ld(x2), _dtype_code(x2), _stream())
    _lib.check(rc, "cw_gemm_ksteps (bias/activation only)")
    return out.reshape(shape)


def _workspace(M: int, N: int, device) -> torch.Tensor:
    nbytes = _lib.load().cw_colsum_workspace_bytes(M, N)
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device)


def _out_dtype(out_dtype: Optional[torch.dtype]) -> torch.dtype:
    """dtype of column-sum results: fp32 unless the caller names the parameter's dtype (the sums are always
    accumulated in fp32 and rounded once on the way out)."""
    out_dtype = out_dtype or torch.float32
    if out_dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TypeError("column sums are stored as float32, bfloat16 or float16, not %s" % out_dtype)
    return out_dtype


_TORCH_CODE = {torch.float32: CW_F32, torch.bfloat16: CW_BF16, torch.float16: CW_F16}


def colsum(dy: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Column sums of a [M,N] tensor (bias gradient): fp32 sums, stored as out_dtype (default float32)."""
    lib = _lib.load()
    dy = _rows(dy)
    _require_device(dy)
    M, N = dy.shape
    out_dtype = _out_dtype(out_dtype)
    out = torch.empty(N, dtype=out_dtype, device=dy.device)
    ws = _workspace(M, N, dy.device)
    rc = lib.cw_colsum(M, N, _p(dy), _ld(dy), _p(out), _TORCH_CODE[out_dtype], _p(ws), ws.numel(), _dtype_code(dy),
                       _stream())
    _lib.check(rc, "cw_colsum")
    return out


def act_bwd_colsum(activation: Optional[str], dy: torch.Tensor, preact: torch.Tensor, want_dbias: bool = True,
                   out_dtype: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """dPre = dy * act'(preact) and (optionally) its column sums (fp32 sums stored as out_dtype, default float32)."""
    lib = _lib.load()
    dy, preact = _rows(dy), _rows(preact)
    _require_device(dy, preact)
    if dy.shape != preact.shape or dy.dtype != preact.dtype:
        raise ValueError("dy and preact must agree in shape and dtype")
    M, N = dy.shape
    dpre = torch.empty((M, N), dtype=dy.dtype, device=dy.device)
    out_dtype = _out_dtype(out_dtype)
    dbias = torch.empty(N, dtype=out_dtype, device=dy.device) if want_dbias else None
    ws = _workspace(M, N, dy.device) if want_dbias else None
    rc = lib.cw_act_bwd_colsum(ACTIVATIONS[activation], M, N, _p(dy), _ld(dy), _p(preact), _ld(preact), _p(dpre),
                               _ld(dpre), _p(dbias), _TORCH_CODE[out_dtype], _p(ws), ws.numel() if ws is not None else 0,
                               _dtype_code(dy), _stream())
    _lib.check(rc, "cw_act_bwd_colsum")
    return dpre, dbias


# --------------------------------------------------------------------------
# LayerNorm
# --------------------------------------------------------------------------
def ln_partial_stats(x: torch.Tensor, mode: int = CW_LN_ONE_PASS, mean: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[R,2] fp32 partial statistics of the local columns of x [R,C]."""
    lib = _lib.load()
    x = _rows(x)
    _require_device(x, mean)
    R, C = x.shape
    stats = torch.empty((R, 2), dtype=torch.float32, device=x.device)
    if mean is not None:
        mean = mean.reshape(-1).to(torch.float32).contiguous()
        if mean.numel() != R:
            raise ValueError("mean must have one entry per row")
    rc = lib.cw_ln_partial_stats(R, C, _p(x), _ld(x), mode, _p(mean), _p(stats), _dtype_code(x), _stream())
    _lib.check(rc, "cw_ln_partial_stats")
    return stats


def ln_normalize(x: torch.Tensor, stats: torch.Tensor, hidden: int, eps: float,
                 gamma: Optional[torch.Tensor] = None, beta: Optional[torch.Tensor] = None,
                 mode: int = CW_LN_ONE_PASS, save_mean_rstd: bool = True):
    """y = gamma*(x-mean)*rstd+beta from whole-hidden-size stats; returns (y, mean_rstd)."""
    lib = _lib.load()
    shape = x.shape
    x = _rows(x)
    _require_device(x, stats, gamma, beta)
    R, C = x.shape
    stats = stats.reshape(R, 2).to(torch.float32).contiguous()
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    beta = None if beta is None else beta.to(x.dtype).contiguous()
    for v in (gamma, beta):
        if v is not None and v.numel() != C:
            raise ValueError("gamma/beta must have C elements")
    y = torch.empty((R, C), dtype=x.dtype, device=x.device)
    mr = torch.empty((R, 2), dtype=torch.float32, device=x.device) if save_mean_rstd else None
    rc = lib.cw_ln_normalize(R, C, _p(x), _ld(x), _p(stats), mode, hidden, eps, _p(gamma), _p(beta), _p(y), _ld(y),
                             _p(mr), _dtype_code(x), _stream())
    _lib.check(rc, "cw_ln_normalize")
    return y.reshape(shape), mr


def ln_forward_fused(x: torch.Tensor, eps: float, gamma: Optional[torch.Tensor] = None,
                     beta: Optional[torch.Tensor] = None, mode: int = CW_LN_ONE_PASS, save_mean_rstd: bool = True):
    """LayerNorm over the last dimension when this rank holds the whole hidden size."""
    lib = _lib.load()
    shape = x.shape
    x = _rows(x)
    _require_device(x, gamma, beta)
    R, C = x.shape
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    beta = None if beta is None else beta.to(x.dtype).contiguous()
    y = torch.empty((R, C), dtype=x.dtype, device=x.device)
    mr = torch.empty((R, 2), dtype=torch.float32, device=x.device) if save_mean_rstd else None
    rc = lib.cw_ln_forward_fused(R, C, _p(x), _ld(x), mode, eps, _p(gamma), _p(beta), _p(y), _ld(y), _p(mr),
                                 _dtype_code(x), _stream())
    _lib.check(rc, "cw_ln_forward_fused")
    return y.reshape(shape), mr


def ln_bwd_partials(dy: torch.Tensor, x: torch.Tensor, mean_rstd: torch.Tensor,
                    gamma: Optional[torch.Tensor] = None, want_param_grads: bool = True,
                    param_dtype: Optional[torch.dtype] = None):
    """Returns (row_sums [R,2] fp32, dgamma [C] or None, dbeta [C] or None); the parameter gradients are fp32
    sums stored as param_dtype (default float32)."""
    lib = _lib.load()
    dy, x = _rows(dy), _rows(x)
    _require_device(dy, x, mean_rstd, gamma)
    if dy.shape != x.shape or dy.dtype != x.dtype:
        raise ValueError("dy and x must agree in shape and dtype")
    R, C = x.shape
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    row_sums = torch.empty((R, 2), dtype=torch.float32, device=x.device)
    dgamma = dbeta = ws = None
    param_dtype = _out_dtype(param_dtype)
    if want_param_grads:
        dgamma = torch.empty(C, dtype=param_dtype, device=x.device)
        dbeta = torch.empty(C, dtype=param_dtype, device=x.device)
        ws = _workspace(R, C, x.device)
    rc = lib.cw_ln_bwd_partials(R, C, _p(dy), _ld(dy), _p(x), _ld(x), _p(mean_rstd), _p(gamma), _p(row_sums),
                                _p(dgamma), _p(dbeta), _TORCH_CODE[param_dtype], _p(ws),
                                ws.numel() if ws is not None else 0, _dtype_code(x), _stream())
    _lib.check(rc, "cw_ln_bwd_partials")
    return row_sums, dgamma, dbeta


def ln_bwd_dx(dy: torch.Tensor, x: torch.Tensor, mean_rstd: torch.Tensor, row_sums: torch.Tensor, hidden: int,
              gamma: Optional[torch.Tensor] = None) -> torch.Tensor:
    lib = _lib.load()
    shape = x.shape
    dy, x = _rows(dy), _rows(x)
    _require_device(dy, x, mean_rstd, row_sums, gamma)
    R, C = x.shape
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    row_sums = row_sums.reshape(R, 2).to(torch.float32).contiguous()
    dx = torch.empty((R, C), dtype=x.dtype, device=x.device)
    rc = lib.cw_ln_bwd_dx(R, C, _p(dy), _ld(dy), _p(x), _ld(x), _p(mean_rstd), _p(gamma), _p(row_sums), hidden,
                          _p(dx), _ld(dx), _dtype_code(x), _stream())
    _lib.check(rc, "cw_ln_bwd_dx")
    return dx.reshape(shape)


def ln_bwd_partials_open(dy: torch.Tensor, x: torch.Tensor, mean_rstd: torch.Tensor,
                         gamma: Optional[torch.Tensor] = None):
    """Row sums [R,2] fp32 now, the parameter gradients later: returns (row_sums, pending), where `pending`
    goes to ln_bwd_dx_close after the row sums have been summed over the ranks. See cw_ln_bwd_partials_open."""
    lib = _lib.load()
    dy, x = _rows(dy), _rows(x)
    _require_device(dy, x, mean_rstd, gamma)
    if dy.shape != x.shape or dy.dtype != x.dtype:
        raise ValueError("dy and x must agree in shape and dtype")
    R, C = x.shape
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    row_sums = torch.empty((R, 2), dtype=torch.float32, device=x.device)
    ws = _workspace(R, C, x.device)
    n_parts = ctypes.c_int64(0)
    rc = lib.cw_ln_bwd_partials_open(R, C, _p(dy), _ld(dy), _p(x), _ld(x), _p(mean_rstd), _p(gamma), _p(row_sums), _p(ws),
                                     ws.numel(), ctypes.cast(ctypes.byref(n_parts), ctypes.c_void_p), _dtype_code(x),
                                     _stream())
    _lib.check(rc, "cw_ln_bwd_partials_open")
    return row_sums, (ws, n_parts.value)


def ln_bwd_dx_close(dy: torch.Tensor, x: torch.Tensor, mean_rstd: torch.Tensor, row_sums: torch.Tensor, hidden: int,
                    pending, gamma: Optional[torch.Tensor] = None, param_dtype: Optional[torch.dtype] = None):
    """(dx, dgamma [C], dbeta [C]): ln_bwd_dx whose launch also finishes the column sums that
    ln_bwd_partials_open left pending (stored as param_dtype, default float32). See cw_ln_bwd_dx_close."""
    lib = _lib.load()
    shape = x.shape
    dy, x = _rows(dy), _rows(x)
    _require_device(dy, x, mean_rstd, row_sums, gamma)
    R, C = x.shape
    ws, n_parts = pending
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    row_sums = row_sums.reshape(R, 2).to(torch.float32).contiguous()
    dx = torch.empty((R, C), dtype=x.dtype, device=x.device)
    param_dtype = _out_dtype(param_dtype)
    dgamma = torch.empty(C, dtype=param_dtype, device=x.device)
    dbeta = torch.empty(C, dtype=param_dtype, device=x.device)
    rc = lib.cw_ln_bwd_dx_close(R, C, _p(dy), _ld(dy), _p(x), _ld(x), _p(mean_rstd), _p(gamma), _p(row_sums), hidden,
                                _p(dx), _ld(dx), _p(ws), n_parts, _p(dgamma), _p(dbeta), _TORCH_CODE[param_dtype],
                                _dtype_code(x), _stream())
    _lib.check(rc, "cw_ln_bwd_dx_close")
    return dx.reshape(shape), dgamma, dbeta


def ln_backward_fused(dy: torch.Tensor, x: torch.Tensor, mean_rstd: torch.Tensor,
                      gamma: Optional[torch.Tensor] = None, want_param_grads: bool = True,
                      param_dtype: Optional[torch.dtype] = None, dx_addend: Optional[torch.Tensor] = None):
    """Backward of LayerNorm over rows this rank holds whole: (dx, dgamma [C] or None, dbeta [C] or None) in
    one pass over dy and x; the parameter gradients are fp32 sums stored as param_dtype (default float32).
    dx_addend: the gradient reaching x along a residual branch, added to dx in the same pass where the kernel
    offers it (else by a separate addition here). See cw_ln_backward_fused."""
    lib = _lib.load()
    shape = x.shape
    dy, x = _rows(dy), _rows(x)
    _require_device(dy, x, mean_rstd, gamma)
    if dy.shape != x.shape or dy.dtype != x.dtype:
        raise ValueError("dy and x must agree in shape and dtype")
    R, C = x.shape
    gamma = None if gamma is None else gamma.to(x.dtype).contiguous()
    row_sums = torch.empty((R, 2), dtype=torch.float32, device=x.device)
    dx = torch.empty((R, C), dtype=x.dtype, device=x.device)
    dgamma = dbeta = ws = None
    param_dtype = _out_dtype(param_dtype)
    if want_param_grads:
        dgamma = torch.empty(C, dtype=param_dtype, device=x.device)
        dbeta = torch.empty(C, dtype=param_dtype, device=x.device)
        ws = _workspace(R, C, x.device)
    add = None
    if dx_addend is not None:
        add = _rows(dx_addend)
        if add.shape != x.shape or add.dtype != x.dtype:
            raise ValueError("dx_addend must agree with x in shape and dtype")
        _require_device(add)

    def call(a):
        return lib.cw_ln_backward_fused(R, C, _p(dy), _ld(dy), _p(x), _ld(x), _p(mean_rstd), _p(gamma), _p(row_sums), _p(dx),
                                        _ld(dx), _p(a), _ld(a) if a is not None else 0, _p(dgamma), _p(dbeta),
                                        _TORCH_CODE[param_dtype], _p(ws), ws.numel() if ws is not None else 0,
                                        _dtype_code(x), _stream())
    rc = call(add)
    if rc == _lib.CW_ERR_UNSUPPORTED and add is not None:   # a shape of the two-kernel path: add separately
        rc = call(None)
        _lib.check(rc, "cw_ln_backward_fused")
        dx = dx + add
        return dx.reshape(shape), dgamma, dbeta
    _lib.check(rc, "cw_ln_backward_fused")
    return dx.reshape(shape), dgamma, dbeta


# --------------------------------------------------------------------------
# vocab-parallel cross-entropy
# --------------------------------------------------------------------------
def vpce_fwd_local(logits: torch.Tensor, targets: torch.Tensor, vocab_start: int):
    """Returns (max, sumexp, pred, mask) of this rank's slice; each [T]."""
    lib = _lib.load()
    logits = _rows(logits)
    _require_device(logits, targets)
    T, V = logits.shape
    targets = targets.reshape(-1).to(torch.int64).contiguous()
    if targets.numel() != T:
        raise ValueError("one target per logits row is required")
    dev = logits.device
    mx = torch.empty(T, dtype=torch.float32, device=dev)
    se = torch.empty(T, dtype=torch.float32, device=dev)
    pr = torch.empty(T, dtype=torch.float32, device=dev)
    mk = torch.empty(T, dtype=torch.uint8, device=dev)
    rc = lib.cw_vpce_fwd_local(T, V, _p(logits), _ld(logits), _p(targets), vocab_start, _p(mx), _p(se), _p(pr), _p(mk),
                               _dtype_code(logits), _stream())
    _lib.check(rc, "cw_vpce_fwd_local")
    return mx, se, pr, mk


def vpce_finalize(max_all: torch.Tensor, sumexp_all: torch.Tensor, pred_all: torch.Tensor, mask_all: torch.Tensor):
    """Inputs [n_ranks, T]; returns (loss, gmax, gsum), each [T] fp32."""
    lib = _lib.load()
    _require_device(max_all, sumexp_all, pred_all, mask_all)
    n, T = max_all.shape
    max_all, sumexp_all, pred_all = (t.to(torch.float32).contiguous() for t in (max_all, sumexp_all, pred_all))
    mask_all = mask_all.to(torch.uint8).contiguous()
    dev = max_all.device
    loss = torch.empty(T, dtype=torch.float32, device=dev)
    gmax = torch.empty(T, dtype=torch.float32, device=dev)
    gsum = torch.empty(T, dtype=torch.float32, device=dev)
    rc = lib.cw_vpce_finalize(T, n, _p(max_all), _p(sumexp_all), _p(pred_all), _p(mask_all), _p(loss), _p(gmax),
                              _p(gsum), _stream())
    _lib.check(rc, "cw_vpce_finalize")
    return loss, gmax, gsum


def vpce_bwd(logits: torch.Tensor, targets: torch.Tensor, vocab_start: int, gmax: torch.Tensor, gsum: torch.Tensor,
             dloss_rows: Optional[torch.Tensor] = None, dloss_scale: float = 1.0,
             grad_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    lib = _lib.load()
    shape = logits.shape
    logits = _rows(logits)
    _require_device(logits, targets, gmax, gsum, dloss_rows)
    T, V = logits.shape
    targets = targets.reshape(-1).to(torch.int64).contiguous()
    grad_dtype = grad_dtype or logits.dtype
    grad = torch.empty((T, V), dtype=grad_dtype, device=logits.device)
    if dloss_rows is not None:
        dloss_rows = dloss_rows.reshape(-1).to(torch.float32).contiguous()
    rc = lib.cw_vpce_bwd(T, V, _p(logits), _ld(logits), _p(targets), vocab_start, _p(gmax), _p(gsum), _p(dloss_rows),
                         dloss_scale, _p(grad), _ld(grad), _dtype_code(logits), _dtype_code(grad), _stream())
    _lib.check(rc, "cw_vpce_bwd")
    return grad.reshape(shape)


# --------------------------------------------------------------------------
# attention core
# --------------------------------------------------------------------------
def _bshd_strides(t: torch.Tensor):
    """(batch, token, head) strides of a [b, s, h, d] view with unit stride in d."""
    if t.dim() != 4 or t.stride(3) != 1:
        raise ValueError("expected a [batch, tokens, heads, head_dim] view with unit stride in head_dim")
    return t.stride(0), t.stride(1), t.stride(2)


def attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None, causal: bool = True,
             want_lse: bool = False):
    """softmax(scale q k^T + causal mask) v for [b, s, h, d] views (e.g. slices of the qkv projection's
    output); returns [b, s, h*d] (and the [b, h, s] log-sum-exp). See cw_attn_fwd."""
    lib = _lib.load()
    _require_device(q, k, v)
    if q.shape != k.shape or q.shape != v.shape or q.dtype != k.dtype or q.dtype != v.dtype:
        raise ValueError("q, k, v must agree in shape and dtype")
    strides = _bshd_strides(q)
    if _bshd_strides(k) != strides or _bshd_strides(v) != strides:
        raise ValueError("q, k, v must share their strides (views of one projection output)")
    B, S, H, D = q.shape
    scale = D ** -0.5 if scale is None else float(scale)
    out = torch.empty((B, S, H, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, S), dtype=torch.float32, device=q.device) if want_lse else None
    rc = lib.cw_attn_fwd(B, H, S, D, _p(q), _p(k), _p(v), strides[0], strides[1], strides[2], scale, 1 if causal else 0,
                         _p(out), out.stride(0), out.stride(1), out.stride(2), _p(lse), _dtype_code(q), _stream())
    _lib.check(rc, "cw_attn_fwd")
    out = out.view(B, S, H * D)
    return (out, lse) if want_lse else out


def attn_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, d_out: torch.Tensor,
             lse: torch.Tensor, dq: torch.Tensor, dk: torch.Tensor, dv: torch.Tensor,
             scale: Optional[float] = None, causal: bool = True) -> None:
    """Gradients of attn_fwd into the [b, s, h, d] views dq, dk, dv (e.g. slices of one buffer shaped like
    the qkv projection's output). out / d_out: [b, s, h*d] or [b, s, h, d]. See cw_attn_bwd."""
    lib = _lib.load()
    _require_device(q, k, v, out, d_out, lse, dq, dk, dv)
    B, S, H, D = q.shape
    strides = _bshd_strides(q)
    if _bshd_strides(k) != strides or _bshd_strides(v) != strides:
        raise ValueError("q, k, v must share their strides")
    gstrides = _bshd_strides(dq)
    if _bshd_strides(dk) != gstrides or _bshd_strides(dv) != gstrides or dq.shape != q.shape:
        raise ValueError("dq, dk, dv must be [b, s, h, d] views sharing their strides")
    out4 = out.reshape(B, S, H, D)
    dout4 = d_out.reshape(B, S, H, D)
    if dout4.stride(3) != 1 or _bshd_strides(dout4) != _bshd_strides(out4):
        out4, dout4 = out4.contiguous(), dout4.contiguous()
    ostr = _bshd_strides(out4)
    scale = D ** -0.5 if scale is None else float(scale)
    ws_bytes = lib.cw_attn_bwd_workspace_bytes(B, H, S)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    rc = lib.cw_attn_bwd(B, H, S, D, _p(q), _p(k), _p(v), strides[0], strides[1], strides[2], _p(out4), _p(dout4),
                         ostr[0], ostr[1], ostr[2], _p(lse), scale, 1 if causal else 0, _p(dq), _p(dk), _p(dv),
                         gstrides[0], gstrides[1], gstrides[2], _p(ws), ws.numel(), _dtype_code(q), _stream())
    _lib.check(rc, "cw_attn_bwd")


def _attn_padded_head(d: int) -> int:
    """Head size the kernels run at for a model head size d: 64 and 128 are native; smaller ones and those in
    between (the reference's opt_125m has 768 / 16 = 48, opt_2_7b and opt_13b have 80, benchmark/opt/opt.py:419-495)
    are zero-padded up - zero columns add nothing to q.k, and the matching output and gradient columns are dropped."""
    if d in (64, 128):
        return d
    if 0 < d < 64:
        return 64
    if 64 < d < 128:
        return 128
    raise NotImplementedError("attention_core: head size %d (the kernels cover head sizes up to 128)" % d)


def _pad_last(t: torch.Tensor, d: int, dp: int) -> torch.Tensor:
    """[..., n*d] -> [..., n*dp] with every group of d columns followed by dp - d zeros."""
    lead, n = t.shape[:-1], t.shape[-1] // d
    out = t.new_zeros(lead + (n, dp))
    out[..., :d] = t.reshape(lead + (n, d))
    return out.view(lead + (n * dp,))


class _AttentionCore(torch.autograd.Function):
    """qkv [b, s, heads*3*d] (per head: q, k, v side by side, benchmark/opt/opt.py:72-76) -> [b, s, heads*d]."""

    @staticmethod
    def forward(ctx, qkv: torch.Tensor, heads: int, scale: Optional[float], causal: bool):
        b, s, w = qkv.shape
        d = w // (3 * heads)
        dp = _attn_padded_head(d)
        if dp != d:
            scale = d ** -0.5 if scale is None else scale  # of the model's head size, not the padded one
            qkv = _pad_last(qkv, d, dp)
        qkv = qkv if qkv.stride(-1) == 1 else qkv.contiguous()
        t = qkv.view(b, s, heads, 3 * dp) if qkv.is_contiguous() else qkv.reshape(b, s, heads, 3 * dp)
        q, k, v = t[..., :dp], t[..., dp:2 * dp], t[..., 2 * dp:]
        out, lse = attn_fwd(q, k, v, scale, causal, want_lse=True)
        ctx.save_for_backward(t, out, lse)
        ctx.meta = (heads, d, dp, scale, causal)
        if dp != d:
            return out.view(b, s, heads, dp)[..., :d].reshape(b, s, heads * d)
        return out

    @staticmethod
    def backward(ctx, d_out: torch.Tensor):
        t, out, lse = ctx.saved_tensors
        heads, d, dp, scale, causal = ctx.meta
        b, s = t.shape[0], t.shape[1]
        q, k, v = t[..., :dp], t[..., dp:2 * dp], t[..., 2 * dp:]
        g = torch.empty((b, s, heads, 3 * dp), dtype=t.dtype, device=t.device)
        d_out = d_out.contiguous() if dp == d else _pad_last(d_out, d, dp)
        attn_bwd(q, k, v, out, d_out, lse, g[..., :dp], g[..., dp:2 * dp], g[..., 2 * dp:], scale, causal)
        if dp != d:
            return g.view(b, s, heads, 3, dp)[..., :d].reshape(b, s, heads * 3 * d), None, None, None
        return g.view(b, s, heads * 3 * d), None, None, None


def attention_core(qkv: torch.Tensor, heads: int, scale: Optional[float] = None, causal: bool = True) -> torch.Tensor:
    """Differentiable fused attention core on the qkv projection's output."""
    return _AttentionCore.apply(qkv, heads, scale, causal)


# --------------------------------------------------------------------------
# vocab-parallel embedding
# --------------------------------------------------------------------------
def embedding_fwd(ids: torch.Tensor, weight: torch.Tensor, vocab_start: int = 0) -> torch.Tensor:
    """Rows of `weight` ([V_loc, E]) for the ids inside [vocab_start, vocab_start + V_loc), zeros for the
    others; ids of any shape, result ids.shape + (E,). See cw_embed_fwd."""
    lib = _lib.load()
    _require_device(ids, weight)
    if ids.dtype not in (torch.int64, torch.int32):
        raise TypeError("ids must be int64 or int32 (what F.embedding takes), got %s" % ids.dtype)
    w = _rows(weight)
    flat = ids.reshape(-1).to(torch.int64).contiguous()   # a no-op for int64 ids
    T, (V_loc, E) = flat.numel(), w.shape
    out = torch.empty((T, E), dtype=w.dtype, device=w.device)
    rc = lib.cw_embed_fwd(T, E, _p(flat), int(vocab_start), V_loc, _p(w), _ld(w), _p(out), _ld(out), _dtype_code(w),
                          _stream())
    _lib.check(rc, "cw_embed_fwd")
    return out.view(tuple(ids.shape) + (E,))


def embedding_token_order(ids: torch.Tensor, num_rows: int, vocab_start: int = 0):
    """(sorted_ids, order) of the flat int64 ids by the row of the slice they select, ties in token order;
    ids outside the slice come last as vocab_start + num_rows. See cw_embed_sort_ids."""
    lib = _lib.load()
    _require_device(ids)
    if ids.dtype != torch.int64:
        raise TypeError("ids must be int64, got %s" % ids.dtype)
    flat = ids.reshape(-1).contiguous()
    T = flat.numel()
    sorted_ids = torch.empty_like(flat)
    order = torch.empty_like(flat)
    ws_bytes = lib.cw_embed_sort_workspace_bytes(T)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=flat.device) if ws_bytes > 0 else None
    rc = lib.cw_embed_sort_ids(T, _p(flat), int(vocab_start), int(num_rows), _p(sorted_ids), _p(order),
                               _p(ws), ws_bytes, _stream())
    _lib.check(rc, "cw_embed_sort_ids")
    return sorted_ids, order


def embedding_bwd(ids: torch.Tensor, d_out: torch.Tensor, num_rows: int, vocab_start: int = 0,
                  skip_row: int = -1, via_token_order: Optional[bool] = None) -> torch.Tensor:
    """Gradient of embedding_fwd with respect to the [num_rows, E] weight slice: one launch from the unsorted
    ids where cw_embed_bwd_ids_supported says that it pays (up to 16384 tokens, 16-byte aligned rows, rows not
    much smaller than the batch's ids), else the token order followed by cw_embed_bwd. via_token_order = True /
    False asks for one path (False: the one launch wherever it is possible at all)."""
    lib = _lib.load()
    _require_device(ids, d_out)
    if ids.dtype not in (torch.int64, torch.int32):
        raise TypeError("ids must be int64 or int32 (what F.embedding takes), got %s" % ids.dtype)
    g = _rows(d_out.reshape(-1, d_out.shape[-1]))
    flat = ids.reshape(-1).to(torch.int64).contiguous()   # a no-op for int64 ids
    T, E = g.shape
    if flat.numel() != T:
        raise ValueError("ids select %d rows, d_out has %d" % (flat.numel(), T))
    dw = torch.empty((num_rows, E), dtype=g.dtype, device=g.device)
    if via_token_order is None:
        direct = bool(lib.cw_embed_bwd_ids_supported(T, E, _p(g), _ld(g), _p(dw), _ld(dw), _dtype_code(g)))
    else:
        direct = not via_token_order
    if direct:
        rc = lib.cw_embed_bwd_ids(T, E, _p(flat), int(vocab_start), num_rows, int(skip_row), _p(g), _ld(g), _p(dw),
                                  _ld(dw), _dtype_code(g), _stream())
        if rc != _lib.CW_ERR_UNSUPPORTED:
            _lib.check(rc, "cw_embed_bwd_ids")
            return dw
    sorted_ids, order = embedding_token_order(flat, num_rows, vocab_start)
    rc = lib.cw_embed_bwd(T, E, _p(sorted_ids), _p(order), int(vocab_start), num_rows, int(skip_row), _p(g), _ld(g),
                          _p(dw), _ld(dw), _dtype_code(g), _stream())
    _lib.check(rc, "cw_embed_bwd")
    return dw


class _VocabEmbedding(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ids, weight, vocab_start, skip_row):
        ctx.save_for_backward(ids)
        ctx.meta = (weight.shape[0], vocab_start, skip_row)
        return embedding_fwd(ids, weight, vocab_start)

    @staticmethod
    def backward(ctx, d_out):
        (ids,) = ctx.saved_tensors
        rows, vocab_start, skip_row = ctx.meta
        return None, embedding_bwd(ids, d_out, rows, vocab_start, skip_row), None, None


def vocab_embedding(ids: torch.Tensor, weight: torch.Tensor, vocab_start: int = 0,
                    padding_idx: Optional[int] = None) -> torch.Tensor:
    """Differentiable masked embedding lookup of one vocabulary slice. padding_idx is the row of `weight`
    that receives no gradient (what F.embedding's padding_idx means for the tensor it is handed)."""
    skip = -1 if padding_idx is None else int(padding_idx)
    return _VocabEmbedding.apply(ids, weight, int(vocab_start), skip)
