"""Oracle for the OPT decoder layer used as the "OPT-1.3B-shaped block" workload: the layer of
benchmark/opt/opt.py:45-211 of the reference (pre-LayerNorm variant, dropout 0) in plain fp32 torch on the
CPU. Test infrastructure only (see oracle/__init__.py).

Pinned by torch library routines (F.layer_norm, F.scaled_dot_product_attention, matmul and their autograd),
the routines the reference's own tests use as their oracle."""
from typing import Dict, Tuple

import torch
import torch.nn.functional as F

from ._precision import compute_dtype

_ACT = {"relu": F.relu, "gelu": F.gelu, "gelu_erf": F.gelu, "gelu_tanh": lambda t: F.gelu(t, approximate="tanh")}


def opt_block_reference(block, x: torch.Tensor, relu_mask=None) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """The same layer in plain torch on the CPU (compute type: fp32 unless oracle.precision says float64), with
    leaf copies of the block's parameters (returned by name so gradients can be compared).
    Weights of the 2D/3D layers are [in, out]; 1D layers keep [out, in].

    relu_mask (optional, bool, the shape of fc1's output): which units the ReLU lets through, instead of
    `fc1 > 0`. ReLU's derivative jumps at 0, so a pre-activation that another arithmetic rounds to the
    other side of 0 flips a whole gradient path; a comparison of gradients hands over the mask of the
    implementation under test, after which both sides differentiate the same piecewise-linear function."""
    ct = compute_dtype()
    x = x.to(ct)
    p = {n: t.detach().cpu().to(ct).clone().requires_grad_(True) for n, t in block.named_parameters()}

    def find(prefix: str, leaf: str) -> torch.Tensor:
        for n, t in p.items():
            if n.startswith(prefix + ".") and n.endswith(leaf):
                return t
        raise KeyError(prefix + "." + leaf)

    def lin(prefix: str, t: torch.Tensor) -> torch.Tensor:
        w, b = find(prefix, "weight"), find(prefix, "bias")
        return t @ w + b if _is_in_out(block, prefix) else F.linear(t, w, b)

    def ln(prefix: str, t: torch.Tensor) -> torch.Tensor:
        return F.layer_norm(t, (t.shape[-1],), find(prefix, "weight"), find(prefix, "bias"), 1e-5)

    heads, hd = block.heads, block.head_dim
    h = ln("self_attn_layer_norm", x)
    qkv = lin("qkv_proj", h)
    b, s, _ = qkv.shape
    qkv = qkv.view(b, s, heads, 3 * hd).permute(0, 2, 1, 3)
    q, k, v = torch.chunk(qkv, 3, dim=-1)
    o = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(b, s, heads * hd)
    x1 = x + lin("out_proj", o)
    pre = lin("fc1", ln("final_layer_norm", x1))
    if relu_mask is not None:
        if block.activation != "relu":
            raise ValueError("relu_mask is for a block whose activation is ReLU")
        h = pre * relu_mask.to(pre.dtype).reshape(pre.shape)
    else:
        h = _ACT[block.activation](pre)
    return x1 + lin("fc2", h), p


def _is_in_out(block, prefix: str) -> bool:
    """True when the layer stores its weight as [in, out] (Linear2D / Linear3D)."""
    inner = getattr(block, prefix).linear
    return type(inner).__name__ in ("Linear2D", "Linear3D")
