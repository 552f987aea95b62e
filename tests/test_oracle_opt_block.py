"""Pins oracle/opt_block.py without the GPU. The layer's structure is that of benchmark/opt/opt.py:135-211
(pre-LayerNorm decoder layer): what a retyped formula would not catch is checked through properties the
structure fixes - the two residual paths, causality of the attention, the [in, out] / [out, in] weight
orientations - and through the other, separately pinned oracle functions (LayerNorm, block GEMM, attention
core) composed by hand."""
import types

import torch
import torch.nn as nn

import oracle
from tests.util import randn


class _Lin(nn.Module):
    def __init__(self, weight, bias, kind):
        super().__init__()
        self.linear = types.new_class(kind, (nn.Module,))()   # the oracle reads the orientation from the class name
        self.linear.weight = nn.Parameter(weight)
        self.linear.bias = nn.Parameter(bias)


class _Norm(nn.Module):
    def __init__(self, h, seed):
        super().__init__()
        self.weight = nn.Parameter(1.0 + 0.1 * randn((h,), torch.float32, seed))
        self.bias = nn.Parameter(0.1 * randn((h,), torch.float32, seed + 1))


def _block(hidden=16, heads=2, ffn=32, kind="Linear2D", activation="gelu_tanh", seed=0):
    blk = nn.Module()
    blk.heads, blk.head_dim, blk.activation = heads, hidden // heads, activation

    def lin(i, o, s):
        w = randn((i, o), torch.float32, s, std=0.2)
        return _Lin(w if kind != "Linear1D_Col" else w.t().contiguous(), 0.1 * randn((o,), torch.float32, s + 1), kind)
    blk.self_attn_layer_norm = _Norm(hidden, seed + 1)
    blk.qkv_proj = lin(hidden, 3 * hidden, seed + 10)
    blk.out_proj = lin(hidden, hidden, seed + 20)
    blk.final_layer_norm = _Norm(hidden, seed + 3)
    blk.fc1 = lin(hidden, ffn, seed + 30)
    blk.fc2 = lin(ffn, hidden, seed + 40)
    return blk


def test_matches_the_composition_of_the_pinned_oracle_functions():
    blk = _block()
    x = randn((2, 7, 16), torch.float32, 5)
    got, _ = oracle.opt_block_reference(blk, x)
    p = dict(blk.named_parameters())
    flat = x.reshape(-1, 16)
    h, _ = oracle.ln_forward_full(flat, p["self_attn_layer_norm.weight"], p["self_attn_layer_norm.bias"], 1e-5)
    qkv = oracle.gemm_ksteps("NN", [h], [p["qkv_proj.linear.weight"]], p["qkv_proj.linear.bias"], None).reshape(2, 7, 48)
    q, k, v = oracle.split_qkv(qkv, 2)
    o = oracle.attention_core(q, k, v, causal=True).reshape(-1, 16)
    x1 = flat + oracle.gemm_ksteps("NN", [o], [p["out_proj.linear.weight"]], p["out_proj.linear.bias"], None)
    h2, _ = oracle.ln_forward_full(x1, p["final_layer_norm.weight"], p["final_layer_norm.bias"], 1e-5)
    f = oracle.gemm_ksteps("NN", [h2], [p["fc1.linear.weight"]], p["fc1.linear.bias"], "gelu_tanh")
    want = x1 + oracle.gemm_ksteps("NN", [f], [p["fc2.linear.weight"]], p["fc2.linear.bias"], None)
    assert torch.allclose(got.detach().reshape(-1, 16), want.detach(), rtol=1e-5, atol=1e-5)


def test_residual_paths_and_causality():
    blk = _block(seed=7)
    with torch.no_grad():   # both branches contribute nothing: the layer is the identity
        for name in ("out_proj", "fc2"):
            getattr(blk, name).linear.weight.zero_()
            getattr(blk, name).linear.bias.zero_()
    x = randn((1, 6, 16), torch.float32, 9)
    y, _ = oracle.opt_block_reference(blk, x)
    assert torch.equal(y.detach(), x)
    blk = _block(seed=11)
    y0, _ = oracle.opt_block_reference(blk, x)
    x2 = x.clone()
    x2[0, 4] += 1.0        # a later token must not reach earlier ones
    y1, _ = oracle.opt_block_reference(blk, x2)
    assert torch.equal(y0[0, :4].detach(), y1[0, :4].detach())
    assert not torch.allclose(y0[0, 4:].detach(), y1[0, 4:].detach())


def test_weight_orientations_agree():
    """The same layer with [in, out] weights (2D / 3D layers) and with [out, in] weights (1D layers)."""
    a, b = _block(kind="Linear2D", seed=3), _block(kind="Linear1D_Col", seed=3)
    x = randn((1, 5, 16), torch.float32, 2)
    ya, _ = oracle.opt_block_reference(a, x)
    yb, _ = oracle.opt_block_reference(b, x)
    assert torch.allclose(ya.detach(), yb.detach(), rtol=1e-6, atol=1e-6)
