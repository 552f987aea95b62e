"""An OPT decoder layer built from the drop-in layers, used as the shape
source of the "OPT-1.3B-shaped block" workload (hidden 2048, 32 heads, FFN
8192).

Structure of benchmark/opt/opt.py:45-211 of the reference (OPTAttention +
OPTDecoderLayer, pre-LayerNorm variant, dropout 0): LayerNorm -> qkv Linear ->
causal attention -> out Linear -> residual -> LayerNorm -> fc1 -> activation ->
fc2 -> residual. The four Linears and two LayerNorms are cubework_amd.module
layers (HIP path). The attention core (scaled QK^T, causal mask, softmax, PV:
benchmark/opt/opt.py:84-117) is the fused HIP kernel pair cw_attn_fwd /
cw_attn_bwd for 16-bit inputs and head sizes up to 128 (64 and 128 natively, the 48 of
opt_125m and the 80 of opt_2_7b / opt_13b zero-padded, benchmark/opt/opt.py:419-495); fp32
inputs or larger heads use torch's scaled_dot_product_attention, as model code would.
"""

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import module as cube_nn
from . import ops
from .module.parallel_2d import LayerNorm2D, Linear2D


class OPTBlock(nn.Module):

    def __init__(self, hidden: int = 2048, heads: int = 32, ffn: int = 8192, dtype=None,
                 activation: str = "relu", fuse_activation: bool = True):
        super().__init__()
        self.hidden, self.heads, self.head_dim = hidden, heads, hidden // heads
        self.activation = activation
        self.fuse_activation = fuse_activation
        self.self_attn_layer_norm = cube_nn.LayerNorm(hidden, dtype=dtype)
        self.qkv_proj = cube_nn.Linear(hidden, 3 * hidden, dtype=dtype)
        self.out_proj = cube_nn.Linear(hidden, hidden, dtype=dtype)
        self.final_layer_norm = cube_nn.LayerNorm(hidden, dtype=dtype)
        fc1_kwargs = {"activation": activation} if fuse_activation else {}
        self.fc1 = cube_nn.Linear(hidden, ffn, dtype=dtype, **fc1_kwargs)
        self.fc2 = cube_nn.Linear(ffn, hidden, dtype=dtype)

    def _attention_core(self, qkv: torch.Tensor) -> torch.Tensor:
        if self.head_dim <= 128 and qkv.dtype in (torch.bfloat16, torch.float16) and qkv.is_cuda:
            return ops.attention_core(qkv, self.heads)
        b, s, _ = qkv.shape
        qkv = qkv.view(b, s, self.heads, 3 * self.head_dim).permute(0, 2, 1, 3)
        q, k, v = torch.chunk(qkv, 3, dim=-1)
        o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return o.transpose(1, 2).reshape(b, s, self.heads * self.head_dim)

    @staticmethod
    def _linear_plus(layer, inp: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        """residual + layer(inp) (benchmark/opt/opt.py:184,206): in the GEMM's epilogue where the layer offers it
        (Linear2D's `residual` option), as a separate addition elsewhere."""
        inner = getattr(layer, "linear", layer)
        # not under autocast: the operator would cast the residual stream to the 16-bit type with its other inputs
        if (isinstance(inner, Linear2D) and inner.activation is None and not inner.skip_bias_add
                and residual.dtype == inp.dtype == inner.weight.dtype and not torch.is_autocast_enabled("cuda")):
            return layer(inp, residual=residual)
        return residual + layer(inp)

    @staticmethod
    def _norm_fork(layer, x: torch.Tensor):
        """(layer(x), x for the residual branch): through LayerNorm2D's `fork_residual` option where the layer is
        one, so that the two branches' gradients are added inside its backward kernel."""
        inner = getattr(layer, "norm", layer)
        if isinstance(inner, LayerNorm2D) and x.dtype == inner.weight.dtype and not torch.is_autocast_enabled("cuda"):
            return layer(x, fork_residual=True)
        return layer(x), x

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        h, x = self._norm_fork(self.self_attn_layer_norm, x)
        x = self._linear_plus(self.out_proj, self._attention_core(self.qkv_proj(h)), x)
        shape = x.shape
        r = x.reshape(-1, shape[-1])
        h, r = self._norm_fork(self.final_layer_norm, r)
        h = self.fc1(h)
        if not self.fuse_activation:
            h = _ACT[self.activation](h)
        return self._linear_plus(self.fc2, h, r).view(shape)


_ACT = {"relu": F.relu, "gelu": F.gelu, "gelu_erf": F.gelu, "gelu_tanh": lambda t: F.gelu(t, approximate="tanh")}
