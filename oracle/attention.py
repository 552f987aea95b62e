"""Oracle for the attention core of the OPT decoder layer. Test infrastructure
only (see oracle/__init__.py).

Reference statements followed (benchmark/opt/opt.py, OPTAttention.forward):
  :72-76   qkv [b, s, heads, 3*d] -> permute (0,2,1,3) -> chunk into q, k, v [b, heads, s, d]
  :84      query_states * self.scaling          (scaling = d ** -0.5, :52)
  :89      attn_weights = bmm(q, k^T)
  :99-100  + attention_mask, clamped at finfo.min (the decoder passes the causal mask, :372-381)
  :107     softmax over the key axis
  :117     attn_output = bmm(attn_probs, v)
  :123-128 -> [b, s, heads*d]
Dropout (:115) has probability 0 in the workload; head masks and cached keys
are not part of the training path.
"""
import math

import torch


from ._precision import to_compute as _f


def split_qkv(qkv: torch.Tensor, heads: int):
    """[b, s, heads*3*d] -> q, k, v as [b, heads, s, d] (opt.py:72-76)."""
    b, s, w = qkv.shape
    d = w // (3 * heads)
    t = qkv.reshape(b, s, heads, 3 * d).permute(0, 2, 1, 3)
    return torch.chunk(t, 3, dim=-1)


def attention_core(q, k, v, scale=None, causal=True, return_lse=False):
    """softmax(scale * q k^T + mask) v in the compute type on [b, heads, s, d] inputs; returns [b, s, heads*d]
    (and the natural-log sum of exponentials [b, heads, s])."""
    q, k, v = _f(q), _f(k), _f(v)
    b, h, s, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    w = torch.matmul(q * scale, k.transpose(-1, -2))
    if causal:
        mask = torch.full((s, s), float("-inf"), dtype=w.dtype).triu(1)
        w = w + mask
    lse = torch.logsumexp(w, dim=-1)
    p = torch.softmax(w, dim=-1)
    o = torch.matmul(p, v).transpose(1, 2).reshape(b, s, h * d)
    return (o, lse) if return_lse else o


def attention_core_backward(q, k, v, d_out, scale=None, causal=True):
    """(dq, dk, dv) of attention_core by the closed form of the softmax-matmul chain:
    dV = P^T dO;  dP = dO V^T;  dS = P * (dP - rowsum(dP * P));  dQ = scale dS K;  dK = scale dS^T Q."""
    q, k, v = _f(q), _f(k), _f(v)
    b, h, s, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    do = _f(d_out).reshape(b, s, h, d).transpose(1, 2)
    w = torch.matmul(q * scale, k.transpose(-1, -2))
    if causal:
        w = w + torch.full((s, s), float("-inf"), dtype=w.dtype).triu(1)
    p = torch.softmax(w, dim=-1)
    dv = torch.matmul(p.transpose(-1, -2), do)
    dp = torch.matmul(do, v.transpose(-1, -2))
    ds = p * (dp - (dp * p).sum(dim=-1, keepdim=True))
    dq = torch.matmul(ds, k) * scale
    dk = torch.matmul(ds.transpose(-1, -2), q) * scale
    return dq, dk, dv


def attention_brute_force(q, k, v, scale, causal):
    """Pure-Python float64 loops, for tiny inputs: pins attention_core."""
    b, h, s, d = q.shape
    q, k, v = q.double().tolist(), k.double().tolist(), v.double().tolist()
    out = torch.zeros((b, s, h * d), dtype=torch.float64)
    for bi in range(b):
        for hi in range(h):
            for i in range(s):
                last = i if causal else s - 1
                sc = [scale * sum(q[bi][hi][i][c] * k[bi][hi][j][c] for c in range(d)) for j in range(last + 1)]
                mx = max(sc)
                e = [math.exp(x - mx) for x in sc]
                z = sum(e)
                for c in range(d):
                    out[bi, i, hi * d + c] = sum(e[j] * v[bi][hi][j][c] for j in range(last + 1)) / z
    return out
