"""GPU parity of the attention core (cw_attn_fwd through the C ABI) against the CPU oracle.
Bar: <= 1e-2 relative (bf16 I/O, fp32 accumulation and softmax)."""
import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu

# The log-sum-exp the forward saves for the backward is stored in fp32 but carries 16-bit accuracy by design: the
# row sum is taken over the probabilities as rounded for the second MFMA product, so that the output's
# normaliser is the sum of exactly the weights that multiplied V. Each term is off by at most one 16-bit
# rounding (2^-8 relative for bf16, 2^-11 for float16), the sum by no more, its logarithm by that much in absolute
# terms; against the largest |lse| of a case (about 3 to 8) that is below the bars here (achieved: 2e-4 / 3e-5).
LSE_BAR = {torch.bfloat16: 1e-3, torch.float16: 1.2e-4}
DEV = "cuda:0"


def _qkv(b, s, h, d, seed, std=1.0):
    """One projection output [b, s, h*3*d] as the reference lays it out (benchmark/opt/opt.py:72-76)."""
    return randn((b, s, h * 3 * d), torch.bfloat16, seed, std=std)


def _views(qkv, h, d):
    b, s, _ = qkv.shape
    t = qkv.view(b, s, h, 3 * d)
    return t[..., :d], t[..., d:2 * d], t[..., 2 * d:]


@pytest.mark.parametrize("shape", [(1, 64, 1), (2, 256, 3), (1, 100, 2), (2, 257, 2), (1, 1, 1), (1, 33, 1),
                                   (1, 640, 2), (1, 1000, 1)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_forward_parity(shape, causal):
    import oracle
    from cubework_amd import ops

    b, s, h = shape
    d = 64
    qkv = _qkv(b, s, h, d, seed=s + h, std=1.5)
    with oracle.precision(torch.float64):
        want, want_lse = oracle.attention_core(*oracle.split_qkv(qkv, h), causal=causal, return_lse=True)
    q, k, v = _views(qkv.to(DEV), h, d)
    got, lse = ops.attn_fwd(q, k, v, causal=causal, want_lse=True)
    torch.cuda.synchronize()
    assert_parity(got, want, torch.bfloat16, "attention out %s causal=%s" % (shape, causal))
    assert_parity(lse, want_lse, torch.float32, "attention lse %s" % (shape,), bar=LSE_BAR[torch.bfloat16])


def test_attention_rows_are_convex_combinations():
    """With V = 1 every output is exactly 1 (the probabilities of a row sum to one), and the first query of
    a causal row attends to key 0 only, so its output is V[0]."""
    from cubework_amd import ops

    b, s, h, d = 1, 512, 2, 64
    qkv = _qkv(b, s, h, d, seed=3).to(DEV)
    q, k, v = _views(qkv, h, d)
    with_ones = qkv.clone()
    q1, k1, v1 = _views(with_ones, h, d)
    v1.fill_(1.0)
    out = ops.attn_fwd(q1, k1, v1)
    assert (out.float() - 1.0).abs().max().item() <= 2 ** -7
    out = ops.attn_fwd(q, k, v)
    assert torch.equal(out[0, 0].view(h, d), v[0, 0])


def test_attention_full_size_sampled_rows():
    """The OPT-1.3B-shaped workload (batch 4, 2048 tokens, 32 heads of 64): sampled (batch, head) pairs
    against the float32 oracle."""
    import oracle
    from cubework_amd import ops

    b, s, h, d = 4, 2048, 32, 64
    g = torch.Generator(device="cpu").manual_seed(0)
    qkv = (torch.randn((b, s, h * 3 * d), generator=g)).to(torch.bfloat16)
    q, k, v = _views(qkv.to(DEV), h, d)
    got = ops.attn_fwd(q, k, v).view(b, s, h, d)
    torch.cuda.synchronize()
    qc, kc, vc = oracle.split_qkv(qkv, h)
    for bi, hi in [(0, 0), (3, 31), (1, 17)]:
        want = oracle.attention_core(qc[bi:bi + 1, hi:hi + 1], kc[bi:bi + 1, hi:hi + 1], vc[bi:bi + 1, hi:hi + 1])
        assert_parity(got[bi, :, hi, :], want[0], torch.bfloat16, "full-size attention (b=%d, h=%d)" % (bi, hi))


def test_attention_rejects_unsupported():
    from cubework_amd import ops

    q = torch.zeros((1, 8, 1, 96), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        ops.attn_fwd(q, q, q)
    q = torch.zeros((1, 8, 1, 64), dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError):
        ops.attn_fwd(q, q, q)


@pytest.mark.parametrize("shape", [(1, 64, 1), (2, 256, 2), (1, 100, 2), (1, 257, 1), (1, 1, 1), (1, 33, 2),
                                   (1, 640, 1), (1, 700, 2)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_parity(shape, causal):
    import oracle
    from cubework_amd import ops

    b, s, h = shape
    d = 64
    qkv = _qkv(b, s, h, d, seed=7 * s + h, std=1.2)
    d_out = randn((b, s, h * d), torch.bfloat16, seed=s + 11)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    want = oracle.attention_core_backward(qc, kc, vc, d_out, causal=causal)
    dev = qkv.to(DEV)
    q, k, v = _views(dev, h, d)
    out, lse = ops.attn_fwd(q, k, v, causal=causal, want_lse=True)
    g = torch.full((b, s, h, 3 * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attn_bwd(q, k, v, out, d_out.to(DEV), lse, g[..., :d], g[..., d:2 * d], g[..., 2 * d:], causal=causal)
    torch.cuda.synchronize()
    if s == 1:
        # a single key: dq and dk are exactly zero, so only the three gradients together have a scale
        assert_parity(g.permute(0, 2, 1, 3), torch.cat(want, dim=-1), torch.bfloat16, "attention grads %s" % (shape,))
        return
    for name, got, ref in (("dq", g[..., :d], want[0]), ("dk", g[..., d:2 * d], want[1]), ("dv", g[..., 2 * d:], want[2])):
        assert_parity(got.permute(0, 2, 1, 3), ref, torch.bfloat16, "attention %s %s causal=%s" % (name, shape, causal))


def test_attention_core_autograd_and_reproducibility():
    """The differentiable wrapper on the qkv projection's layout: gradient of the whole [b, s, 3*h*d] tensor
    against the oracle's closed form, and bit-identical results from call to call (no atomics)."""
    import oracle
    from cubework_amd import ops

    b, s, h, d = 2, 384, 4, 64
    qkv = _qkv(b, s, h, d, seed=21)
    d_out = randn((b, s, h * d), torch.bfloat16, seed=22)
    x = qkv.to(DEV).requires_grad_(True)
    y = ops.attention_core(x, h)
    y.backward(d_out.to(DEV))
    g1 = x.grad.clone()
    x.grad = None
    ops.attention_core(x, h).backward(d_out.to(DEV))
    assert torch.equal(g1, x.grad)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    dq, dk, dv = oracle.attention_core_backward(qc, kc, vc, d_out)
    want = torch.cat([dq, dk, dv], dim=-1).permute(0, 2, 1, 3).reshape(b, s, h * 3 * d)
    assert_parity(g1, want, torch.bfloat16, "d qkv")
    assert_parity(y, oracle.attention_core(qc, kc, vc), torch.bfloat16, "attention_core forward")


@pytest.mark.parametrize("shape", [(1, 64, 1), (2, 256, 2), (1, 100, 2), (1, 257, 1), (1, 1, 1), (1, 33, 2), (1, 700, 2),
                                   (1, 129, 3)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_head_size_128(shape, causal):
    """Head size 128 (OPT-6.7B and larger): two 64-column panels per tile; forward, log-sum-exp and the
    three gradients against the oracle. 129 and 257 tokens cross the key-block size of the dK/dV kernel
    (128 keys at this head size)."""
    import oracle
    from cubework_amd import ops

    b, s, h = shape
    d = 128
    qkv = _qkv(b, s, h, d, seed=3 * s + h, std=1.2)
    d_out = randn((b, s, h * d), torch.bfloat16, seed=s + 17)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    with oracle.precision(torch.float64):
        want, want_lse = oracle.attention_core(qc, kc, vc, causal=causal, return_lse=True)
    want_g = oracle.attention_core_backward(qc, kc, vc, d_out, causal=causal)
    dev = qkv.to(DEV)
    q, k, v = _views(dev, h, d)
    out, lse = ops.attn_fwd(q, k, v, causal=causal, want_lse=True)
    g = torch.full((b, s, h, 3 * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attn_bwd(q, k, v, out, d_out.to(DEV), lse, g[..., :d], g[..., d:2 * d], g[..., 2 * d:], causal=causal)
    torch.cuda.synchronize()
    assert_parity(out, want, torch.bfloat16, "attention out d=128 %s" % (shape,))
    assert_parity(lse, want_lse, torch.float32, "attention lse d=128 %s" % (shape,), bar=LSE_BAR[torch.bfloat16])
    if s == 1:
        assert_parity(g.permute(0, 2, 1, 3), torch.cat(want_g, dim=-1), torch.bfloat16, "attention grads d=128 %s" % (shape,))
        return
    for name, got, ref in (("dq", g[..., :d], want_g[0]), ("dk", g[..., d:2 * d], want_g[1]), ("dv", g[..., 2 * d:], want_g[2])):
        assert_parity(got.permute(0, 2, 1, 3), ref, torch.bfloat16, "attention %s d=128 %s causal=%s" % (name, shape, causal))


@pytest.mark.parametrize("d", [48, 80, 8])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_core_head_sizes_between_the_kernels(d, causal):
    """Head sizes of the reference's model list that are neither 64 nor 128 (opt_125m: 768 / 16 = 48; opt_2_7b and
    opt_13b: 80, benchmark/opt/opt.py:419-495) go through the same kernels zero-padded to 64 / 128, with the softmax
    scale of the model's own head size: forward and the gradient of the whole qkv tensor against the oracle."""
    import oracle
    from cubework_amd import ops

    b, s, h = 2, 200, 3
    qkv = _qkv(b, s, h, d, seed=41 + d)
    d_out = randn((b, s, h * d), torch.bfloat16, seed=42 + d)
    x = qkv.to(DEV).requires_grad_(True)
    y = ops.attention_core(x, h, None, causal)
    assert y.shape == (b, s, h * d)
    y.backward(d_out.to(DEV))
    g1 = x.grad.clone()
    x.grad = None
    ops.attention_core(x, h, None, causal).backward(d_out.to(DEV))
    assert torch.equal(g1, x.grad)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    assert_parity(y, oracle.attention_core(qc, kc, vc, causal=causal), torch.bfloat16, "attention_core forward, head size %d" % d)
    dq, dk, dv = oracle.attention_core_backward(qc, kc, vc, d_out, causal=causal)
    want = torch.cat([dq, dk, dv], dim=-1).permute(0, 2, 1, 3).reshape(b, s, h * 3 * d)
    assert_parity(g1, want, torch.bfloat16, "d qkv, head size %d" % d)


def test_attention_core_rejects_head_sizes_above_128():
    from cubework_amd import ops

    x = torch.zeros((1, 8, 3 * 160), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):
        ops.attention_core(x, 1)


def test_attention_head_size_128_autograd():
    import oracle
    from cubework_amd import ops

    b, s, h, d = 2, 320, 3, 128
    qkv = _qkv(b, s, h, d, seed=31)
    d_out = randn((b, s, h * d), torch.bfloat16, seed=32)
    x = qkv.to(DEV).requires_grad_(True)
    ops.attention_core(x, h).backward(d_out.to(DEV))
    g1 = x.grad.clone()
    x.grad = None
    ops.attention_core(x, h).backward(d_out.to(DEV))
    assert torch.equal(g1, x.grad)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    dq, dk, dv = oracle.attention_core_backward(qc, kc, vc, d_out)
    want = torch.cat([dq, dk, dv], dim=-1).permute(0, 2, 1, 3).reshape(b, s, h * 3 * d)
    assert_parity(g1, want, torch.bfloat16, "d qkv, head size 128")


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("shape", [(2, 256, 2), (1, 100, 2), (1, 257, 1), (1, 1, 1), (1, 700, 2)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_float16(shape, causal, d):
    """float16 q/k/v (what the projections return under a plain autocast): forward, log-sum-exp and the three
    gradients against the oracle at the float16 bar (probabilities and dS are rounded to 11 significand bits
    instead of bfloat16's 8 on their way into the second MFMA)."""
    import oracle
    from cubework_amd import ops

    b, s, h = shape
    f16 = torch.float16
    qkv = _qkv(b, s, h, d, seed=5 * s + h, std=1.2).to(f16)
    d_out = randn((b, s, h * d), f16, seed=s + 19)
    qc, kc, vc = oracle.split_qkv(qkv, h)
    with oracle.precision(torch.float64):
        want, want_lse = oracle.attention_core(qc, kc, vc, causal=causal, return_lse=True)
    want_g = oracle.attention_core_backward(qc, kc, vc, d_out, causal=causal)
    dev = qkv.to(DEV)
    q, k, v = _views(dev, h, d)
    out, lse = ops.attn_fwd(q, k, v, causal=causal, want_lse=True)
    g = torch.full((b, s, h, 3 * d), float("nan"), dtype=f16, device=DEV)
    ops.attn_bwd(q, k, v, out, d_out.to(DEV), lse, g[..., :d], g[..., d:2 * d], g[..., 2 * d:], causal=causal)
    torch.cuda.synchronize()
    assert out.dtype == f16
    assert_parity(out, want, f16, "float16 attention out d=%d %s" % (d, shape))
    assert_parity(lse, want_lse, torch.float32, "float16 attention lse d=%d %s" % (d, shape), bar=LSE_BAR[torch.float16])
    if s == 1:  # dq and dk are exactly zero: judged against the size of the whole gradient
        assert_parity(g.permute(0, 2, 1, 3), torch.cat(want_g, dim=-1), f16, "float16 attention grads d=%d %s" % (d, shape))
        return
    for name, got, ref in (("dq", g[..., :d], want_g[0]), ("dk", g[..., d:2 * d], want_g[1]), ("dv", g[..., 2 * d:], want_g[2])):
        assert_parity(got.permute(0, 2, 1, 3), ref, f16, "float16 attention %s d=%d %s causal=%s" % (name, d, shape, causal))
