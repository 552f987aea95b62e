"""The benchmark definition's first and fifth workloads at their full sizes, checked for values.

At these sizes the GEMMs take other kernel paths than the small parity cases do (fp32 ring kernels with a
reduction of 4096; 16-bit 256 x 256 ring tiles, reductions of 8192, split-k and small-tile weight gradients;
the attention kernels over 2048 tokens), so the results are compared with float64 on the CPU:

  * Linear1D column-parallel backward, fp32: dX = dY W ([4096,4096] x [4096,1024]) and dW = dY^T X in full
    against float64 matmul, at 1e-5.
  * One OPT-1.3B-shaped decoder layer (hidden 2048, 32 heads, FFN 8192, batch 4 x 2048 tokens, bf16),
    forward + backward through cubework_amd.opt_block.OPTBlock. Every operator of the layer is checked on a
    sample against float64 evaluated on that sample, from the operator's own inputs as the GPU run produced
    them (captured with hooks): LayerNorm rows, rows of each linear's output and input gradient, a block of
    each weight gradient (all 8192 tokens reduced), columns of each bias gradient, and whole (batch, head)
    pairs of the attention core, forward and backward. An output row of the whole layer depends on every
    earlier token through the attention, so sampling the layer end to end would mean evaluating all of it;
    the composition of the operators is what tests/test_gpu_modules.py checks at a reduced size.
"""
import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_linear1d_fp32_backward_full_size():
    """dX and dW of F.linear(x [8*512, 1024], W [4096, 1024]) (parallel_1d/module.py:269 and its autograd)
    with dY [4096, 4096] ~ N(0,1), x ~ N(0,1), W xavier-uniform; reductions of 4096 in fp32 MFMA."""
    from cubework_amd import ops

    x = randn((4096, 1024), torch.float32, 1)
    w = ((torch.rand((4096, 1024), generator=torch.Generator().manual_seed(2)) * 2 - 1) * (6.0 / 5120) ** 0.5)
    dy = randn((4096, 4096), torch.float32, 3)
    xd, wd, dyd = x.to(DEV), w.to(DEV), dy.to(DEV)
    dx = ops.gemm_ksteps("NN", [dyd], [wd])     # dX = dY W
    dw = ops.gemm_ksteps("TN", [dyd], [xd])     # dW = dY^T X
    y = ops.gemm_ksteps("NT", [xd], [wd], torch.zeros(4096, device=DEV))
    torch.cuda.synchronize()
    assert_parity(y, x.double() @ w.double().t(), torch.float32, "config 1 forward [4096,1024]x[4096,1024]^T")
    assert_parity(dx, dy.double() @ w.double(), torch.float32, "config 1 dX, K=4096")
    assert_parity(dw, dy.double().t() @ x.double(), torch.float32, "config 1 dW, K=4096")
    # the bias gradient of the same layer: column sums over 4096 rows
    db = ops.colsum(dyd)
    assert_parity(db, dy.double().sum(0), torch.float32, "config 1 dbias")


def _rows(t, idx):
    return t.detach().reshape(-1, t.shape[-1]).index_select(0, idx).double().cpu()


def _cols(t, idx):
    return t.detach().reshape(-1, t.shape[-1]).index_select(1, idx).double().cpu()


@pytest.mark.parametrize("activation", ["relu", "gelu_tanh"])
def test_opt_block_full_size_operator_by_operator(activation):
    from cubework_amd.distributed import initialize
    from cubework_amd.opt_block import OPTBlock

    hidden, heads, ffn, batch, seq = 2048, 32, 8192, 4, 2048
    hd = hidden // heads
    initialize("2d", 1)
    torch.manual_seed(0)
    blk = OPTBlock(hidden=hidden, heads=heads, ffn=ffn, dtype=torch.bfloat16, activation=activation).to(DEV)
    with torch.no_grad():  # OPT-like parameters: weights ~ N(0, 0.02), biases ~ N(0, 0.02), gamma near 1
        for name, prm in blk.named_parameters():
            g = torch.Generator().manual_seed(len(name) + prm.numel() % 97)
            if "layer_norm" in name and name.endswith("weight"):
                prm.copy_((1.0 + 0.1 * torch.randn(prm.shape, generator=g)).to(torch.bfloat16))
            else:
                prm.copy_((0.02 * torch.randn(prm.shape, generator=g)).to(torch.bfloat16))
    x = randn((batch, seq, hidden), torch.bfloat16, 11).to(DEV).requires_grad_(True)
    dy = randn((batch, seq, hidden), torch.bfloat16, 12).to(DEV)

    names = ["self_attn_layer_norm", "qkv_proj", "out_proj", "final_layer_norm", "fc1", "fc2"]
    cap = {n: {} for n in names}
    hooks = []
    for n in names:
        mod = getattr(blk, n)

        def fwd(m, args, kwargs, out, n=n):
            # the LayerNorms are called with fork_residual=True: (normalised, input again for the residual branch)
            cap[n]["in"], cap[n]["out"] = args[0].detach(), (out[0] if isinstance(out, tuple) else out).detach()
            res = kwargs.get("residual")   # out_proj and fc2 add the residual stream in their epilogue
            cap[n]["residual"] = None if res is None else res.detach()

        def bwd(m, gin, gout, n=n):
            cap[n]["d_in"], cap[n]["d_out"] = gin[0].detach(), gout[0].detach()
            # a forked LayerNorm also receives the residual branch's gradient, which its kernel adds to dx
            cap[n]["d_res"] = gout[1].detach() if len(gout) > 1 and gout[1] is not None else None
        hooks += [mod.register_forward_hook(fwd, with_kwargs=True), mod.register_full_backward_hook(bwd)]
    y = blk(x)
    y.backward(dy)
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    assert cap["out_proj"]["residual"] is not None and cap["fc2"]["residual"] is not None  # both ride the epilogue
    params = dict(blk.named_parameters())

    def prm(prefix, leaf):
        for n, t in params.items():
            if n.startswith(prefix + ".") and n.endswith(leaf):
                return t
        raise KeyError(prefix + "." + leaf)

    T = batch * seq
    gen = torch.Generator().manual_seed(5)
    rows = torch.cat([torch.tensor([0, 1, 255, 256, T - 1]), torch.randint(0, T, (59,), generator=gen)]).to(DEV)
    BF = torch.bfloat16

    # ---- LayerNorms: sampled rows forward and dX; dgamma / dbeta in full (all 8192 rows reduced)
    for n in ("self_attn_layer_norm", "final_layer_norm"):
        c = cap[n]
        gam, bet = prm(n, "weight"), prm(n, "bias")
        xr = _rows(c["in"], rows).requires_grad_(True)
        gr, br = gam.detach().double().cpu(), bet.detach().double().cpu()
        ref = F.layer_norm(xr, (hidden,), gr, br, 1e-5)
        ref.backward(_rows(c["d_out"], rows))
        assert_parity(_rows(c["out"], rows), ref.detach(), BF, n + " forward rows")
        assert c["d_res"] is not None, "the residual branch's gradient did not reach the LayerNorm's backward"
        assert_parity(_rows(c["d_in"], rows), xr.grad + _rows(c["d_res"], rows), BF, n + " dX rows (+ residual branch)")
        xa = c["in"].detach().reshape(T, hidden).double().cpu()
        da = c["d_out"].detach().reshape(T, hidden).double().cpu()
        mu = xa.mean(-1, keepdim=True)
        xh = (xa - mu) / torch.sqrt(xa.var(-1, unbiased=False, keepdim=True) + 1e-5)
        assert_parity(gam.grad, (da * xh).sum(0), BF, n + " dgamma (8192 rows)")
        assert_parity(bet.grad, da.sum(0), BF, n + " dbeta (8192 rows)")
        del xa, da, xh

    # ---- the four linears: weights are [in, out] (Linear2D)
    act = {"relu": F.relu, "gelu_tanh": lambda t: F.gelu(t, approximate="tanh")}[activation]
    for n in ("qkv_proj", "out_proj", "fc1", "fc2"):
        c = cap[n]
        W, b = prm(n, "weight"), prm(n, "bias")
        K, N = W.shape
        Wd, bd = W.detach().double().cpu(), b.detach().double().cpu()
        xin = _rows(c["in"], rows).requires_grad_(True)
        pre = xin @ Wd + bd
        if c["residual"] is not None:
            pre = pre + _rows(c["residual"], rows)
        out_rows = _rows(c["out"], rows)
        if n == "fc1":
            if activation == "relu":
                # both sides differentiate with the units the GPU let through (its rounded output's sign)
                mask = (out_rows > 0).double()
                near0 = pre.detach().abs() < 1e-4 * pre.detach().abs().max()  # fp32 accumulation error can flip these
                assert bool(((pre.detach() > 0).double() == mask)[~near0].all()), "ReLU mask differs away from 0"
                ref = pre * mask
            else:
                ref = act(pre)
        else:
            ref = pre
        ref.backward(_rows(c["d_out"], rows))
        assert_parity(out_rows, ref.detach(), BF, n + " forward rows [%d -> %d]" % (K, N))
        assert_parity(_rows(c["d_in"], rows), xin.grad, BF, n + " dX rows")
        # gradient entering the GEMMs of the backward: d_out, through the activation's derivative for fc1
        kk = torch.randint(0, K, (48,), generator=gen).to(DEV)
        cc = torch.randint(0, N, (64,), generator=gen).to(DEV)
        d_out_c = _cols(c["d_out"], cc)
        if n == "fc1":
            if activation == "relu":
                d_pre_c = d_out_c * (_cols(c["out"], cc) > 0).double()
            else:
                pre_c = c["in"].detach().reshape(T, K).double().cpu() @ Wd[:, cc.cpu()] + bd[cc.cpu()]
                p = pre_c.clone().requires_grad_(True)
                act(p).backward(d_out_c)
                d_pre_c = p.grad
        else:
            d_pre_c = d_out_c
        in_k = _cols(c["in"], kk)
        want_dw = in_k.t() @ d_pre_c                       # [48, 64] block of dW, all tokens reduced
        got_dw = W.grad.detach().index_select(0, kk).index_select(1, cc)
        assert_parity(got_dw, want_dw, BF, n + " dW block (8192 tokens reduced)")
        assert_parity(b.grad.detach().index_select(0, cc), d_pre_c.sum(0), BF, n + " dbias columns")

    # ---- attention core: whole (batch, head) pairs, forward and backward
    qkv = cap["qkv_proj"]["out"].reshape(batch, seq, heads, 3 * hd)
    o = cap["out_proj"]["in"].reshape(batch, seq, heads, hd)
    d_o = cap["out_proj"]["d_in"].reshape(batch, seq, heads, hd)
    d_qkv = cap["qkv_proj"]["d_out"].reshape(batch, seq, heads, 3 * hd)
    for b_, h_ in ((0, 0), (3, 31), (1, 17)):
        t = qkv[b_, :, h_].double().cpu()
        q, k, v = (t[:, :hd].clone().requires_grad_(True), t[:, hd:2 * hd].clone().requires_grad_(True),
                   t[:, 2 * hd:].clone().requires_grad_(True))
        s = (q * hd ** -0.5) @ k.t() + torch.full((seq, seq), float("-inf"), dtype=torch.float64).triu(1)
        ref = torch.softmax(s, dim=-1) @ v
        ref.backward(d_o[b_, :, h_].double().cpu())
        assert_parity(o[b_, :, h_], ref.detach(), BF, "attention forward (b=%d, h=%d), 2048 tokens" % (b_, h_))
        want = torch.cat([q.grad, k.grad, v.grad], dim=-1)
        # the backward rounds the recomputed probabilities and dS to bf16 as MFMA operands: two roundings
        assert_parity(d_qkv[b_, :, h_], want, BF, "attention backward (b=%d, h=%d)" % (b_, h_))
