"""The entry points enqueue work on the caller's stream and neither allocate nor synchronise, so a sequence
of them can be recorded into a HIP graph (torch.cuda.graph) and replayed: every replay must reproduce the
eager results bit for bit, also with other work and synchronisations between the replays."""
import pytest
import torch

from tests.util import randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _pipeline(x, w1, b1, w2, gamma, beta, targets, ids, table_rows, wide_w, clip_params):
    from cubework_amd import ops

    h = ops.gemm_ksteps("NN", [x], [w1], b1, "gelu_tanh")                      # LDS-ring kernel
    y, _ = ops.ln_forward_fused(h, 1e-5, gamma, beta)
    small = ops.gemm_ksteps("TN", [y], [x])                                    # few tiles, long k: split k with scratch
    logits = ops.gemm_ksteps("NT", [y], [w2])
    mx, se, pr, mask = ops.vpce_fwd_local(logits, targets, 0)
    loss, gmax, gsum = ops.vpce_finalize(mx[None], se[None], pr[None], mask[None])
    grad = ops.vpce_bwd(logits, targets, 0, gmax, gsum, None, 1.0 / targets.numel())
    dw = ops.embedding_bwd(ids, y, table_rows, 0)
    qkv = ops.gemm_ksteps("NN", [y], [w1[:, :768].contiguous()])               # 4 heads of 64: q, k, v side by side
    att = ops.attention_core(qkv.view(4, -1, 768), 4)
    # attention backward (two launches, the first leaves D for the second in scratch)
    t4 = qkv.view(4, -1, 4, 192)
    q, k, v = t4[..., :64], t4[..., 64:128], t4[..., 128:]
    o, lse = ops.attn_fwd(q, k, v, want_lse=True)
    g = torch.empty_like(t4)
    ops.attn_bwd(q, k, v, o, att, lse, g[..., :64], g[..., 64:128], g[..., 128:])
    # 16 x 18 tiles of 256 x 256: the last 32 go to the small-tile kernel as a second launch
    wide = ops.gemm_ksteps("NN", [x], [wide_w], None, "relu")
    # gradient clipping (norm stage + scaling stage; a coefficient of 1 keeps the replays idempotent)
    from cubework_amd.clip_grad import clip_grad_norm
    norm = clip_grad_norm(clip_params, 1e30)
    # LayerNorm backward of a row-split layer: the dx launch finishes the first launch's column sums
    _, mr = ops.ln_forward_fused(h, 1e-5, gamma, beta)
    rs, pending = ops.ln_bwd_partials_open(x, h, mr, gamma)
    ln_dx, ln_dg, ln_db = ops.ln_bwd_dx_close(x, h, mr, rs, h.shape[-1], pending, gamma)
    return h, y, small, loss, grad, dw, att, g, wide, norm.reshape(1), ln_dx, ln_dg, ln_db


def test_entry_points_replay_from_a_graph():
    from cubework_amd.distributed import initialize

    initialize(None, 1)  # whatever an earlier test set up: the clipping below is a single rank's
    T, H, V = 4096, 2048, 1024
    x = randn((T, H), torch.bfloat16, 0).to(DEV)
    w1 = randn((H, H), torch.bfloat16, 1, std=0.03).to(DEV)
    b1 = randn((H,), torch.bfloat16, 2, std=0.1).to(DEV)
    w2 = randn((V, H), torch.bfloat16, 3, std=0.03).to(DEV)
    gamma = (1.0 + 0.1 * randn((H,), torch.float32, 4)).to(torch.bfloat16).to(DEV)
    beta = randn((H,), torch.bfloat16, 5, std=0.1).to(DEV)
    targets = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(6)).to(DEV)
    ids = torch.randint(0, 300, (T,), generator=torch.Generator().manual_seed(7)).to(DEV)
    wide_w = randn((H, 4376), torch.bfloat16, 8, std=0.03).to(DEV)
    clip_params = []
    for i, shape in enumerate([(70000,), (300, 7), (65536,)]):
        p = torch.nn.Parameter(torch.zeros(shape, dtype=torch.bfloat16, device=DEV))
        p.grad = randn(shape, torch.bfloat16, 20 + i).to(DEV)
        clip_params.append(p)
    args = (x, w1, b1, w2, gamma, beta, targets, ids, 300, wide_w, clip_params)

    eager = [t.clone() for t in _pipeline(*args)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _pipeline(*args)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _pipeline(*args)
    for replay in range(3):
        for t in outs:
            t.fill_(float("nan")) if t.is_floating_point() else t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want in zip(("gemm", "layernorm", "split-k gemm", "loss", "logits grad", "embedding grad", "attention",
                                    "attention grad", "two-launch gemm", "gradient norm", "layernorm dx", "layernorm dgamma",
                                    "layernorm dbeta"),
                                   outs, eager):
            assert torch.equal(got, want), "%s differs on replay %d" % (name, replay)
        # the program's own eager work between replays
        again = _pipeline(*args)
        torch.cuda.synchronize()
        assert torch.equal(again[0], eager[0])


def test_decoder_block_step_replays_from_a_graph():
    """A whole training step of the mirrored layers - LayerNorm2D, Linear2D (fused activation, residual in the
    epilogue), the attention core, their autograd backward - recorded once and replayed: with new input data in the
    static buffers every replay gives the output and every gradient of the eager step, bit for bit, and eager steps
    between the replays do not disturb it."""
    from cubework_amd.distributed import initialize
    from cubework_amd.opt_block import OPTBlock

    initialize("2d", 1)
    torch.manual_seed(0)
    blk = OPTBlock(hidden=512, heads=8, ffn=2048, dtype=torch.bfloat16, activation="relu").to(DEV)
    params = [p for p in blk.parameters()]
    inputs = [(randn((2, 384, 512), torch.bfloat16, 70 + i).to(DEV), randn((2, 384, 512), torch.bfloat16, 80 + i).to(DEV))
              for i in range(3)]

    def eager_step(x_data, dy_data):
        for p in params:
            p.grad = None
        x = x_data.clone().requires_grad_(True)
        y = blk(x)
        y.backward(dy_data)
        return [y.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in params]

    want = [eager_step(*io) for io in inputs]
    torch.cuda.synchronize()

    x_static = inputs[0][0].clone().requires_grad_(True)
    dy_static = inputs[0][1].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # warm-up on a side stream: every kernel's first-use set-up happens outside the capture
            for p in params:
                p.grad = None
            x_static.grad = None
            blk(x_static).backward(dy_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for p in params:
        p.grad = None
    x_static.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = blk(x_static)
        y_static.backward(dy_static)
    names = ["output", "input gradient"] + [n + ".grad" for n, _ in blk.named_parameters()]
    for replay, (x_data, dy_data) in enumerate(inputs):
        with torch.no_grad():
            x_static.copy_(x_data)
            dy_static.copy_(dy_data)
        graph.replay()
        torch.cuda.synchronize()
        got = [y_static, x_static.grad] + [p.grad for p in params]
        for name, g, w in zip(names, got, want[replay]):
            assert torch.equal(g, w), "%s differs on replay %d" % (name, replay)
        # an eager step between the replays (it replaces the parameters' .grad tensors: put the graph's back)
        held = [p.grad for p in params]
        again = eager_step(*inputs[replay])
        torch.cuda.synchronize()
        assert torch.equal(again[0], want[replay][0])
        for p, h in zip(params, held):
            p.grad = h
