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
