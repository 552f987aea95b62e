"""GPU parity of the vocab-parallel cross-entropy entry points (through the C
ABI) against the CPU oracle and against F.cross_entropy on the concatenated
slices (the reference tests' own oracle, tests/test_1d/check_1d_modules.py:499-523).
Mask, shifted index, gathered logit and row maximum must be bit-exact. The floating-point
expected values are evaluated in float64 (oracle.precision), the fp32 results (sum of
exponentials, loss, fp32 gradient) are held to 1e-5 of the largest expected magnitude.
"""
import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _targets(T, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (T,), generator=g, dtype=torch.int64)


def _run_all_ranks(T, V, p, dtype, seed, grad_dtype=None, targets=None):
    """Run every slice through the HIP kernels; compare each with the oracle
    and the combination with F.cross_entropy."""
    import oracle
    from cubework_amd import ops

    full = randn((T, V * p), dtype, seed, std=2.0)
    t = _targets(T, V * p, seed + 1) if targets is None else targets
    slices = list(torch.chunk(full, p, dim=-1))
    stats_got, stats_want = [], []
    with oracle.precision(torch.float64):
        for r, s in enumerate(slices):
            s_dev = s.contiguous().to(DEV)
            got = ops.vpce_fwd_local(s_dev, t.to(DEV), r * V)
            want = oracle.vpce_fwd_local(s, t, r * V)
            # integer / gather part: bit exact (the values are inputs, exact in either precision)
            assert torch.equal(got[3].cpu(), want[3]), "mask"
            assert torch.equal(got[2].cpu(), want[2].float()), "gathered logit"
            assert torch.equal(got[0].cpu(), want[0].float()), "row max"
            assert_parity(got[1], want[1], torch.float32, "sum exp rank %d" % r)
            stats_got.append(got)
            stats_want.append(want)
        stk = lambda lst, k: torch.stack([x[k] for x in lst])  # noqa: E731
        loss_g, gmax_g, gsum_g = ops.vpce_finalize(*(stk(stats_got, k) for k in range(4)))
        loss_w, gmax_w, gsum_w = oracle.vpce_finalize(*(stk(stats_want, k) for k in range(4)))
        assert torch.equal(gmax_g.cpu(), gmax_w.float())
        assert_parity(gsum_g, gsum_w, torch.float32, "global sum")
        assert_parity(loss_g, loss_w, torch.float32, "loss")
        # the reference tests' oracle
        logits_ref = full.double().requires_grad_(True)
        loss_ref = torch.nn.functional.cross_entropy(logits_ref, t, reduction="none")
        assert_parity(loss_g, loss_ref.detach(), torch.float32, "loss vs F.cross_entropy")
        dl = torch.linspace(0.5, 1.5, T)
        loss_ref.backward(dl.double())
        gd = grad_dtype or dtype
        for r, s in enumerate(slices):
            grad = ops.vpce_bwd(s.contiguous().to(DEV), t.to(DEV), r * V, gmax_g, gsum_g, dl.to(DEV), 1.0, grad_dtype=gd)
            # the kernel is handed the fp32 statistics of the forward; so is the oracle
            want = oracle.vpce_bwd(s, t, r * V, gmax_g.cpu(), gsum_g.cpu(), dl)
            assert grad.dtype == gd
            assert_parity(grad, want, gd, "grad rank %d vs oracle" % r)
            ref = logits_ref.grad[:, r * V:(r + 1) * V]
            assert_parity(grad, ref, gd, "grad rank %d vs autograd" % r)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(64, 1024, 4), (37, 1571 * 8, 2), (16, 100, 4), (5, 7, 3), (130, 4104, 1)])
def test_vpce_all_ranks(shape, dtype):
    T, V, p = shape
    _run_all_ranks(T, V, p, dtype, seed=T + V)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_vpce_16bit_logits_fp32_grad(dtype):
    _run_all_ranks(32, 2048, 2, dtype, seed=3, grad_dtype=torch.float32)
    _run_all_ranks(9, 12568, 1, dtype, seed=4, grad_dtype=torch.float32)


@pytest.mark.parametrize("amp_dtype", [torch.float16, torch.bfloat16])
def test_loss_under_autocast_keeps_16bit_logits(amp_dtype):
    """Classifier + loss inside torch.autocast: the logits reach the loss in the autocast dtype and are not
    copied to float32 (the reference's custom_fwd(cast_inputs=torch.float32) does; the cast is exact, so the
    loss and the gradient are those of F.cross_entropy on the float32 copy)."""
    from cubework_amd.distributed import initialize
    from cubework_amd.module.loss import VocabParallelCrossEntropyLoss1D

    initialize("1d", 1)
    T, V = 96, 2000
    logits = randn((T, V), amp_dtype, 0, std=2.0).to(DEV).requires_grad_(True)
    t = _targets(T, V, 1).to(DEV)
    crit = VocabParallelCrossEntropyLoss1D()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    with torch.autocast("cuda", dtype=amp_dtype):
        loss = crit(logits, t)
    loss.backward()
    torch.cuda.synchronize()
    assert loss.dtype == torch.float32 and logits.grad.dtype == amp_dtype
    # one gradient of the logits' size and per-row statistics: no float32 copy (T * V * 4 bytes) was made
    assert torch.cuda.max_memory_allocated() - before < T * V * 2 + T * V * 4
    ref_in = logits.detach().double().cpu().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(ref_in, t.cpu())
    ref.backward()
    assert_parity(loss, ref.detach(), torch.float32, "loss")
    assert_parity(logits.grad, ref_in.grad, amp_dtype, "logits grad")


def test_vpce_edge_targets():
    """Targets on the slice borders: start-1, start, end-1, end, 0, V-1."""
    V, p = 256, 4
    edge = []
    for r in range(p):
        edge += [max(r * V - 1, 0), r * V, (r + 1) * V - 1, min((r + 1) * V, V * p - 1)]
    edge += [0, V * p - 1]
    t = torch.tensor(edge, dtype=torch.int64)
    _run_all_ranks(len(edge), V, p, torch.bfloat16, seed=11, targets=t)
    _run_all_ranks(len(edge), V, p, torch.float32, seed=12, targets=t)


def test_vpce_does_not_modify_logits_and_handles_padding():
    from cubework_amd import ops
    import oracle

    T, V = 24, 520
    parent = randn((T, V + 24), torch.bfloat16, 5, std=2.0).to(DEV)
    view = parent[:, :V]
    before = parent.clone()
    t = _targets(T, 2 * V, 6).to(DEV)
    got = ops.vpce_fwd_local(view, t, V)
    with oracle.precision(torch.float64):
        want = oracle.vpce_fwd_local(view.cpu(), t.cpu(), V)
    assert torch.equal(got[2].cpu(), want[2].float()) and torch.equal(got[3].cpu(), want[3])
    assert_parity(got[1], want[1], torch.float32, "sumexp")
    loss, gmax, gsum = ops.vpce_finalize(*(g.unsqueeze(0) for g in got))
    ops.vpce_bwd(view, t, V, gmax, gsum, None, 0.25)
    torch.cuda.synchronize()
    assert torch.equal(parent, before)


def test_vpce_baseline_shape_properties():
    """The benchmark's cross-entropy workload at full size (rank 1 of 4, V_loc = 12568): rows of the
    softmax gradient sum to zero across the 4 slices; loss equals logsumexp
    minus the target logit on sampled rows; grad = -dloss*(1-softmax) at the
    target column."""
    from cubework_amd import ops

    T, V, p = 8192, 12568, 4
    t = _targets(T, V * p, 1).to(DEV)
    slices = [randn((T, V), torch.bfloat16, 10 + r, std=2.0, device=DEV) for r in range(p)]
    stats = [ops.vpce_fwd_local(s, t, r * V) for r, s in enumerate(slices)]
    loss, gmax, gsum = ops.vpce_finalize(*(torch.stack([st[k] for st in stats]) for k in range(4)))
    # exactly one rank owns each target
    owners = torch.stack([st[3] for st in stats]).to(torch.int32)
    assert torch.equal((1 - owners).sum(dim=0), torch.ones(T, dtype=torch.int32, device=DEV))
    rows = torch.arange(0, T, 257, device=DEV)
    full = torch.cat([s[rows] for s in slices], dim=1).float().cpu()
    want = torch.logsumexp(full.double(), dim=1) - full.double()[torch.arange(len(rows)), t[rows].cpu()]
    assert_parity(loss[rows].cpu().double(), want, torch.float32, "loss on sampled rows")
    dl = 1.0 / T
    total = torch.zeros(T, dtype=torch.float64, device=DEV)
    for r, s in enumerate(slices):
        g = ops.vpce_bwd(s, t, r * V, gmax, gsum, None, dl, grad_dtype=torch.float32)
        total += g.double().sum(dim=1)
    assert (total.abs() / dl).max().item() < 1e-4


def test_vpce_baseline_shape_sampled_rows_against_the_float64_oracle():
    """The benchmark's cross-entropy workload at exactly its size (8192 tokens x 12568 classes of 50272, rank 1 of
    4, bf16 logits ~ N(0, 2), dloss = 1/8192): 64 sampled rows of the bf16 and of the fp32 gradient against the
    oracle's formula in float64, evaluated with the global (max, sum) the GPU forward produced (what the rank is
    handed after the all-reduce), and the local forward statistics of those rows (mask / gathered logit / max
    bit-exact)."""
    import oracle
    from cubework_amd import ops

    T, V, p, r = 8192, 12568, 4, 1
    t = _targets(T, V * p, 1)
    slices = [randn((T, V), torch.bfloat16, 10 + k, std=2.0) for k in range(p)]
    dev_slices = [s.to(DEV) for s in slices]
    stats = [ops.vpce_fwd_local(s, t.to(DEV), k * V) for k, s in enumerate(dev_slices)]
    loss, gmax, gsum = ops.vpce_finalize(*(torch.stack([st[k] for st in stats]) for k in range(4)))
    g = torch.Generator().manual_seed(4)
    rows = torch.cat([torch.tensor([0, 1, 255, 256, T - 1]), torch.randint(0, T, (59,), generator=g)])
    dl = torch.full((T,), 1.0 / T)
    with oracle.precision(torch.float64):
        want = oracle.vpce_fwd_local(slices[r][rows], t[rows], r * V)
        got = [st.cpu()[rows] for st in stats[r]]
        assert torch.equal(got[3], want[3]) and torch.equal(got[2], want[2].float()) and torch.equal(got[0], want[0].float())
        assert_parity(got[1], want[1], torch.float32, "sum exp, 64 rows of 8192 x 12568")
        want_g = oracle.vpce_bwd(slices[r][rows], t[rows], r * V, gmax.cpu()[rows], gsum.cpu()[rows], dl[rows])
        for gd in (torch.bfloat16, torch.float32):
            grad = ops.vpce_bwd(dev_slices[r], t.to(DEV), r * V, gmax, gsum, None, 1.0 / T, grad_dtype=gd)
            assert_parity(grad.cpu()[rows], want_g, gd, "vpce_bwd %s grad, 64 rows of 8192 x 12568" % str(gd).split(".")[-1])


def test_vpce_empty():
    from cubework_amd import ops

    x = torch.zeros((0, 64), dtype=torch.bfloat16, device=DEV)
    t = torch.zeros((0,), dtype=torch.int64, device=DEV)
    out = ops.vpce_fwd_local(x, t, 0)
    assert all(o.numel() == 0 for o in out)
