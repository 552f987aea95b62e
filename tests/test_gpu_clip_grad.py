"""GPU parity of clip_grad_norm (cw_multi_norm_partials / cw_multi_scale through the C ABI) against
torch.nn.utils.clip_grad_norm_, which the reference's function is adapted from and equals at
tensor-parallel size 1 (cubework/utils/clip_grad.py:1-4)."""
import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _params(shapes, dtype, seed, tp_every=2):
    from cubework_amd.global_vars import NUM_PARTITIONS
    ps = []
    for i, shp in enumerate(shapes):
        p = torch.nn.Parameter(torch.zeros(shp, dtype=dtype, device=DEV))
        p.grad = randn(shp, dtype, seed + i, std=0.5 + 0.1 * i).to(DEV)
        if i % tp_every == 0:
            setattr(p, NUM_PARTITIONS, 1)
        ps.append(p)
    return ps


SHAPES = [(1000, 33), (7,), (70000,), (256, 256), (1,), (65536,), (65537,), (3, 5, 11)] + [(129, 17)] * 60


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("norm_type", [2.0, float("inf"), 1.0, 3.0])
@pytest.mark.parametrize("max_norm", [0.5, 1e9])
def test_clip_grad_norm_matches_torch(dtype, norm_type, max_norm):
    from cubework_amd.clip_grad import clip_grad_norm
    from cubework_amd.distributed import initialize

    initialize("2d", 1)
    ours = _params(SHAPES, dtype, 1)
    ref = [torch.nn.Parameter(torch.zeros_like(p, dtype=torch.float32, device="cpu")) for p in ours]
    for r, p in zip(ref, ours):
        r.grad = p.grad.detach().float().cpu()
    want = torch.nn.utils.clip_grad_norm_(ref, max_norm, norm_type)
    got = clip_grad_norm(ours, max_norm, norm_type)
    torch.cuda.synchronize()
    assert abs(got.item() - want.item()) <= 1e-4 * abs(want.item()), (got.item(), want.item())
    for r, p in zip(ref, ours):
        if dtype == torch.float16:
            # a small clip coefficient takes float16 gradients into the subnormal range (steps of 2^-24), where
            # a relative bound means nothing: one step of slack on top of the relative tolerance
            torch.testing.assert_close(p.grad.float().cpu(), r.grad.to(dtype).float(), rtol=1e-3, atol=2.0 ** -24)
        else:
            assert_parity(p.grad, r.grad, dtype, "clipped gradient")


def test_tensor_parallel_weighting_and_mixed_dtypes():
    """Parameters tagged with NUM_PARTITIONS = n enter the norm n times (clip_grad.py:41-43); gradients of
    two dtypes are clipped with one common coefficient; parameters without a gradient are skipped."""
    from cubework_amd.clip_grad import clip_grad_norm
    from cubework_amd.distributed import initialize
    from cubework_amd.global_vars import NUM_PARTITIONS

    initialize(None, 1)
    a = torch.nn.Parameter(torch.zeros(300, device=DEV))
    b = torch.nn.Parameter(torch.zeros((40, 8), dtype=torch.bfloat16, device=DEV))
    c = torch.nn.Parameter(torch.zeros(5, device=DEV))
    a.grad = randn((300,), torch.float32, 1).to(DEV)
    b.grad = randn((40, 8), torch.bfloat16, 2).to(DEV)
    setattr(b, NUM_PARTITIONS, 4)
    ga, gb = a.grad.clone(), b.grad.clone()
    import oracle
    want, clipped = oracle.clip_grad_norm([ga, gb], [0, 4], 1.0)
    got = clip_grad_norm([a, b, c], 1.0)
    assert abs(got.item() - want.item()) <= 1e-5 * want.item()
    assert_parity(a.grad, clipped[0], torch.float32, "fp32 gradient")
    assert_parity(b.grad, clipped[1], torch.bfloat16, "bf16 gradient")
    assert c.grad is None


def test_clip_grad_norm_empty_and_reproducible():
    from cubework_amd.clip_grad import clip_grad_norm

    assert clip_grad_norm([], 1.0).item() == 0.0
    ps = _params([(50000,), (123, 45)], torch.bfloat16, 9)
    n1 = clip_grad_norm(ps, 1e9)
    n2 = clip_grad_norm(ps, 1e9)
    assert n1.item() == n2.item()


@pytest.mark.parametrize("norm_type", [2.0, float("inf")])
def test_clip_grad_norm_with_peer_sums(norm_type):
    """A tensor-parallel group of 4 with the peers' results pre-staged: the tensor-parallel sum is
    all-reduced and divided by the group size (clip_grad.py:48-49), the maximum norm is the maximum over
    the group (:34-35)."""
    from cubework_amd.clip_grad import clip_grad_norm
    from cubework_amd.distributed import ParallelManager as pm
    from cubework_amd.distributed import initialize
    from cubework_amd.global_vars import NUM_PARTITIONS

    initialize("1d", 4)
    a = torch.nn.Parameter(torch.zeros(500, device=DEV))
    b = torch.nn.Parameter(torch.zeros((64, 9), device=DEV))
    a.grad = randn((500,), torch.float32, 5).to(DEV)
    b.grad = randn((64, 9), torch.float32, 6).to(DEV)
    setattr(b, NUM_PARTITIONS, 4)
    ga, gb = a.grad.double().cpu(), b.grad.double().cpu()
    if norm_type == 2.0:
        peers = [torch.tensor(v, dtype=torch.float32, device=DEV) for v in (1000.0, 2000.0, 3000.0)]
        want = ((ga ** 2).sum() + (4 * (gb ** 2).sum() + 6000.0) / 4) ** 0.5
    else:
        peers = [torch.tensor([v], dtype=torch.float32, device=DEV) for v in (0.5, 7.25, 1.0)]
        want = torch.tensor(7.25, dtype=torch.float64)
    pm.TENSOR.stage("all_reduce", peers)
    got = clip_grad_norm([a, b], 2.0, norm_type)
    assert abs(got.item() - want.item()) <= 1e-5 * want.item(), (got.item(), want.item())
    coef = min(2.0 / (want.item() + 1e-6), 1.0)
    assert_parity(a.grad, ga * coef, torch.float32, "gradient a")
    assert_parity(b.grad, gb * coef, torch.float32, "gradient b")
    initialize(None, 1)


@pytest.mark.parametrize("norm_type", [2.0, float("inf")])
@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
def test_clip_grad_norm_nonfinite_gradients(norm_type, bad):
    """A NaN or infinite gradient element gives the non-finite total norm torch gives (the maximum norm
    included: torch's abs().max() propagates NaN), the same scaled gradients, and error_if_nonfinite
    raises (clip_grad.py:51-57)."""
    from cubework_amd.clip_grad import clip_grad_norm
    from cubework_amd.distributed import initialize

    initialize(None, 1)
    ours = _params([(300, 7), (65,), (70000,)], torch.float32, 3)
    with torch.no_grad():
        ours[2].grad[12345] = bad
    ref = [torch.nn.Parameter(torch.zeros_like(p, device="cpu")) for p in ours]
    for r, p in zip(ref, ours):
        r.grad = p.grad.detach().cpu().clone()
    keep = [p.grad.clone() for p in ours]
    want = torch.nn.utils.clip_grad_norm_(ref, 1.0, norm_type)
    got = clip_grad_norm(ours, 1.0, norm_type)
    torch.cuda.synchronize()
    assert torch.isnan(got).item() == torch.isnan(want).item() and torch.isinf(got).item() == torch.isinf(want).item()
    for r, p in zip(ref, ours):
        assert torch.equal(torch.isnan(p.grad.cpu()), torch.isnan(r.grad))
        finite = torch.isfinite(r.grad)
        assert torch.allclose(p.grad.cpu()[finite], r.grad[finite], rtol=1e-5, atol=0)
    for p, k in zip(ours, keep):
        p.grad = k
    with pytest.raises(RuntimeError):
        clip_grad_norm(ours, 1.0, norm_type, error_if_nonfinite=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("norm_type", [2.0, float("inf"), 3.0])
def test_clip_scale_from_partials_equals_the_separate_launches(dtype, norm_type):
    """cw_clip_scale on the unfinished block partials (two launches) against cw_multi_norm_partials with its
    finalize, cw_clip_coef and cw_multi_scale (four launches): both add the partials in the same order, so the
    norm, the coefficient and every scaled gradient agree to the bit. 70 tensors: two launches of the scaling."""
    import ctypes as C
    from cubework_amd import _lib, ops

    lib = _lib.load()
    shapes = [(300000,), (65536,), (7,), (1000, 33)] + [(129, 17)] * 66
    a = [randn(s, dtype, 40 + i, std=0.3 + 0.05 * (i % 7)).to(DEV) for i, s in enumerate(shapes)]
    b = [t.clone() for t in a]
    n = len(a)
    numels = (C.c_int64 * n)(*[t.numel() for t in a])
    numels_p = C.cast(numels, C.c_void_p)
    factors = (C.c_float * n)(*[float(1 + i % 3) for i in range(n)])
    groups = (C.c_ubyte * n)(*[i % 2 for i in range(n)])
    code = ops._dtype_code(a[0])
    count = lib.cw_multi_norm_partial_count(n, numels_p)
    assert count == 5 + 1 + 1 + 1 + 66
    assert lib.cw_multi_norm_workspace_bytes(n, numels_p) == 8 * count
    stream = ops._stream()

    def tables(ts):
        return (C.c_void_p * n)(*[t.data_ptr() for t in ts])

    ws_a = torch.empty(2 * count, dtype=torch.float32, device=DEV)
    sets = torch.empty(2, dtype=torch.float32, device=DEV)
    out_a = torch.empty(2, dtype=torch.float32, device=DEV)
    pa = tables(a)
    assert lib.cw_multi_norm_partials(n, pa, numels_p, C.cast(factors, C.c_void_p), C.cast(groups, C.c_void_p), norm_type,
                                      sets.data_ptr(), ws_a.data_ptr(), 8 * count, code, stream) == 0
    assert lib.cw_clip_coef(1, sets.data_ptr(), 0.5, norm_type, 0.25, out_a.data_ptr(), stream) == 0
    assert lib.cw_multi_scale(n, pa, numels_p, out_a[1:].data_ptr(), code, stream) == 0

    ws_b = torch.full((2 * count,), float("nan"), dtype=torch.float32, device=DEV)
    out_b = torch.empty(2, dtype=torch.float32, device=DEV)
    pb = tables(b)
    assert lib.cw_multi_norm_partials(n, pb, numels_p, C.cast(factors, C.c_void_p), C.cast(groups, C.c_void_p), norm_type,
                                      None, ws_b.data_ptr(), 8 * count, code, stream) == 0
    assert lib.cw_clip_scale(n, pb, numels_p, code, 0, None, count, ws_b.data_ptr(), 0.5, norm_type, 0.25,
                             out_b.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(ws_a, ws_b)
    assert torch.equal(out_a, out_b), (out_a, out_b)
    assert 0.0 < out_a[1].item() < 1.0
    for x, y in zip(a, b):
        assert torch.equal(x, y)

    # finished sets and unfinished partials together: (sets + partials) of the same gradients count them twice
    out_c = torch.empty(2, dtype=torch.float32, device=DEV)
    assert lib.cw_clip_scale(0, None, None, code, 1, sets.data_ptr(), count, ws_b.data_ptr(), 0.5, norm_type, 1e9,
                             out_c.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    if norm_type == float("inf"):
        assert out_c[0].item() == out_a[0].item()
    else:
        want = out_a[0].double().item() * 2.0 ** (1.0 / norm_type)
        assert abs(out_c[0].item() - want) <= 1e-5 * want
    assert out_c[1].item() == 1.0


def test_clip_scale_argument_checks():
    from cubework_amd import _lib

    lib = _lib.load()
    out = torch.empty(2, dtype=torch.float32, device=DEV)
    assert lib.cw_clip_scale(0, None, None, 0, 65, None, 0, None, 1.0, 2.0, 1.0, out.data_ptr(), None) == -1
    assert lib.cw_clip_scale(0, None, None, 0, 1, None, 0, None, 1.0, 2.0, 1.0, out.data_ptr(), None) == -1
    assert lib.cw_clip_scale(0, None, None, 0, 0, None, 3, None, 1.0, 2.0, 1.0, out.data_ptr(), None) == -1
    assert lib.cw_clip_scale(0, None, None, 0, 0, None, 0, None, 1.0, 2.0, 1.0, None, None) == -1
    assert lib.cw_clip_scale(0, None, None, 0, 0, None, 0, None, 1.0, -2.0, 1.0, out.data_ptr(), None) == -1
    assert lib.cw_clip_scale(0, None, None, 7, 0, None, 0, None, 1.0, 2.0, 1.0, out.data_ptr(), None) == -1
    # no gradients at all: norm 0, coefficient 1
    assert lib.cw_clip_scale(0, None, None, 0, 0, None, 0, None, 1.0, 2.0, 1.0, out.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert out.tolist() == [0.0, 1.0]


def test_clip_scale_with_more_pairs_than_a_workgroup_should_read():
    """Beyond 2048 block partials (here 2100 chunks of 65536 elements plus two small tensors) cw_clip_scale combines
    them with one launch of their own instead of in every workgroup of the scaling launch; the results still equal
    those of cw_multi_norm_partials with its finalize, cw_clip_coef and cw_multi_scale to the bit."""
    import ctypes as C
    from cubework_amd import _lib, ops

    lib = _lib.load()
    shapes = [(2100 * 65536,), (1000, 33), (7,)]
    a = [randn(s, torch.bfloat16, 70 + i, std=0.01).to(DEV) for i, s in enumerate(shapes)]
    b = [t.clone() for t in a]
    n = len(a)
    numels = (C.c_int64 * n)(*[t.numel() for t in a])
    numels_p = C.cast(numels, C.c_void_p)
    code = ops._dtype_code(a[0])
    count = lib.cw_multi_norm_partial_count(n, numels_p)
    assert count == 2100 + 1 + 1
    stream = ops._stream()
    ws = torch.empty(2 * count, dtype=torch.float32, device=DEV)
    sets = torch.empty(2, dtype=torch.float32, device=DEV)
    out_a = torch.empty(2, dtype=torch.float32, device=DEV)
    out_b = torch.empty(2, dtype=torch.float32, device=DEV)
    pa = (C.c_void_p * n)(*[t.data_ptr() for t in a])
    pb = (C.c_void_p * n)(*[t.data_ptr() for t in b])
    assert lib.cw_multi_norm_partials(n, pa, numels_p, None, None, 2.0, sets.data_ptr(), ws.data_ptr(), 8 * count, code, stream) == 0
    assert lib.cw_clip_coef(1, sets.data_ptr(), 1.0, 2.0, 1.0, out_a.data_ptr(), stream) == 0
    assert lib.cw_multi_scale(n, pa, numels_p, out_a[1:].data_ptr(), code, stream) == 0
    assert lib.cw_multi_norm_partials(n, pb, numels_p, None, None, 2.0, None, ws.data_ptr(), 8 * count, code, stream) == 0
    assert lib.cw_clip_scale(n, pb, numels_p, code, 0, None, count, ws.data_ptr(), 1.0, 2.0, 1.0, out_b.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b), (out_a, out_b)
    want = (2100 * 65536 + 33000 + 7) ** 0.5 * 0.01
    assert abs(out_a[0].item() - want) < 0.02 * want and 0.0 < out_a[1].item() < 1.0
    for x, y in zip(a, b):
        assert torch.equal(x, y)
