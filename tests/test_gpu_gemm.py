"""GPU parity of cw_gemm_ksteps (through the C ABI) against the CPU oracle.

Bars: <= 1e-2 relative for bf16 I/O with fp32 accumulation, <= 1e-5 relative
for fp32 (relative to the largest magnitude of the expected result).
"""
import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu

LAYOUTS = ["NN", "NT", "TN"]
DEV = "cuda:0"


def _operands(layout, M, N, K, steps, dtype, seed, pad_a=0, pad_b=0):
    """Step operands on the CPU; pad_* adds unused columns so that the leading
    dimension differs from the row length."""
    a_shape = (K, M) if layout == "TN" else (M, K)
    b_shape = (N, K) if layout == "NT" else (K, N)
    A, B = [], []
    for s in range(steps):
        a = randn((a_shape[0], a_shape[1] + pad_a), dtype, seed + 10 * s)
        b = randn((b_shape[0], b_shape[1] + pad_b), dtype, seed + 10 * s + 1, std=0.05)
        A.append(a[:, :a_shape[1]])
        B.append(b[:, :b_shape[1]])
    return A, B


def _to_dev(t, pad, dev):
    """Copy to the device keeping `pad` unused columns behind every row."""
    if pad == 0:
        return t.to(dev)
    parent = torch.zeros((t.shape[0], t.shape[1] + pad), dtype=t.dtype, device=dev)
    view = parent[:, :t.shape[1]]
    view.copy_(t)
    return view


def _run(layout, M, N, K, steps, dtype, act=None, bias=True, n_add=0, preact=False, pad_a=0, pad_b=0, seed=0):
    import oracle
    from cubework_amd import ops

    A, B = _operands(layout, M, N, K, steps, dtype, seed, pad_a, pad_b)
    b = randn((N,), dtype, seed + 100, std=0.5) if bias else None
    adds = [randn((M, N), dtype, seed + 200 + i) for i in range(n_add)]
    want = oracle.gemm_ksteps(layout, A, B, b, act, adds, return_preact=preact)
    dev = "cuda:0"
    Ad = [_to_dev(a, pad_a, dev) for a in A]
    Bd = [_to_dev(b_, pad_b, dev) for b_ in B]
    got = ops.gemm_ksteps(layout, Ad, Bd, None if b is None else b.to(dev), act, [t.to(dev) for t in adds],
                          want_preact=preact)
    torch.cuda.synchronize()
    tag = "%s %dx%dx%d steps=%d %s act=%s" % (layout, M, N, K, steps, dtype, act)
    if preact:
        assert_parity(got[0], want[0], dtype, tag + " out")
        assert_parity(got[1], want[1], dtype, tag + " preact")
    else:
        assert_parity(got, want, dtype, tag)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_bf16_exact_tiles_small_config(layout):
    # 128x128 tiles, no guards
    _run(layout, 256, 384, 192, 2, torch.bfloat16, act=None)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_bf16_exact_tiles_big_config(layout):
    # 256x256 tiles (>= 128 of them), two k-steps, fused bias + GeLU(tanh)
    _run(layout, 4096, 2048, 256, 2, torch.bfloat16, act="gelu_tanh")


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(4104, 8200, 64), (4096, 8216, 128), (8200, 4096, 64)])
def test_bf16_ragged_around_aligned_core(layout, shape):
    """Large outputs whose M and / or N are not tile multiples (a vocabulary slice: 12568 = 49 x 256 + 24):
    aligned core on the LDS-DMA kernel, strips on the guarded kernel, every part with bias, addend,
    pre-activation copy and activation."""
    M, N, K = shape
    _run(layout, M, N, K, 2, torch.bfloat16, act="gelu_tanh", n_add=1, preact=True, seed=5)


@pytest.mark.parametrize("layout", ["NN", "TN"])
@pytest.mark.parametrize("K", [72, 344, 1000, 1048])
def test_bf16_ragged_reduction_length(layout, K):
    """K = 32 n + 8 / 16 / 24 on a large output with B stored [K, N]: regular steps over the first K - K % 32
    columns plus one short step over [K-32, K) whose overlap is zeroed in a scratch copy of B's last rows.
    Inputs are kept large in the overlap so that counting it twice would show."""
    _run(layout, 4096, 8192, K, 1, torch.bfloat16, act="relu", n_add=1, preact=True, seed=7)


def test_bf16_vocab_slice_as_reduction_length():
    # input gradient of a vocabulary-slice classifier, reduced M: dC [2048, 12568] x W [12568, 8192]
    _run("NN", 2048, 8192, 12568, 1, torch.bfloat16, act=None, bias=False, seed=8)


def test_bf16_vocab_slice_classifier_shape():
    # logits of one vocabulary slice: [8192, 2048] x [12568, 2048]^T (reduced K keeps the CPU oracle quick)
    _run("NT", 8192, 12568, 256, 1, torch.bfloat16, act=None, seed=6)


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(4096, 4376, 128), (4096, 4608, 64), (4100, 4480, 192), (8472, 2048, 128)])
def test_bf16_mostly_empty_last_round_goes_to_small_tiles(layout, shape):
    """16 or 17 x 18 tiles of 256 x 256 are one round of the 256 compute units plus 32 or 50 tiles: when the
    remainder is whole tile columns (the first two shapes: 280 and 512 columns) they are a second launch of the
    128 x 128 tile kernel, with their share of the bias, the addend and the pre-activation copy; the third shape's
    remainder (17 x 18 = 306 = 256 + 50, not a multiple of 17) stays in the one launch; the fourth is 34 x 8 tiles,
    whose last 16 are two tile rows (280 rows)."""
    M, N, K = shape
    _run(layout, M, N, K, 2, torch.bfloat16, act="gelu_tanh", n_add=1, preact=True, seed=11)


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(300, 200, 100), (257, 264, 72), (1, 8, 8), (129, 1, 3), (64, 130, 520)])
def test_bf16_ragged(layout, shape):
    M, N, K = shape
    _run(layout, M, N, K, 3, torch.bfloat16, act="relu", seed=3)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_bf16_ragged_big_config(layout):
    # guarded 256x256 path: 4100 x 2056 is not a multiple of the tile
    _run(layout, 4100, 2056, 136, 2, torch.bfloat16, act="gelu_erf", seed=5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_half_small_tile_ring(layout, dtype):
    """Outputs with fewer than 128 tiles of 256 x 256, aligned operands and a reduction that is a multiple of
    64: the ring kernel with 128 x 128 tiles. One and several k-steps, a single k tile, M and N that are not
    tile multiples (last tiles moved back), every epilogue piece, padded leading dimensions."""
    _run(layout, 2048, 2048, 512, 1, dtype, act="gelu_tanh", seed=41)
    _run(layout, 256, 384, 192, 3, dtype, act=None, n_add=2, preact=True, seed=42)
    _run(layout, 128, 128, 64, 1, dtype, act="relu", seed=43)
    _run(layout, 392, 264, 128, 2, dtype, act="gelu_erf", n_add=1, preact=True, seed=44)
    _run(layout, 1024, 136, 320, 1, dtype, act=None, bias=False, pad_a=8, pad_b=24, seed=45)


@pytest.mark.parametrize("act", [None, "gelu_tanh", "gelu_erf", "relu"])
def test_bf16_epilogues_with_preact_and_addends(act):
    _run("NN", 384, 256, 128, 2, torch.bfloat16, act=act, n_add=2, preact=True, seed=7)


def test_bf16_no_bias_no_act():
    _run("NT", 512, 256, 64, 1, torch.bfloat16, act=None, bias=False, seed=9)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_bf16_padded_leading_dimensions(layout):
    _run(layout, 256, 256, 128, 2, torch.bfloat16, act=None, pad_a=8, pad_b=16, seed=11)
    _run(layout, 130, 70, 50, 2, torch.bfloat16, act=None, pad_a=3, pad_b=5, seed=12)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_fp32_exact_and_ragged(layout):
    _run(layout, 256, 384, 128, 2, torch.float32, act="gelu_tanh", seed=13)
    _run(layout, 300, 200, 100, 3, torch.float32, act=None, n_add=1, preact=True, seed=14)
    _run(layout, 7, 5, 3, 1, torch.float32, act="relu", seed=15)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_fp32_tall_tiles(layout):
    """Outputs large enough for the 256-row tiles: exact tiles with addend and pre-activation copy, and a
    ragged shape through the guarded instantiation."""
    _run(layout, 4096, 4096, 32, 2, torch.float32, act="gelu_tanh", n_add=1, preact=True, seed=16)
    _run(layout, 4100, 4104, 40, 1, torch.float32, act="relu", n_add=1, preact=True, seed=17)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_fp32_ring_kernel(layout):
    """fp32 outputs of at least 128 tiles of 256 x 256 with aligned operands: the LDS-ring kernel. Several
    k-steps (the ring runs across the seam between two steps' allocations), addend, pre-activation copy and
    activation; the shortest reduction the ring takes (one stage); M and N that are not tile multiples
    (last tiles moved back to the edge); padded leading dimensions."""
    # 256 x 256 tiles need a total reduction above 2048 (shorter ones take the 128 x 128 tiles)
    _run(layout, 4096, 2048, 704, 3, torch.float32, act="gelu_tanh", n_add=1, preact=True, seed=21)
    _run(layout, 2048, 4096, 2064, 1, torch.float32, act=None, bias=False, seed=22)
    _run(layout, 4104, 2060, 1040, 2, torch.float32, act="relu", n_add=2, preact=True, seed=23)
    _run(layout, 4096, 2048, 2080, 1, torch.float32, act="gelu_erf", pad_a=4, pad_b=8, seed=24)
    # the same outputs with short reductions: 128 x 128 tiles, several rounds of two workgroups per unit
    _run(layout, 4096, 2048, 64, 3, torch.float32, act="gelu_tanh", n_add=1, preact=True, seed=25)
    _run(layout, 2048, 4096, 16, 1, torch.float32, act=None, bias=False, seed=26)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_fp32_ring_kernel_smaller_tiles(layout):
    """Outputs with too few 256 x 256 tiles for the chip: the ring kernel with 128 x 128 tiles (3072 x 2048:
    384 of them) and with 128 x 64 tiles (config 1's gradient shapes, 4096 x 1024), exact and with ragged
    edges, several k-steps, addends and the pre-activation copy."""
    _run(layout, 3072, 2048, 48, 2, torch.float32, act="gelu_tanh", n_add=1, preact=True, seed=31)
    _run(layout, 3080, 2052, 32, 1, torch.float32, act="relu", n_add=2, preact=True, seed=32)
    _run(layout, 4096, 1024, 64, 3, torch.float32, act=None, n_add=1, preact=True, seed=33)
    _run(layout, 4100, 1028, 16, 1, torch.float32, act="gelu_erf", seed=34)
    _run(layout, 4096, 1024, 32, 1, torch.float32, act=None, bias=False, pad_a=4, pad_b=12, seed=35)


def test_fp32_linear1d_col_shape():
    # the fp32 Linear1D workload: x [8,512,1024] fp32, W [4096,1024], b zeros -> F.linear
    import oracle
    from cubework_amd import ops

    x = randn((8 * 512, 1024), torch.float32, 0)
    bound = (6.0 / (1024 + 4096)) ** 0.5
    g = torch.Generator().manual_seed(1)
    W = (torch.rand((4096, 1024), generator=g) * 2 - 1) * bound
    b = torch.zeros(4096)
    want = torch.nn.functional.linear(x, W, b)
    got = ops.gemm_ksteps("NT", [x.cuda()], [W.cuda()], b.cuda())
    assert_parity(got, want, torch.float32, "Linear1D_Col forward")
    assert_parity(got, oracle.gemm_ksteps("NT", [x], [W], b), torch.float32, "oracle")


def test_kstep_sum_equals_concatenated_gemm():
    # size-independent property at the benchmark's Linear2D shape: two k-steps ==
    # one GEMM over the concatenated operands (both through the HIP path)
    from cubework_amd import ops

    dev = "cuda:0"
    A = [randn((8192, 2048), torch.bfloat16, s, device=dev) for s in (0, 1)]
    B = [randn((2048, 2048), torch.bfloat16, s, std=0.02, device=dev) for s in (2, 3)]
    bias = randn((2048,), torch.bfloat16, 4, std=0.02, device=dev)
    two = ops.gemm_ksteps("NN", A, B, bias, "gelu_tanh")
    one = ops.gemm_ksteps("NN", [torch.cat(A, dim=1)], [torch.cat(B, dim=0)], bias, "gelu_tanh")
    torch.cuda.synchronize()
    assert torch.equal(two, one)
    # and a sampled check of rows against the oracle
    import oracle
    rows = torch.tensor([0, 1, 255, 256, 4095, 8191])
    want = oracle.gemm_ksteps("NN", [a[rows].cpu() for a in A], [b.cpu() for b in B], bias.cpu(), "gelu_tanh")
    assert_parity(two[rows.to(dev)], want, torch.bfloat16, "config-2 sampled rows")


@pytest.mark.parametrize("layout", LAYOUTS)
def test_bf16_split_k_long_reduction(layout):
    # 2 x 3 output tiles of 256x256 and k = 2 x 1024: few tiles, long reduction -> the k range of every
    # step is split over several workgroups per tile (cw_gemm_workspace_bytes > 0)
    from cubework_amd import _lib
    from cubework_amd.ops import LAYOUTS as CODES

    assert _lib.load().cw_gemm_workspace_bytes(CODES[layout], 512, 768, 1024, 2, 0) > 0
    _run(layout, 512, 768, 1024, 2, torch.bfloat16, act="gelu_tanh", n_add=1, preact=True, seed=5)
    _run(layout, 512, 768, 1024, 2, torch.bfloat16, act=None, bias=False, seed=6)


def test_split_k_matches_unsplit_call():
    """The same product through cw_gemm_ksteps (no scratch: one workgroup per tile) and through
    cw_gemm_ksteps_ws (split k): both round one fp32 sum to bf16, so they agree to the parity bar, and the
    split result is bit-reproducible from call to call."""
    from cubework_amd import _lib, ops

    dev = "cuda:0"
    M, N, K, steps = 256, 512, 4096, 2
    A = [randn((K, M), torch.bfloat16, 40 + i).to(dev) for i in range(steps)]
    B = [randn((K, N), torch.bfloat16, 50 + i, std=0.05).to(dev) for i in range(steps)]
    lib = _lib.load()
    split1 = ops.gemm_ksteps("TN", A, B)
    split2 = ops.gemm_ksteps("TN", A, B)
    plain = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    rc = lib.cw_gemm_ksteps(ops.LAYOUTS["TN"], M, N, K, steps, ops._ptr_table(A), M, ops._ptr_table(B), N, None, 0,
                            plain.data_ptr(), N, None, 0, None, 0, 0, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.cw_last_error()
    torch.cuda.synchronize()
    assert torch.equal(split1, split2)
    assert_parity(split1, plain.float().cpu(), torch.bfloat16, "split k vs one workgroup per tile")


def test_rejects_bad_arguments():
    from cubework_amd import ops, _lib

    a = torch.zeros((8, 8), dtype=torch.bfloat16, device="cuda:0")
    with pytest.raises(ValueError):
        ops.gemm_ksteps("NN", [a], [torch.zeros((4, 8), dtype=torch.bfloat16, device="cuda:0")])
    with pytest.raises(RuntimeError):
        ops.gemm_ksteps("NN", [a.cpu()], [a.cpu()])
    with pytest.raises(TypeError):
        ops.gemm_ksteps("NN", [a.double()], [a.double()])
    with pytest.raises(TypeError):
        ops.gemm_ksteps("NN", [a.half()], [a])  # operands of two dtypes
    lib = _lib.load()
    rc = lib.cw_gemm_ksteps(7, 8, 8, 8, 1, None, 8, None, 8, None, 0, None, 8, None, 0, None, 0, 0, 0, None)
    assert rc < 0 and b"layout" in lib.cw_last_error()


@pytest.mark.parametrize("shape", [(64, 128, 64), (4096, 2048, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_relu_epilogue_keeps_nan(shape, dtype):
    """torch.relu(NaN) is NaN: a NaN in one row of A reaches exactly that row of the output (register-staged
    and LDS-DMA kernels, fp32 kernel)."""
    import oracle
    from cubework_amd import ops

    M, N, K = shape
    A = randn((M, K), dtype, 1)
    B = randn((K, N), dtype, 2, std=0.1)
    bias = randn((N,), dtype, 3)
    A[5, 7] = float("nan")
    want = oracle.gemm_ksteps("NN", [A], [B], bias, "relu")
    got = ops.gemm_ksteps("NN", [A.cuda()], [B.cuda()], bias.cuda(), "relu").cpu()
    assert torch.isnan(want[5]).all() and torch.equal(torch.isnan(got), torch.isnan(want))
    ok = ~torch.isnan(want)
    assert_parity(got[ok], want[ok], dtype, "relu epilogue beside a NaN row")


def test_ring_kernel_order_of_summation_is_fixed_per_shape_and_bounded_across_shapes():
    """The ring kernel starts each tile's reduction at a k offset that depends on the tile's position (an eighth
    of the range per XCD), and only where M and N are tile multiples. So: (1) the same call twice gives the same
    bits; (2) the same logical product reached another way - as rows of a product whose M is not a tile multiple
    (no rotated start), or with CW_GEMM_IMPL=onelaunch in a fresh process for a shape whose last round of tiles
    is otherwise peeled off into a second launch - may differ in the last bits, by no more than fp32
    reassociation of the K-term sums allows: here at most one bf16 step of the largest magnitude, in few
    elements."""
    import os
    import subprocess
    import sys
    from cubework_amd import ops

    M, N, K = 4096, 4096, 2048       # 256 tiles: the ring kernel, rotated starts
    a = randn((M + 8, K), torch.bfloat16, 71).to(DEV)
    b = randn((K, N), torch.bfloat16, 72, 0.05).to(DEV)
    c1 = ops.gemm_ksteps("NN", [a[:M]], [b])
    c2 = ops.gemm_ksteps("NN", [a[:M]], [b])
    assert torch.equal(c1, c2)
    ragged = ops.gemm_ksteps("NN", [a], [b])[:M]          # M + 8 rows: overlapping last tiles, no rotation
    step = c1.float().abs().max().item() * 2.0 ** -8      # one bf16 step at the largest magnitude
    diff = (c1.float() - ragged.float()).abs()
    assert diff.max().item() <= step
    assert (diff > 0).float().mean().item() < 0.05
    # the second launch for a mostly empty last round, against the one launch (read once per process: a fresh one)
    Ms, Ns, Ks = 4096, 4376, 128
    a2 = randn((Ms, Ks), torch.bfloat16, 73)
    b2 = randn((Ks, Ns), torch.bfloat16, 74, 0.05)
    here = ops.gemm_ksteps("NN", [a2.to(DEV)], [b2.to(DEV)]).cpu()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import sys, torch; sys.path.insert(0, %r)\n"
            "from tests.util import randn\nfrom cubework_amd import ops\n"
            "a = randn((%d, %d), torch.bfloat16, 73).to('cuda:0'); b = randn((%d, %d), torch.bfloat16, 74, 0.05).to('cuda:0')\n"
            "torch.save(ops.gemm_ksteps('NN', [a], [b]).cpu(), sys.argv[1])\n" % (root, Ms, Ks, Ks, Ns))
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "c.pt")
        env = dict(os.environ, CW_GEMM_IMPL="onelaunch")
        proc = subprocess.run([sys.executable, "-c", code, path], capture_output=True, text=True, timeout=300, env=env)
        assert proc.returncode == 0, proc.stdout + proc.stderr
        other = torch.load(path, weights_only=True)
    step = here.float().abs().max().item() * 2.0 ** -8
    diff = (here.float() - other.float()).abs()
    assert diff.max().item() <= step
    assert (diff > 0).float().mean().item() < 0.05
