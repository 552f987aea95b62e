"""GPU tests of the layer API (the drop-in for cubework.module): forward and
backward of each layer against the reference tests' own oracles — plain torch
on the master tensors (tests/test_2d/check_2d_modules.py:77, tests/test_1d/
check_1d_modules.py:74,144, tests/test_3d/check_3d_modules.py:132) — at
tensor-parallel size 1, and as one rank of a 2 x 2 grid / of a 1D pair / of a
2 x 2 x 2 cube / of 4 vocabulary slices with the peers' data pre-staged.

The fp32 tests evaluate the master computation in float64 on the fp32 values (staged peer data is rounded
to fp32, as a peer would send it) and hold every result to 1e-5 of the largest expected magnitude.
"""
import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _leaf(t):
    return t.detach().clone().requires_grad_(True)


def randn64(shape, seed, std=1.0):
    """fp32 values (exactly what the fp32 layers are given) held in float64, for the master computation."""
    return randn(shape, torch.float32, seed, std).double()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["1d", "2d", "3d"])
def test_facade_linear_size1(mode, dtype):
    from cubework_amd.distributed import initialize
    import cubework_amd.module as cube_nn

    initialize(mode, 1)
    layer = cube_nn.Linear(96, 160, dtype=dtype).to(DEV)
    second = cube_nn.Linear(160, 96, dtype=dtype).to(DEV)  # 1d: row-parallel after the column-parallel layer
    x = _leaf(randn((4, 24, 96), dtype, 0).to(DEV))
    dy = randn((4, 24, 96), dtype, 1).to(DEV)
    y = second(layer(x))
    y.backward(dy)
    xr = _leaf(x.detach().double().cpu())
    ws = []
    h = xr
    for lyr in (layer, second):
        w = _leaf(lyr.weight.detach().double().cpu())
        b = _leaf(lyr.bias.detach().double().cpu())
        ws.append((w, b))
        h_in = h if dtype == torch.float32 else h.to(dtype).double()  # the 16-bit layers hand over a rounded tensor
        h = F.linear(h_in, w, b) if mode == "1d" else h_in @ w + b
    h.backward(dy.double().cpu())
    assert_parity(y, h.detach(), dtype, "forward")
    assert_parity(x.grad, xr.grad, dtype, "dX")
    for lyr, (w, b) in zip((layer, second), ws):
        assert_parity(lyr.weight.grad, w.grad, dtype, "dW")
        assert_parity(lyr.bias.grad, b.grad, dtype, "dbias")
    names = set(dict(layer.named_parameters()).keys())
    assert names == {"linear.weight", "linear.bias"} or names == {"linear.linear.weight", "linear.linear.bias"}


@pytest.mark.parametrize("act", ["gelu_tanh", "gelu", "relu"])
def test_linear2d_fused_activation(act):
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_2d import Linear2D

    initialize("2d", 1)
    layer = Linear2D(128, 256, activation=act).to(torch.bfloat16).to(DEV)
    x = _leaf(randn((64, 128), torch.bfloat16, 0).to(DEV))
    dy = randn((64, 256), torch.bfloat16, 1).to(DEV)
    y = layer(x)
    y.backward(dy)
    xr = _leaf(x.detach().float().cpu())
    w = _leaf(layer.weight.detach().float().cpu())
    b = _leaf(layer.bias.detach().float().cpu())
    pre = xr @ w + b
    ref = {"gelu_tanh": lambda t: F.gelu(t, approximate="tanh"), "gelu": F.gelu, "relu": F.relu}[act](pre)
    ref.backward(dy.float().cpu())
    assert_parity(y, ref.detach(), torch.bfloat16, "fused forward")
    assert_parity(x.grad, xr.grad, torch.bfloat16, "dX")
    assert_parity(layer.weight.grad, w.grad, torch.bfloat16, "dW")
    assert_parity(layer.bias.grad, b.grad, torch.bfloat16, "dbias")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_linear2d_residual_addend(dtype):
    """Linear2D's additive `residual` option: residual + x W + b in the GEMM's epilogue, the residual's
    gradient being the output's; the bias gradient arrives in the parameter's dtype (fp32 sums rounded once)."""
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_2d import Linear2D

    initialize("2d", 1)
    layer = Linear2D(128, 256).to(dtype).to(DEV)
    x = _leaf(randn((3, 40, 128), dtype, 0).to(DEV))
    res = _leaf(randn((3, 40, 256), dtype, 2).to(DEV))
    dy = randn((3, 40, 256), dtype, 1).to(DEV)
    y = layer(x, residual=res)
    y.backward(dy)
    xr, rr = _leaf(x.detach().double().cpu()), _leaf(res.detach().double().cpu())
    w = _leaf(layer.weight.detach().double().cpu())
    b = _leaf(layer.bias.detach().double().cpu())
    ref = rr + xr @ w + b
    ref.backward(dy.double().cpu())
    assert_parity(y, ref.detach(), dtype, "residual forward")
    assert_parity(x.grad, xr.grad, dtype, "dX")
    assert torch.equal(res.grad, dy)
    assert_parity(layer.weight.grad, w.grad, dtype, "dW")
    assert layer.bias.grad.dtype == dtype
    assert_parity(layer.bias.grad, b.grad, dtype, "dbias")
    with pytest.raises(ValueError):
        Linear2D(128, 256, activation="relu").to(dtype).to(DEV)(x, residual=res)
    with pytest.raises(AssertionError):
        layer(x, residual=res[:, :, :128])


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_column_sums_stored_in_the_parameter_dtype(out_dtype):
    """The finalize stage stores its fp32 totals as bf16 / fp16 when asked: the same bits as the fp32 result
    cast afterwards (one rounding to nearest even), for every entry point with column sums."""
    from cubework_amd import ops

    io = out_dtype
    dy = randn((700, 520), io, 3).to(DEV)
    pre = randn((700, 520), io, 4).to(DEV)
    assert torch.equal(ops.colsum(dy, out_dtype=out_dtype), ops.colsum(dy).to(out_dtype))
    _, want = ops.act_bwd_colsum("gelu_tanh", dy, pre)
    _, got = ops.act_bwd_colsum("gelu_tanh", dy, pre, out_dtype=out_dtype)
    assert got.dtype == out_dtype and torch.equal(got, want.to(out_dtype))
    x = randn((700, 520), io, 5).to(DEV)
    gamma = randn((520,), io, 6).to(DEV)
    _, mr = ops.ln_forward_fused(x, 1e-5, gamma, None)
    dx0, dg0, db0 = ops.ln_backward_fused(dy, x, mr, gamma)
    dx1, dg1, db1 = ops.ln_backward_fused(dy, x, mr, gamma, param_dtype=out_dtype)
    assert torch.equal(dx0, dx1) and torch.equal(dg1, dg0.to(out_dtype)) and torch.equal(db1, db0.to(out_dtype))
    rs0, dg0, db0 = ops.ln_bwd_partials(dy, x, mr, gamma)
    rs1, dg1, db1 = ops.ln_bwd_partials(dy, x, mr, gamma, param_dtype=out_dtype)
    assert torch.equal(rs0, rs1) and torch.equal(dg1, dg0.to(out_dtype)) and torch.equal(db1, db0.to(out_dtype))
    rs, pending = ops.ln_bwd_partials_open(dy, x, mr, gamma)
    _, dg0, db0 = ops.ln_bwd_dx_close(dy, x, mr, rs, 520, pending, gamma)
    _, dg1, db1 = ops.ln_bwd_dx_close(dy, x, mr, rs, 520, pending, gamma, param_dtype=out_dtype)
    assert torch.equal(dg1, dg0.to(out_dtype)) and torch.equal(db1, db0.to(out_dtype))
    with pytest.raises(TypeError):
        ops.colsum(dy, out_dtype=torch.float64)


def test_skip_bias_add_and_errors():
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_1d import Linear1D_Col, Linear1D_Row
    from cubework_amd.module.parallel_2d import Linear2D

    initialize("2d", 1)
    layer = Linear2D(64, 64, skip_bias_add=True).to(DEV)
    out, bias = layer(randn((8, 64), torch.float32, 0).to(DEV))
    assert out.shape == (8, 64) and torch.equal(bias, layer.bias.detach())
    with pytest.raises(AssertionError):
        layer(torch.zeros((8, 32), device=DEV))  # "Invalid shapes ... for AB."
    initialize("1d", 1)
    with pytest.raises(ValueError):
        Linear1D_Col(8, 8, bias=False, skip_bias_add=True)
    with pytest.raises(ValueError):
        Linear1D_Row(8, 8, bias=False, skip_bias_add=True)
    col = Linear1D_Col(64, 64, skip_bias_add=True).to(DEV)
    o, b = col(randn((8, 64), torch.float32, 0).to(DEV))
    assert b is col.bias and o.shape == (8, 64)
    initialize(None, 1)
    with pytest.raises(AssertionError):
        Linear2D(8, 8)  # 2D groups not initialised


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["2d", "3d"])
def test_facade_layernorm_size1(mode, dtype):
    from cubework_amd.distributed import initialize
    import cubework_amd.module as cube_nn

    initialize(mode, 1)
    H = 512
    norm = cube_nn.LayerNorm(H, eps=1e-5, dtype=dtype).to(DEV)
    with torch.no_grad():
        norm.weight.copy_(torch.rand(H) * 0.2 + 0.9)
        norm.bias.copy_(torch.randn(H) * 0.02)
    x = _leaf(randn((6, 20, H), dtype, 3).to(DEV))
    dy = randn((6, 20, H), dtype, 4).to(DEV)
    y = norm(x)
    y.backward(dy)
    xr = _leaf(x.detach().double().cpu())
    g = _leaf(norm.weight.detach().double().cpu())
    b = _leaf(norm.bias.detach().double().cpu())
    ref = F.layer_norm(xr, (H,), g, b, 1e-5)
    ref.backward(dy.double().cpu())
    assert_parity(y, ref.detach(), dtype, "forward")
    assert_parity(x.grad, xr.grad, dtype, "dX")
    assert_parity(norm.weight.grad, g.grad, dtype, "dgamma")
    assert_parity(norm.bias.grad, b.grad, dtype, "dbeta")


@pytest.mark.parametrize("mode", ["1d", "2d", "3d"])
@pytest.mark.parametrize("vocab_parallel", [False, True])
def test_facade_classifier_and_loss_size1(mode, vocab_parallel):
    from cubework_amd.distributed import initialize
    from cubework_amd.global_vars import env
    import cubework_amd.module as cube_nn

    initialize(mode, 1)
    env.vocab_parallel = vocab_parallel
    head = cube_nn.Classifier(128, 520, dtype=torch.float32).to(DEV)
    crit = cube_nn.CrossEntropyLoss()
    x = _leaf(randn((48, 128), torch.float32, 5).to(DEV))
    t = torch.randint(0, 520, (48,), generator=torch.Generator().manual_seed(6)).to(DEV)
    loss = crit(head(x), t)
    loss.backward()
    xr = _leaf(x.detach().double().cpu())
    w = _leaf(head.weight.detach().double().cpu())
    b = _leaf(head.bias.detach().double().cpu())
    ref = F.cross_entropy(F.linear(xr, w, b), t.cpu())
    ref.backward()
    assert_parity(loss, ref.detach(), torch.float32, "loss")
    assert_parity(x.grad, xr.grad, torch.float32, "dX")
    assert_parity(head.weight.grad, w.grad, torch.float32, "dW")
    assert_parity(head.bias.grad, b.grad, torch.float32, "dbias")


def test_linear2d_one_rank_of_2x2_grid():
    """Rank (row 0, col 1) of a 2 x 2 grid, peers' operands pre-staged; checked
    against the master computation with the reference test's shard layout
    (tests/test_2d/check_2d_modules.py:38-110)."""
    import oracle
    from oracle.grid import bias_shard, shard
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.parallel_2d import Linear2D

    q, i, j = 2, 0, 1
    B_, S_, IN, OUT = 8, 4, 256, 384
    dt = torch.float32
    A_master = randn64((B_, S_, IN), 0)
    W_master = randn64((IN, OUT), 1, std=0.05)
    b_master = randn64((OUT,), 2)
    dC_master = randn64((B_, S_, OUT), 3)
    A2, dC2 = A_master.reshape(-1, IN), dC_master.reshape(-1, OUT)

    initialize("2d", q * q, row=i, col=j)
    layer = Linear2D(IN, OUT).to(DEV)
    assert layer.weight.shape == (IN // q, OUT // q) and layer.bias.shape == (OUT // q ** 2,)
    with torch.no_grad():
        layer.weight.copy_(shard(W_master, q, i, j))
        layer.bias.copy_(bias_shard(b_master, q, i, j))
    row, col = pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    # forward: step 0's A comes from the rank at column 0 of my row, step 0's B is mine? no: B_k comes from row k
    row.stage("broadcast", d(shard(A2, q, i, 0)))           # A of step 0 (I am column 1)
    col.stage("broadcast", d(shard(W_master, q, 1, j)))     # B of step 1 (I am row 0)
    col.stage("all_gather", [None, d(bias_shard(b_master, q, 1, j))])
    x = _leaf(d(shard(A2, q, i, j)))
    out = layer(x)
    C_master = A2 @ W_master + b_master
    assert_parity(out, shard(C_master, q, i, j), dt, "Linear2D forward shard")

    # backward: every "collective" of the three backward operators, in the order they run
    dC = shard(dC2, q, i, j)
    gemm = lambda *a: oracle.gemm_ksteps(*a, compute_dtype=torch.float64)  # noqa: E731
    col.stage("reduce_scatter", [d(shard(dC2, q, 1, j).sum(0))])                    # peers' bias-grad column sums
    col.stage("broadcast", d(shard(W_master, q, 1, j)))                             # summa_ABT: B of step 1
    row.stage("reduce", [d(gemm("NT", [shard(dC2, q, i, 0)], [shard(W_master, q, j, 0)]))])  # peer's product for my column
    row.stage("broadcast", d(shard(A2, q, i, 0)))                                   # summa_ATB: A of step 0
    col.stage("reduce", [d(gemm("TN", [shard(A2, q, 1, i)], [shard(dC2, q, 1, j)]))])        # peer's product for my row
    out.backward(d(dC))
    dA_master = dC2 @ W_master.t()
    dW_master = A2.t() @ dC2
    assert_parity(x.grad, shard(dA_master, q, i, j), dt, "dA shard")
    assert_parity(layer.weight.grad, shard(dW_master, q, i, j), dt, "dW shard")
    assert_parity(layer.bias.grad, bias_shard(dC2.sum(0), q, i, j), dt, "dbias shard")
    # what this rank would have sent: its products for the peers
    sent_row = dict(row.outbox["reduce"])
    assert_parity(sent_row[0], gemm("NT", [dC], [shard(W_master, q, 0, j)]), dt, "product sent to column 0")
    assert not any(row.inbox.values()) and not any(col.inbox.values())


@pytest.mark.parametrize("rank", [0, 1])
def test_linear1d_col_row_one_rank_of_two(rank):
    """Column-parallel then row-parallel Linear1D (the Megatron MLP the reference's 1D mode builds from two
    `Linear`s, parallel_1d/module.py:38-58) as one rank of two, the peer's partial product and input gradient
    pre-staged; checked against the master computation as tests/test_1d/check_1d_modules.py:38-150 does."""
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.parallel_1d import Linear1D_Col, Linear1D_Row

    p, other = 2, 1 - rank
    T_, IN, HID, OUT = 48, 128, 256, 192
    dt = torch.float32
    X = randn64((T_, IN), 0)
    W1, b1 = randn64((HID, IN), 1, std=0.05), randn64((HID,), 2)
    W2, b2 = randn64((OUT, HID), 3, std=0.05), randn64((OUT,), 4)
    dY = randn64((T_, OUT), 5)
    Xr, W1r, b1r, W2r, b2r = (_leaf(t) for t in (X, W1, b1, W2, b2))
    ref = F.linear(F.gelu(F.linear(Xr, W1r, b1r), approximate="tanh"), W2r, b2r)
    ref.backward(dY)
    rows = lambda t, r: torch.chunk(t, p, dim=0)[r]   # noqa: E731  column-parallel: output features
    cols = lambda t, r: torch.chunk(t, p, dim=-1)[r]  # noqa: E731  row-parallel: input features

    initialize("1d", p, rank=rank)
    col = Linear1D_Col(IN, HID, activation="gelu_tanh").to(DEV)
    row = Linear1D_Row(HID, OUT).to(DEV)
    assert col.weight.shape == (HID // p, IN) and col.bias.shape == (HID // p,)
    assert row.weight.shape == (OUT, HID // p) and row.bias.shape == (OUT,)
    with torch.no_grad():
        col.weight.copy_(rows(W1, rank)); col.bias.copy_(rows(b1, rank))
        row.weight.copy_(cols(W2, rank)); row.bias.copy_(b2)
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    mode = pm.PARALLEL_1D
    h_other = F.gelu(F.linear(X, rows(W1, other), rows(b1, other)), approximate="tanh")
    mode.stage("all_reduce", [d(h_other @ cols(W2, other).t())])          # the peer's partial product
    x = _leaf(d(X))
    y = row(col(x))
    assert_parity(y, ref.detach(), dt, "Linear1D col->row forward")
    # backward: the peer's share of the input gradient arrives through the all-reduce of reduce_grad
    pre_other = F.linear(X, rows(W1, other), rows(b1, other))
    _g = _leaf(pre_other)
    F.gelu(_g, approximate="tanh").backward(dY @ cols(W2, other))
    mode.stage("all_reduce", [d(_g.grad @ rows(W1, other))])
    y.backward(d(dY))
    assert_parity(x.grad, Xr.grad, dt, "dX")
    assert_parity(col.weight.grad, rows(W1r.grad, rank), dt, "column-parallel dW shard")
    assert_parity(col.bias.grad, rows(b1r.grad, rank), dt, "column-parallel dbias shard")
    assert_parity(row.weight.grad, cols(W2r.grad, rank), dt, "row-parallel dW shard")
    assert_parity(row.bias.grad, b2r.grad, dt, "row-parallel dbias")
    assert not any(mode.inbox.values())


def test_linear3d_one_rank_of_2x2x2_cube():
    """Linear3D as rank (input 1, weight 0, output 1) of a depth-2 cube with the reference test's shard layout
    (tests/test_3d/check_3d_modules.py:40-110: j = input rank, i = weight rank, k = output rank), every
    gather / reduce-scatter the operator performs pre-staged from the master tensors."""
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_3d import Linear3D

    dep, j, i, k = 2, 1, 0, 1
    B_, S_, IN, OUT = 8, 4, 128, 256
    dt = torch.float32
    A_m = randn64((B_, S_, IN), 0)
    W_m = randn64((IN, OUT), 1, std=0.05)
    b_m = randn64((OUT,), 2)
    G_m = randn64((B_, S_, OUT), 3)
    ch = lambda t, dim, r: torch.chunk(t, dep, dim=dim)[r]  # noqa: E731
    a_shard = lambda jj, ii, kk: ch(ch(ch(A_m, 0, ii), -1, kk), 0, jj)    # noqa: E731  [B/d^2, S, IN/d]
    w_shard = lambda jj, ii, kk: ch(ch(ch(W_m, 0, kk), -1, jj), -1, ii)   # noqa: E731  [IN/d, OUT/d^2]
    c_shard = lambda t, jj, ii, kk: ch(ch(ch(t, 0, ii), -1, jj), 0, kk)   # noqa: E731  [B/d^2, S, OUT/d]
    a_rows = lambda ii, kk: ch(ch(A_m, 0, ii), -1, kk)                    # noqa: E731  gathered over the input group
    w_blk = lambda jj, kk: ch(ch(W_m, 0, kk), -1, jj)                     # noqa: E731  gathered over the weight group
    g_rows = lambda ii, jj: ch(ch(G_m, 0, ii), -1, jj)                    # noqa: E731  gathered over the output group

    initialize("3d", dep ** 3, coords=(j, i, k))
    layer = Linear3D(IN, OUT).to(DEV)
    in_mode, w_mode, out_mode = layer.input_parallel_mode, layer.weight_parallel_mode, layer.output_parallel_mode
    assert (in_mode.local_rank, w_mode.local_rank, out_mode.local_rank) == (j, i, k)
    assert layer.weight.shape == (IN // dep, OUT // dep ** 2) and layer.bias.shape == (OUT // dep,)
    with torch.no_grad():
        layer.weight.copy_(w_shard(j, i, k))
        layer.bias.copy_(ch(b_m, 0, j))
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    in_mode.stage("all_gather", [d(a_shard(jj, i, k)) for jj in range(dep)])
    w_mode.stage("all_gather", [d(w_shard(j, ii, k)) for ii in range(dep)])
    out_mode.stage("reduce_scatter", [d(a_rows(i, kk) @ w_blk(j, kk)) for kk in range(dep) if kk != k])
    x = _leaf(d(a_shard(j, i, k)))
    out = layer(x)
    A_r, W_r, b_r = _leaf(A_m), _leaf(W_m), _leaf(b_m)
    C_m = A_r @ W_r + b_r
    C_m.backward(G_m)
    assert_parity(out, c_shard(C_m.detach(), j, i, k), dt, "Linear3D forward shard")

    flat = lambda t: t.reshape(-1, t.shape[-1])  # noqa: E731
    out_mode.stage("all_gather", [d(c_shard(G_m, j, i, kk)) for kk in range(dep)])
    w_mode.stage("all_reduce", [d(flat(g_rows(ii, j)).sum(0)) for ii in range(dep) if ii != i])
    w_mode.stage("reduce_scatter", [d(flat(a_rows(ii, k)).t() @ flat(g_rows(ii, j))) for ii in range(dep) if ii != i])
    in_mode.stage("reduce_scatter", [d(g_rows(i, jj) @ w_blk(jj, k).t()) for jj in range(dep) if jj != j])
    out.backward(d(c_shard(G_m, j, i, k)))
    assert_parity(x.grad, a_shard_of(A_r.grad, dep, j, i, k), dt, "dA shard")
    assert_parity(layer.weight.grad, ch(ch(ch(W_r.grad, 0, k), -1, j), -1, i), dt, "dW shard")
    assert_parity(layer.bias.grad, ch(b_r.grad, 0, j), dt, "dbias shard")
    assert not any(in_mode.inbox.values()) and not any(w_mode.inbox.values()) and not any(out_mode.inbox.values())


@pytest.mark.usefixtures("oracle64")
def test_layernorm3d_one_rank_of_2x2x2_cube():
    """LayerNorm3D (two-pass statistics, parallel_3d/_operation.py:256-313) as rank (input 0, weight 1,
    output 1) of a depth-2 cube with the shard layout of tests/test_3d/check_3d_modules.py:137-173: the
    output-group peer holds the other half of every row, the other row shards contribute to dgamma / dbeta."""
    import oracle
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_3d import LayerNorm3D

    dep, j, i, k = 2, 0, 1, 1
    R, H, eps = 16, 512, 1e-6
    dt = torch.float32
    A = randn64((R, H), 0)
    dY = randn64((R, H), 1)
    gamma = (torch.rand(H, generator=torch.Generator().manual_seed(2)) * 0.2 + 0.9).double()
    beta = randn64((H,), 3, std=0.02)
    ch = lambda t, dim, r: torch.chunk(t, dep, dim=dim)[r]  # noqa: E731
    rows_of = lambda t, jj, ii: ch(ch(t, 0, ii), 0, jj)     # noqa: E731

    initialize("3d", dep ** 3, coords=(j, i, k))
    norm = LayerNorm3D(H, eps).to(DEV)
    assert norm.weight.shape == (H // dep,)
    with torch.no_grad():
        norm.weight.copy_(ch(gamma, 0, k))
        norm.bias.copy_(ch(beta, 0, k))
    out_mode, ixw_mode = norm.output_parallel_mode, norm.input_x_weight_parallel_mode
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    my_rows, peer_k = rows_of(A, j, i), 1 - k
    mean = my_rows.mean(-1)
    out_mode.stage("all_reduce", [d(ch(my_rows, -1, peer_k).sum(-1))])                           # sum x
    out_mode.stage("all_reduce", [d(((ch(my_rows, -1, peer_k) - mean[:, None]) ** 2).sum(-1))])  # sum (x - mean)^2
    x = _leaf(d(ch(my_rows, -1, k)))
    y = norm(x)
    Ar, gr, br = _leaf(A), _leaf(gamma), _leaf(beta)
    ref = F.layer_norm(Ar, (H,), gr, br, eps)
    ref.backward(dY)
    assert_parity(y, ch(rows_of(ref.detach(), j, i), -1, k), dt, "LayerNorm3D forward shard")

    var = A.var(-1, unbiased=False)
    mr = torch.stack([A.mean(-1), 1.0 / torch.sqrt(var + eps)], dim=-1)
    rs_peer, _, _ = oracle.ln2d_backward_partials(ch(rows_of(dY, j, i), -1, peer_k), ch(my_rows, -1, peer_k),
                                                  rows_of(mr, j, i), ch(gamma, 0, peer_k))
    out_mode.stage("all_reduce", [d(rs_peer)])
    others = [(jj, ii) for jj in range(dep) for ii in range(dep) if (jj, ii) != (j, i)]
    parts = [oracle.ln2d_backward_partials(ch(rows_of(dY, jj, ii), -1, k), ch(rows_of(A, jj, ii), -1, k),
                                           rows_of(mr, jj, ii), ch(gamma, 0, k)) for jj, ii in others]
    ixw_mode.stage("all_reduce", [d(p_[1]) for p_ in parts])
    ixw_mode.stage("all_reduce", [d(p_[2]) for p_ in parts])
    y.backward(d(ch(rows_of(dY, j, i), -1, k)))
    assert_parity(x.grad, ch(rows_of(Ar.grad, j, i), -1, k), dt, "dX shard")
    assert_parity(norm.weight.grad, ch(gr.grad, 0, k), dt, "dgamma shard")
    assert_parity(norm.bias.grad, ch(br.grad, 0, k), dt, "dbeta shard")
    assert not any(out_mode.inbox.values()) and not any(ixw_mode.inbox.values())


def a_shard_of(t, dep, j, i, k):
    """The activation shard of rank (input j, weight i, output k): rows chunk i then j, columns chunk k."""
    ch = lambda x, dim, r: torch.chunk(x, dep, dim=dim)[r]  # noqa: E731
    return ch(ch(ch(t, 0, i), -1, k), 0, j)


def test_classifier2d_one_rank_of_2x2_grid():
    """Classifier2D (parallel_2d/_operation.py:364-419) as rank (row 1, col 0) of a 2 x 2 grid with the shard
    layout of tests/test_2d/check_2d_modules.py:345-403: the column peers' weight slices, the row peer's
    partial product and the column peers' gradient contributions pre-staged."""
    from oracle.grid import shard
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.parallel_2d import Classifier2D

    q, i, j = 2, 1, 0
    B_, S_, IN, NC = 8, 4, 256, 40
    dt = torch.float32
    A_m = randn64((B_ * S_, IN), 0)
    W_m = randn64((NC, IN), 1, std=0.05)
    b_m = randn64((NC,), 2)
    G_m = randn64((B_ * S_, NC), 3)
    ch = lambda t, dim, r: torch.chunk(t, q, dim=dim)[r]  # noqa: E731
    w_shard = lambda ii, jj: ch(ch(W_m, -1, jj), -1, ii)   # noqa: E731  [NC, IN/q^2]

    initialize("2d", q * q, row=i, col=j)
    head = Classifier2D(IN, NC).to(DEV)
    assert head.weight.shape == (NC, IN // q ** 2) and head.bias.shape == (NC,)
    with torch.no_grad():
        head.weight.copy_(w_shard(i, j))
        head.bias.copy_(b_m)
    row, col = pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    col.stage("all_gather", [d(w_shard(ii, j)) for ii in range(q)])
    row.stage("all_reduce", [d(shard(A_m, q, i, jj) @ ch(W_m, -1, jj).t()) for jj in range(q) if jj != j])
    x = _leaf(d(shard(A_m, q, i, j)))
    out = head(x)
    Ar, Wr, br = _leaf(A_m), _leaf(W_m), _leaf(b_m)
    C_m = F.linear(Ar, Wr, br)
    C_m.backward(G_m)
    assert_parity(out, ch(C_m.detach(), 0, i), dt, "Classifier2D forward rows")
    col.stage("reduce_scatter", [d(ch(G_m, 0, ii).t() @ shard(A_m, q, ii, j)) for ii in range(q) if ii != i])
    col.stage("all_reduce", [d(ch(G_m, 0, ii).sum(0)) for ii in range(q) if ii != i])
    out.backward(d(ch(G_m, 0, i)))
    assert_parity(x.grad, shard(Ar.grad, q, i, j), dt, "dA shard")
    assert_parity(head.weight.grad, ch(ch(Wr.grad, -1, j), -1, i), dt, "dW shard")
    assert_parity(head.bias.grad, br.grad, dt, "dbias")
    assert not any(row.inbox.values()) and not any(col.inbox.values())


@pytest.mark.parametrize("pos", [(0, 1), (1, 0)])
def test_vocab_parallel_classifier2d_one_rank_of_2x2_grid(pos):
    """VocabParallelClassifier2D (summa_ABT forward, summa_AB / summa_ATB backward: the lm head of the 2D
    models) as one rank of a 2 x 2 grid with the shard layout of tests/test_2d/check_2d_modules.py:422-478."""
    import oracle
    from oracle.grid import bias_shard, shard
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.parallel_2d import VocabParallelClassifier2D

    q = 2
    i, j = pos
    oi, oj = 1 - i, 1 - j
    T_, IN, V = 32, 256, 512
    dt = torch.float32
    A_m = randn64((T_, IN), 0)
    W_m = randn64((V, IN), 1, std=0.05)
    b_m = randn64((V,), 2)
    G_m = randn64((T_, V), 3)
    a, w, g_ = (lambda r, c: shard(A_m, q, r, c)), (lambda r, c: shard(W_m, q, r, c)), (lambda r, c: shard(G_m, q, r, c))  # noqa: E731

    initialize("2d", q * q, row=i, col=j)
    head = VocabParallelClassifier2D(IN, V).to(DEV)
    assert head.weight.shape == (V // q, IN // q) and head.bias.shape == (V // q ** 2,)
    with torch.no_grad():
        head.weight.copy_(w(i, j))
        head.bias.copy_(bias_shard(b_m, q, i, j))
    row, col = pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    gemm = lambda *a: oracle.gemm_ksteps(*a, compute_dtype=torch.float64)  # noqa: E731
    # forward, summa_ABT: the weight block of the other grid row arrives by broadcast; my output block
    # C[i, j] = sum_k A[i, k] W[j, k]^T collects the row peer's product
    col.stage("broadcast", d(w(oi, j)))
    row.stage("reduce", [d(gemm("NT", [a(i, oj)], [w(j, oj)]))])
    gathered = [None, None]
    gathered[oi] = d(bias_shard(b_m, q, oi, j))
    col.stage("all_gather", gathered)
    x = _leaf(d(a(i, j)))
    out = head(x)
    Ar, Wr, br = _leaf(A_m), _leaf(W_m), _leaf(b_m)
    C_m = F.linear(Ar, Wr, br)
    C_m.backward(G_m)
    assert_parity(out, shard(C_m.detach(), q, i, j), dt, "logits shard")
    # backward: bias column sums of the column peer; summa_AB (dA[i, j] = sum_t G[i, t] W[t, j]) and
    # summa_ATB (dW[i, j] = sum_t G[t, i]^T A[t, j]) with their broadcasts and the column peer's product
    col.stage("reduce_scatter", [d(g_(oi, j).sum(0))])
    row.stage("broadcast", d(g_(i, oj)))
    col.stage("broadcast", d(w(oi, j)))
    row.stage("broadcast", d(g_(i, oj)))
    col.stage("reduce", [d(gemm("TN", [g_(oi, i)], [a(oi, j)]))])
    out.backward(d(g_(i, j)))
    assert_parity(x.grad, shard(Ar.grad, q, i, j), dt, "dA shard")
    assert_parity(head.weight.grad, shard(Wr.grad, q, i, j), dt, "dW shard")
    assert_parity(head.bias.grad, bias_shard(br.grad, q, i, j), dt, "dbias shard")
    assert not any(row.inbox.values()) and not any(col.inbox.values())


@pytest.mark.parametrize("coords", [(1, 0, 1), (0, 1, 1)])
def test_classifier3d_one_rank_of_2x2x2_cube(coords):
    """Classifier3D (parallel_3d/_operation.py:91-152) as one rank of a depth-2 cube with the shard layout of
    tests/test_3d/check_3d_modules.py:199-286 (j = input rank, i = weight rank, k = output rank): weight
    [classes, in/d] = column chunk k, activation rows chunk i then j and columns chunk k, output rows chunk i
    then j with all classes. Rank (1, 0, 1) is the destination of the weight-gradient reduce over its input group
    (input rank == output rank) and goes on to the all-reduce over the weight group; rank (0, 1, 1) receives
    the weight by broadcast, sends its product away and keeps no weight gradient."""
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_3d import Classifier3D

    dep = 2
    j, i, k = coords
    B_, S_, IN, NC = 8, 4, 128, 40
    dt = torch.float32
    A_m, W_m, b_m, G_m = randn64((B_, S_, IN), 0), randn64((NC, IN), 1, std=0.05), randn64((NC,), 2), randn64((B_, S_, NC), 3)
    ch = lambda t, dim, r: torch.chunk(t, dep, dim=dim)[r]  # noqa: E731
    a_shard = lambda jj, ii, kk: ch(ch(ch(A_m, 0, ii), -1, kk), 0, jj)   # noqa: E731  [B/d^2, S, IN/d]
    g_shard = lambda jj, ii: ch(ch(G_m, 0, ii), 0, jj)                    # noqa: E731  [B/d^2, S, NC]
    flat = lambda t: t.reshape(-1, t.shape[-1])                           # noqa: E731
    d = lambda t: t.to(DEV, dt)                                           # noqa: E731

    initialize("3d", dep ** 3, coords=(j, i, k))
    head = Classifier3D(IN, NC).to(DEV)
    in_mode, w_mode, out_mode = head.input_parallel_mode, head.weight_parallel_mode, head.output_parallel_mode
    assert head.weight.shape == (NC, IN // dep) and head.bias.shape == (NC,)
    with torch.no_grad():
        head.weight.copy_(ch(W_m, -1, k))
        head.bias.copy_(b_m)
    is_dst = j == k
    if not is_dst:
        in_mode.stage("broadcast", d(ch(W_m, -1, k)))   # from the input-group member whose input rank equals my output rank
    out_mode.stage("all_reduce", [d(flat(a_shard(j, i, kk)) @ ch(W_m, -1, kk).t()) for kk in range(dep) if kk != k])
    x = _leaf(d(a_shard(j, i, k)))
    out = head(x)
    Ar, Wr, br = _leaf(A_m), _leaf(W_m), _leaf(b_m)
    C_m = F.linear(Ar, Wr, br)
    C_m.backward(G_m)
    assert_parity(out, ch(ch(C_m.detach(), 0, i), 0, j), dt, "Classifier3D forward rows")

    dW_of = lambda jj, ii: flat(g_shard(jj, ii)).t() @ flat(a_shard(jj, ii, k))   # noqa: E731  one rank's product
    if is_dst:
        in_mode.stage("reduce", [d(dW_of(jj, i)) for jj in range(dep) if jj != j])
        w_mode.stage("all_reduce", [d(sum(dW_of(jj, ii) for jj in range(dep))) for ii in range(dep) if ii != i])
    in_mode.stage("all_reduce", [d(flat(g_shard(jj, i)).sum(0)) for jj in range(dep) if jj != j])
    w_mode.stage("all_reduce", [d(sum(flat(g_shard(jj, ii)).sum(0) for jj in range(dep))) for ii in range(dep) if ii != i])
    out.backward(d(g_shard(j, i)))
    assert_parity(x.grad, a_shard_of(Ar.grad, dep, j, i, k), dt, "dA shard")
    assert_parity(head.bias.grad, br.grad, dt, "dbias")
    if is_dst:
        assert_parity(head.weight.grad, ch(Wr.grad, -1, k), dt, "dW column chunk")
    else:
        assert head.weight.grad is None
        (dst, sent), = in_mode.outbox["reduce"]
        assert dst == k
        assert_parity(sent, dW_of(j, i), dt, "product sent to the weight's owner")
    assert not any(in_mode.inbox.values()) and not any(w_mode.inbox.values()) and not any(out_mode.inbox.values())


def test_vocab_parallel_classifier3d_one_rank_of_2x2x2_cube():
    """VocabParallelClassifier3D (parallel_3d/_operation.py:167-229) as rank (input 1, weight 0, output 1) of a
    depth-2 cube with the shard layout of tests/test_3d/check_3d_modules.py:289-380: weight [classes/d^2, in/d]
    = class chunk j then i, input chunk k; bias chunk j; output rows chunk i, classes chunk j, rows chunk k."""
    from cubework_amd.distributed import initialize
    from cubework_amd.module.parallel_3d import VocabParallelClassifier3D

    dep, j, i, k = 2, 1, 0, 1
    B_, S_, IN, V = 8, 4, 128, 256
    dt = torch.float32
    A_m, W_m, b_m, G_m = randn64((B_, S_, IN), 0), randn64((V, IN), 1, std=0.05), randn64((V,), 2), randn64((B_, S_, V), 3)
    ch = lambda t, dim, r: torch.chunk(t, dep, dim=dim)[r]  # noqa: E731
    a_shard = lambda jj, ii, kk: ch(ch(ch(A_m, 0, ii), -1, kk), 0, jj)    # noqa: E731  [B/d^2, S, IN/d]
    a_rows = lambda ii, kk: ch(ch(A_m, 0, ii), -1, kk)                     # noqa: E731  gathered over the input group
    w_shard = lambda jj, ii, kk: ch(ch(ch(W_m, 0, jj), 0, ii), -1, kk)     # noqa: E731  [V/d^2, IN/d]
    w_blk = lambda jj, kk: ch(ch(W_m, 0, jj), -1, kk)                      # noqa: E731  gathered over the weight group: [V/d, IN/d]
    c_shard = lambda t, jj, ii, kk: ch(ch(ch(t, 0, ii), -1, jj), 0, kk)    # noqa: E731  [B/d^2, S, V/d]
    g_rows = lambda ii, jj: ch(ch(G_m, 0, ii), -1, jj)                     # noqa: E731  gathered over the output group
    flat = lambda t: t.reshape(-1, t.shape[-1])                            # noqa: E731
    d = lambda t: t.to(DEV, dt)                                            # noqa: E731

    initialize("3d", dep ** 3, coords=(j, i, k))
    head = VocabParallelClassifier3D(IN, V).to(DEV)
    in_mode, w_mode, out_mode = head.input_parallel_mode, head.weight_parallel_mode, head.output_parallel_mode
    assert (in_mode.local_rank, w_mode.local_rank, out_mode.local_rank) == (j, i, k)
    assert head.weight.shape == (V // dep ** 2, IN // dep) and head.bias.shape == (V // dep,)
    with torch.no_grad():
        head.weight.copy_(w_shard(j, i, k))
        head.bias.copy_(ch(b_m, 0, j))
    in_mode.stage("all_gather", [d(a_shard(jj, i, k)) for jj in range(dep)])
    w_mode.stage("all_gather", [d(w_shard(j, ii, k).t()) for ii in range(dep)])
    out_mode.stage("reduce_scatter", [d(a_rows(i, kk) @ w_blk(j, kk).t()) for kk in range(dep) if kk != k])
    x = _leaf(d(a_shard(j, i, k)))
    out = head(x)
    Ar, Wr, br = _leaf(A_m), _leaf(W_m), _leaf(b_m)
    C_m = F.linear(Ar, Wr, br)
    C_m.backward(G_m)
    assert_parity(out, c_shard(C_m.detach(), j, i, k), dt, "VocabParallelClassifier3D logits shard")

    out_mode.stage("all_gather", [d(c_shard(G_m, j, i, kk)) for kk in range(dep)])
    w_mode.stage("reduce_scatter", [d((flat(a_rows(ii, k)).t() @ flat(g_rows(ii, j))).t()) for ii in range(dep) if ii != i])
    w_mode.stage("all_reduce", [d(flat(g_rows(ii, j)).sum(0)) for ii in range(dep) if ii != i])
    in_mode.stage("reduce_scatter", [d(g_rows(i, jj) @ w_blk(jj, k)) for jj in range(dep) if jj != j])
    out.backward(d(c_shard(G_m, j, i, k)))
    assert_parity(x.grad, a_shard_of(Ar.grad, dep, j, i, k), dt, "dA shard")
    assert_parity(head.weight.grad, ch(ch(ch(Wr.grad, 0, j), 0, i), -1, k), dt, "dW shard")
    assert_parity(head.bias.grad, ch(br.grad, 0, j), dt, "dbias shard")
    assert not any(in_mode.inbox.values()) and not any(w_mode.inbox.values()) and not any(out_mode.inbox.values())


def test_linear2d_missing_peer_data_is_an_error():
    from cubework_amd.distributed import MissingPeerData, initialize
    from cubework_amd.module.parallel_2d import Linear2D

    initialize("2d", 4, row=0, col=0)
    layer = Linear2D(64, 64).to(DEV)
    with pytest.raises(MissingPeerData):
        layer(torch.zeros((4, 32), device=DEV))


@pytest.mark.usefixtures("oracle64")
def test_layernorm2d_one_rank_of_2x2_grid():
    """tests/test_2d/check_2d_modules.py:113-162 for one rank, with affine."""
    from oracle.grid import bias_shard, shard
    import oracle
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.parallel_2d import LayerNorm2D

    q, i, j = 2, 1, 0
    R, H, eps = 16, 512, 1e-5
    dt = torch.float32
    A = randn64((R, H), 0)
    dY = randn64((R, H), 1)
    gamma = (torch.rand(H, generator=torch.Generator().manual_seed(2)) * 0.2 + 0.9).double()
    beta = randn64((H,), 3, std=0.02)
    initialize("2d", q * q, row=i, col=j)
    norm = LayerNorm2D(H, eps).to(DEV)
    assert norm.weight.shape == (H // q ** 2,)
    with torch.no_grad():
        norm.weight.copy_(bias_shard(gamma, q, i, j))
        norm.bias.copy_(bias_shard(beta, q, i, j))
    row, col = pm.PARALLEL_2D_ROW, pm.PARALLEL_2D_COL
    d = lambda t: t.to(DEV, dt)  # noqa: E731
    peer_col = 1 - j
    col.stage("all_gather", [d(bias_shard(gamma, q, 0, j)), None])
    col.stage("all_gather", [d(bias_shard(beta, q, 0, j)), None])
    row.stage("all_reduce", [d(oracle.ln2d_partial_stats(shard(A, q, i, peer_col)))])
    x = _leaf(d(shard(A, q, i, j)))
    y = norm(x)
    Ar = _leaf(A)
    ref = F.layer_norm(Ar, (H,), gamma, beta, eps)
    ref.backward(dY)
    assert_parity(y, shard(ref.detach(), q, i, j), dt, "LayerNorm2D forward shard")
    # backward: the row peer's partial sums, then the column peers' dgamma/dbeta sums
    stats = oracle.ln2d_partial_stats(A)
    mr = oracle.ln2d_mean_rstd(stats, H, eps)
    g_peer = torch.chunk(gamma, q, dim=-1)[peer_col]
    rs_peer, _, _ = oracle.ln2d_backward_partials(shard(dY, q, i, peer_col), shard(A, q, i, peer_col), mr[i * R // q:(i + 1) * R // q], g_peer)
    row.stage("all_reduce", [d(rs_peer)])
    other_row = 1 - i
    _, dg_o, db_o = oracle.ln2d_backward_partials(shard(dY, q, other_row, j), shard(A, q, other_row, j),
                                                  mr[other_row * R // q:(other_row + 1) * R // q], torch.chunk(gamma, q, dim=-1)[j])
    col.stage("reduce_scatter", [d(dg_o)])
    col.stage("reduce_scatter", [d(db_o)])
    y.backward(d(shard(dY, q, i, j)))
    assert_parity(x.grad, shard(Ar.grad, q, i, j), dt, "dX shard")
    xh = (A - mr[:, 0:1]) * mr[:, 1:2]
    assert_parity(norm.weight.grad, bias_shard((dY * xh).sum(0), q, i, j), dt, "dgamma shard")
    assert_parity(norm.bias.grad, bias_shard(dY.sum(0), q, i, j), dt, "dbeta shard")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_vocab_parallel_loss_one_rank_of_four(dtype):
    """Rank 1 of 4 vocabulary slices (tests/test_1d/check_1d_modules.py:491-524
    with [tokens, vocab] logits)."""
    import oracle
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.loss import VocabParallelCrossEntropyLoss1D

    p, r, T, V = 4, 1, 96, 1000
    full = randn((T, V * p), dtype, 0, std=2.0)
    t = torch.randint(0, V * p, (T,), generator=torch.Generator().manual_seed(1))
    slices = list(torch.chunk(full, p, dim=-1))
    initialize("1d", p, rank=r)
    with oracle.precision(torch.float64):
        peers = [oracle.vpce_fwd_local(s, t, k * V) for k, s in enumerate(slices) if k != r]
    stk = lambda n: torch.stack([pk[n] for pk in peers])  # noqa: E731
    pm.PARALLEL_1D.stage("vpce_stats", [stk(n).to(DEV, torch.float32) for n in range(3)] + [stk(3).to(DEV)])
    crit = VocabParallelCrossEntropyLoss1D()
    x = _leaf(slices[r].contiguous().to(DEV))
    before = x.detach().clone()
    loss = crit(x, t.to(DEV))
    loss.backward()
    fr = _leaf(full.double())
    ref = F.cross_entropy(fr, t)
    ref.backward()
    assert_parity(loss, ref.detach(), torch.float32, "mean loss")
    assert_parity(x.grad, fr.grad[:, r * V:(r + 1) * V], dtype, "logits grad")
    assert torch.equal(x.detach(), before), "the caller's logits must stay intact"


def test_vocab_parallel_loss2d_one_rank_of_2x2_grid():
    """VocabParallelCrossEntropyLoss2D as rank (row 1, col 0) of a 2 x 2 grid
    (tests/test_2d/check_2d_modules.py:635-661): the classes are split over the grid columns, the tokens over
    the grid rows; the row peer's per-token statistics and the column peer's mean loss are pre-staged."""
    import oracle
    from oracle.grid import shard
    from cubework_amd.distributed import initialize, pm
    from cubework_amd.module.loss import VocabParallelCrossEntropyLoss2D

    q, i, j = 2, 1, 0
    oi, oj = 1 - i, 1 - j
    T, V = 64, 600
    dt = torch.float32
    full = randn64((T, V), 0, std=2.0)
    t = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(1))
    t_rows = torch.chunk(t, q)[i]
    initialize("2d", q * q, row=i, col=j)
    with oracle.precision(torch.float64):
        peer = oracle.vpce_fwd_local(shard(full, q, i, oj), t_rows, oj * (V // q))
    pm.PARALLEL_2D_ROW.stage("vpce_stats", [pk.unsqueeze(0).to(DEV, dt) for pk in peer[:3]] + [peer[3].unsqueeze(0).to(DEV)])
    pm.PARALLEL_2D_COL.stage("all_reduce", [F.cross_entropy(torch.chunk(full, q)[oi], torch.chunk(t, q)[oi]).to(DEV, dt)])
    crit = VocabParallelCrossEntropyLoss2D()
    x = _leaf(shard(full, q, i, j).contiguous().to(DEV, dt))
    loss = crit(x, t.to(DEV))
    loss.backward()
    fr = _leaf(full)
    ref = F.cross_entropy(fr, t)
    ref.backward()
    assert_parity(loss, ref.detach(), dt, "mean loss")
    assert_parity(x.grad, shard(fr.grad, q, i, j), dt, "logits grad shard")
    assert not any(pm.PARALLEL_2D_ROW.inbox.values()) and not any(pm.PARALLEL_2D_COL.inbox.values())


@pytest.mark.parametrize("amp_dtype", [torch.float16, torch.bfloat16])
def test_opt_block_under_autocast(amp_dtype):
    """fp32 parameters and input inside torch.autocast, as the reference's training scripts run
    (benchmark/opt/train.py:85-86): the four Linear2D cast to the autocast dtype (float16 by default, the
    reference's custom_fwd dtype), LayerNorm2D runs in fp32, the fused attention core takes the projections'
    dtype; output and every gradient against the same block in fp32 torch."""
    from cubework_amd.distributed import initialize
    from cubework_amd.opt_block import OPTBlock
    from oracle import opt_block_reference

    initialize("2d", 1)
    torch.manual_seed(0)
    blk = OPTBlock(hidden=256, heads=4, ffn=1024, dtype=torch.float32, activation="gelu_tanh").to(DEV)
    x = _leaf(randn((2, 64, 256), torch.float32, 1).to(DEV))
    dy = randn((2, 64, 256), torch.float32, 2).to(DEV)
    with torch.autocast("cuda", dtype=amp_dtype):
        y = blk(x)
    y.backward(dy)
    xr = _leaf(x.detach().cpu())
    ref, params = opt_block_reference(blk, xr)
    ref.backward(dy.cpu())
    assert_parity(y, ref.detach(), amp_dtype, "block forward under autocast")
    assert_parity(x.grad, xr.grad, amp_dtype, "block dX under autocast")
    for name, prm in blk.named_parameters():
        assert prm.grad is not None and prm.grad.dtype == torch.float32, name
        assert_parity(prm.grad, params[name].grad, amp_dtype, name + ".grad under autocast")


@pytest.mark.parametrize("activation", ["gelu_tanh", "relu"])
def test_opt_block_shapes_small(activation):
    """A reduced OPT decoder layer (benchmark/opt/opt.py:135-211 shapes: pre-LN,
    qkv/out/fc1/fc2 Linear2D) at tensor-parallel size 1, forward+backward in
    bf16 against the same block in float64 torch: output, input gradient and every
    parameter gradient. ReLU (OPT's activation, opt.py:144,200) is not differentiable at 0: a
    pre-activation that bf16 rounding puts on the other side of 0 than the float64 value switches a whole
    term of fc1's weight gradient on or off, which is not a rounding-sized difference. The reference
    computation is therefore handed the mask the GPU used (which units of fc1's output are positive), so that
    both sides differentiate the same piecewise-linear function; the mask itself is checked against the
    float64 pre-activation wherever that is not within bf16 rounding of 0."""
    from cubework_amd.distributed import initialize
    from cubework_amd.opt_block import OPTBlock
    import oracle

    initialize("2d", 1)
    torch.manual_seed(0)
    blk = OPTBlock(hidden=256, heads=4, ffn=1024, dtype=torch.bfloat16, activation=activation).to(DEV)
    x = _leaf(randn((2, 64, 256), torch.bfloat16, 1).to(DEV))
    dy = randn((2, 64, 256), torch.bfloat16, 2).to(DEV)
    seen = {}
    hook = blk.fc1.register_forward_hook(lambda mod, args, out: seen.__setitem__("fc1", out.detach()))
    y = blk(x)
    hook.remove()
    y.backward(dy)
    mask = None
    if activation == "relu":
        mask = (seen["fc1"] > 0).cpu()
    with oracle.precision(torch.float64):
        xr = _leaf(x.detach().double().cpu())
        ref, params = oracle.opt_block_reference(blk, xr, relu_mask=mask)
        ref.backward(dy.double().cpu())
        if mask is not None:
            # the GPU's mask is the sign of the float64 pre-activation except within rounding distance of 0
            free, _ = oracle.opt_block_reference(blk, x.detach().double().cpu())
            assert_parity(free.detach(), ref.detach(), torch.float32, "ReLU mask leaves the forward unchanged", bar=2e-3)
    # a chain of ten 16-bit operators (two LayerNorms, four linears, attention, activation, two residual adds), each rounding once
    assert_parity(y, ref.detach(), torch.bfloat16, "block forward")
    assert_parity(x.grad, xr.grad, torch.bfloat16, "block dX")
    for name, prm in blk.named_parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad.float()).all(), name
        assert_parity(prm.grad, params[name].grad, torch.bfloat16, name + ".grad")


def test_opt_block_half_model():
    """The same layer as a float16 model (parameters and activations in float16, no autocast: nothing
    casts, every operator of the layer receives float16), against the block in fp32 torch."""
    from cubework_amd.distributed import initialize
    from cubework_amd.opt_block import OPTBlock
    from oracle import opt_block_reference

    initialize("2d", 1)
    torch.manual_seed(0)
    blk = OPTBlock(hidden=256, heads=4, ffn=1024, dtype=torch.float16, activation="gelu_tanh").to(DEV)
    x = _leaf(randn((2, 64, 256), torch.float16, 1).to(DEV))
    dy = randn((2, 64, 256), torch.float16, 2).to(DEV)
    y = blk(x)
    assert y.dtype == torch.float16
    y.backward(dy)
    xr = _leaf(x.detach().float().cpu())
    ref, params = opt_block_reference(blk, xr)
    ref.backward(dy.float().cpu())
    assert_parity(y, ref.detach(), torch.float16, "block forward")
    assert_parity(x.grad, xr.grad, torch.float16, "block dX")
    for name, prm in blk.named_parameters():
        assert prm.grad is not None and prm.grad.dtype == torch.float16, name
        assert_parity(prm.grad, params[name].grad, torch.float16, name + ".grad")
