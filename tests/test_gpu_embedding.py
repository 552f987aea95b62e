"""GPU parity of the vocab-parallel embedding (cw_embed_fwd, cw_embed_bwd_ids and cw_embed_sort_ids +
cw_embed_bwd through the C ABI): the lookup is a bit-exact copy with integer-exact masking; the gradient
is an fp32 sum rounded once. Every backward case runs both ways: in one launch from the unsorted ids
(where the shapes qualify) and through the token order."""
import pytest
import torch

from tests.util import assert_parity, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
both_paths = pytest.mark.parametrize("via_order", [False, True], ids=["from_ids", "token_order"])


def _ids(shape, vocab, seed, hot=None):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab, shape, generator=g)
    if hot is not None:  # a frequent token: long runs in the sorted order
        ids.view(-1)[::3] = hot
    return ids


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("case", [(4, 37, 1000, 256, 250, 64), (2, 128, 50272, 12568, 12568, 2048),
                                  (1, 5, 64, 64, 0, 8), (3, 11, 300, 100, 100, 52), (1, 1, 16, 4, 12, 520)])
@both_paths
def test_embedding_forward_backward_parity(case, dtype, via_order):
    import oracle
    from cubework_amd import ops

    b, s, vocab, v_loc, start, e = case
    ids = _ids((b, s), vocab, seed=b * s, hot=start + 1 if v_loc > 1 else None)
    edges = torch.tensor([start - 1, start, start + v_loc - 1, start + v_loc, 0, vocab - 1]).clamp(0, vocab - 1)
    n = min(6, ids.numel())
    ids.view(-1)[:n] = edges[:n]
    w = randn((v_loc, e), dtype, 5)
    want = oracle.vocab_embedding_fwd(ids, w, start)
    got = ops.embedding_fwd(ids.to(DEV), w.to(DEV), start)
    torch.cuda.synchronize()
    assert got.shape == (b, s, e)
    assert torch.equal(got.cpu(), want), "the lookup must be a bit-exact copy / exact zeros"

    d_out = randn((b, s, e), dtype, 6)
    for pad in (None, 1 if v_loc > 1 else 0):
        want_dw = oracle.vocab_embedding_bwd(ids, d_out, v_loc, start, pad)
        got_dw = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), v_loc, start, -1 if pad is None else pad, via_order)
        again = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), v_loc, start, -1 if pad is None else pad, via_order)
        torch.cuda.synchronize()
        assert torch.equal(got_dw, again), "no atomics: bit-reproducible"
        assert_parity(got_dw, want_dw, dtype, "embedding d_weight %s pad=%s" % (case, pad))
        untouched = torch.ones(v_loc, dtype=torch.bool)
        local = ids.view(-1) - start
        live = (local >= 0) & (local < v_loc)
        untouched[local[live]] = False
        assert (got_dw.cpu()[untouched] == 0).all(), "rows without tokens are exactly zero"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("e", [520, 2048, 4104])
@both_paths
def test_embedding_backward_every_run_length(e, dtype, via_order):
    """Id j occurs j + 1 times (runs of 1 .. 45 tokens in the sorted order, shuffled over the batch): the
    short-run path, the shared path with its four column-sharing blocks and ragged last slices, and runs
    that end inside and at the edge of a wavefront's group of tokens all meet the oracle's sums."""
    import oracle
    from cubework_amd import ops

    ids = torch.cat([torch.full((j + 1,), 3 + 2 * j, dtype=torch.int64) for j in range(45)])
    ids = ids[torch.randperm(ids.numel(), generator=torch.Generator().manual_seed(e))]
    v_loc, start = 100, 0
    d_out = randn((ids.numel(), e), dtype, 7)
    want = oracle.vocab_embedding_bwd(ids, d_out, v_loc, start, None)
    got = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), v_loc, start, -1, via_order)
    torch.cuda.synchronize()
    assert_parity(got, want, dtype, "embedding d_weight, runs of 1..45, E=%d" % e)
    assert (got.cpu()[0:3] == 0).all() and (got.cpu()[4::2][:44] == 0).all(), "rows without tokens are exactly zero"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@both_paths
def test_embedding_backward_one_id_thousands_of_times(dtype, via_order):
    """Token frequencies of text: one id 3000 times among 5000 tokens (a run that every wavefront of the
    sharing blocks walks for many rounds), the rest spread over the table; compared in float64."""
    from cubework_amd import ops

    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 400, (5000,), generator=g)
    ids[torch.randperm(5000, generator=g)[:3000]] = 17
    e, v_loc = 1032, 400
    d_out = randn((5000, e), dtype, 8)
    want = torch.zeros((v_loc, e), dtype=torch.float64).index_add_(0, ids, d_out.double())
    got = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), v_loc, 0, -1, via_order)
    again = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), v_loc, 0, -1, via_order)
    torch.cuda.synchronize()
    assert torch.equal(got, again)
    # the longest run sums 3000 rows in fp32
    assert_parity(got, want, dtype, "embedding d_weight with a run of 3000")


def test_vocab_slices_sum_to_the_full_lookup():
    """Four vocabulary slices: every token is live in exactly one, so the slices' outputs sum (the
    all-reduce of parallel_1d/module.py:454) to F.embedding on the whole table, bit for bit."""
    from cubework_amd import ops

    vocab, e, p = 1024, 128, 4
    ids = _ids((2, 77), vocab, 3).to(DEV)
    table = randn((vocab, e), torch.bfloat16, 4).to(DEV)
    total = torch.zeros((2, 77, e), dtype=torch.float32, device=DEV)
    for r in range(p):
        total += ops.embedding_fwd(ids, table[r * vocab // p:(r + 1) * vocab // p], r * vocab // p).float()
    assert torch.equal(total.to(torch.bfloat16), torch.nn.functional.embedding(ids, table))


@pytest.mark.parametrize("mode", [None, "1d", "2d", "3d"])
@pytest.mark.parametrize("vocab_parallel", [False, True])
def test_facade_embedding_size1(mode, vocab_parallel):
    import cubework_amd.module as cube_nn
    from cubework_amd.distributed import initialize

    initialize(mode, 1)
    torch.manual_seed(0)
    emb = cube_nn.Embedding(200, 64, vocab_parallel=vocab_parallel and mode is not None, padding_idx=3,
                            dtype=torch.bfloat16).to(DEV)
    assert emb.weight.shape == (200, 64) and (emb.weight[3] == 0).all()
    ids = _ids((8, 16), 200, 9).to(DEV)   # 8 rows: divisible by every batch split at size 1
    ids[0, :4] = 3
    out = emb(ids)
    ref_w = emb.weight.detach().clone().requires_grad_(True)
    ref = torch.nn.functional.embedding(ids, ref_w, padding_idx=3)
    assert torch.equal(out, ref)
    d = randn((8, 16, 64), torch.bfloat16, 10).to(DEV)
    out.backward(d)
    ref.backward(d)
    assert_parity(emb.weight.grad, ref_w.grad.float().cpu(), torch.bfloat16, "embedding weight grad (%s)" % mode)
    assert (emb.weight.grad[3] == 0).all()


def test_vocab_parallel_embedding_one_rank_of_four():
    """Rank 1 of a 1D group of 4: the layer's own slice through the kernel, the peers' contribution staged
    where the all-reduce would deliver it."""
    import cubework_amd.module as cube_nn
    from cubework_amd.distributed import ParallelManager as pm
    from cubework_amd.distributed import initialize

    initialize("1d", 4, rank=1)
    torch.manual_seed(0)
    emb = cube_nn.VocabParallelEmbedding1D(400, 32).to(torch.bfloat16).to(DEV)
    assert emb.weight.shape == (100, 32) and emb.vocab_start_index == 100
    ids = _ids((4, 9), 400, 2).to(DEV)
    peers = randn((4, 9, 32), torch.bfloat16, 7).to(DEV)
    pm.PARALLEL_1D.stage("all_reduce", [peers])
    out = emb(ids)
    local = torch.nn.functional.embedding((ids - 100).clamp(0, 99), emb.weight.detach())
    local[(ids < 100) | (ids >= 200)] = 0
    assert torch.equal(out, local + peers)


@pytest.mark.parametrize("T", [1, 2, 3, 100, 1023, 8192, 16384, 16385, 50000, 140000])
def test_token_order_is_the_stable_sort(T):
    """cw_embed_sort_ids against Python's sorted() on (row, position) pairs: bit-exact, including ids
    below, inside and above the slice, negative ids and the extremes of int64. Sizes cover one workgroup
    in LDS (<= 16384) and the multi-launch network with 4 and 16 chunks."""
    from cubework_amd import ops

    start, rows = 1000, 777
    g = torch.Generator().manual_seed(T)
    ids = torch.randint(start - 300, start + rows + 300, (T,), generator=g, dtype=torch.int64)
    edges = torch.tensor([start - 1, start, start + rows - 1, start + rows, 0, -5, 2 ** 63 - 1, -2 ** 63], dtype=torch.int64)
    n = min(T, edges.numel())
    ids[:n] = edges[:n]
    keyed = sorted((((v - start) if start <= v < start + rows else rows), i) for i, v in enumerate(ids.tolist()))
    want_ids = torch.tensor([start + r for r, _ in keyed], dtype=torch.int64)
    want_order = torch.tensor([i for _, i in keyed], dtype=torch.int64)
    got_ids, got_order = ops.embedding_token_order(ids.to(DEV), rows, start)
    torch.cuda.synchronize()
    assert torch.equal(got_ids.cpu(), want_ids)
    assert torch.equal(got_order.cpu(), want_order)


def test_token_order_repeated_id():
    """Every token selects the same row: the order is the identity."""
    from cubework_amd import ops

    ids = torch.full((5000,), 42, dtype=torch.int64, device=DEV)
    got_ids, got_order = ops.embedding_token_order(ids, 100, 0)
    assert torch.equal(got_ids, ids)
    assert torch.equal(got_order.cpu(), torch.arange(5000))


@pytest.mark.parametrize("T", [0, 1, 16384])
def test_embedding_backward_from_ids_edges(T):
    """The one-launch backward on ids below, at and above the slice's edges, negative ids and the extremes
    of int64 (none of which may select a row), on an empty batch (all zeros) and on the longest batch it
    takes; float64 sums within the bar everywhere (bit equality with the token-order path is the subject of
    test_embedding_backward_from_ids_order_of_addition)."""
    from cubework_amd import ops

    start, rows, e = 1000, 777, 264
    g = torch.Generator().manual_seed(T + 1)
    ids = torch.randint(start - 300, start + rows + 300, (T,), generator=g, dtype=torch.int64)
    edges = torch.tensor([start - 1, start, start + rows - 1, start + rows, 0, -5, 2 ** 63 - 1, -2 ** 63], dtype=torch.int64)
    n = min(T, edges.numel())
    ids[:n] = edges[:n]
    d_out = randn((T, e), torch.float32, 12)
    got = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, start, 5, via_token_order=False)
    torch.cuda.synchronize()
    local = ids - start
    live = (ids >= start) & (ids < start + rows) & (local != 5)
    want = torch.zeros((rows, e), dtype=torch.float64).index_add_(0, local[live], d_out.double()[live])
    assert_parity(got, want, torch.float32, "embedding d_weight from ids, T=%d" % T)
    assert (got[5] == 0).all()
    if T <= 1:
        via = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, start, 5, via_token_order=True)
        assert torch.equal(got, via)


def test_embedding_backward_from_ids_order_of_addition():
    """The one-launch backward walks a row's token positions in blocks of 32, round by round the lowest remaining
    token of every block. Rows whose tokens (2 to 8 of them) all sit in different blocks are therefore added in
    ascending token position and equal the token-order path bit for bit; a row with two tokens in one block and
    later ones ({0, 1, 40}, {64, 70, 75, 130, 131}) may be added in another fixed order: the same bits on every
    call, equal to the token-order path only up to fp32 reassociation - bit equality with it is waived there,
    by design."""
    from cubework_amd import ops

    rows, e, T = 64, 264, 512
    d_out = randn((T, e), torch.float32, 21)
    # (a) tokens of each row in distinct 32-blocks: row r gets tokens r%32 + 32*k for k < 2 + r % 7
    ids = torch.full((T,), rows + 5, dtype=torch.int64)   # outside the slice
    for r in range(20):
        for k in range(2 + r % 7):
            ids[(r % 32) + 32 * k + (0 if r < 32 else 1)] = r
    a = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, 0, -1, via_token_order=False)
    b = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, 0, -1, via_token_order=True)
    assert torch.equal(a, b)
    # (b) {0, 1, 40} and friends: two tokens in one block plus later ones
    ids = torch.full((T,), rows + 5, dtype=torch.int64)
    ids[[0, 1, 40]] = 3
    ids[[64, 70, 75, 130, 131]] = 9
    a1 = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, 0, -1, via_token_order=False)
    a2 = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, 0, -1, via_token_order=False)
    b = ops.embedding_bwd(ids.to(DEV), d_out.to(DEV), rows, 0, -1, via_token_order=True)
    assert torch.equal(a1, a2)                                            # a fixed order
    untouched = torch.ones(rows, dtype=torch.bool)
    untouched[[3, 9]] = False
    assert torch.equal(a1[untouched], b[untouched])                       # every other row: the same bits
    assert_parity(a1, b, torch.float32, "one launch against the token order, tokens sharing a block")
    want = torch.zeros((rows, e), dtype=torch.float64).index_add_(0, ids[ids < rows], d_out.double()[ids < rows])
    assert_parity(a1, want, torch.float32, "embedding d_weight from ids, tokens sharing a block")
    # int32 ids, which F.embedding also takes, give the same result
    assert torch.equal(ops.embedding_bwd(ids.int().to(DEV), d_out.to(DEV), rows, 0, -1, via_token_order=False), a1)
    w = randn((rows, e), torch.float32, 22).to(DEV)
    assert torch.equal(ops.embedding_fwd(ids.int().to(DEV), w, 0), ops.embedding_fwd(ids.to(DEV), w, 0))


def test_embedding_backward_from_ids_refuses_what_it_cannot_take():
    """More than 16384 tokens, or rows that are not 16-byte aligned: CW_ERR_UNSUPPORTED from the entry point
    (nothing launched), and the wrapper goes through the token order instead."""
    from cubework_amd import _lib, ops

    lib = _lib.load()
    T, e, rows = 16385, 64, 50
    ids = torch.randint(0, rows, (T,), generator=torch.Generator().manual_seed(1)).to(DEV)
    d_out = randn((T, e), torch.bfloat16, 2).to(DEV)
    dw = torch.full((rows, e), 7.0, dtype=torch.bfloat16, device=DEV)
    assert lib.cw_embed_bwd_ids_supported(T, e, d_out.data_ptr(), e, dw.data_ptr(), e, _lib.CW_BF16) == 0
    rc = lib.cw_embed_bwd_ids(T, e, ids.data_ptr(), 0, rows, -1, d_out.data_ptr(), e, dw.data_ptr(), e, _lib.CW_BF16, None)
    assert rc == -3  # CW_ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert (dw == 7.0).all(), "a refused call writes nothing"
    got = ops.embedding_bwd(ids, d_out, rows)  # the wrapper's other path
    want = torch.zeros((rows, e), dtype=torch.float64).index_add_(0, ids.cpu(), d_out.double().cpu())
    assert_parity(got, want, torch.bfloat16, "embedding d_weight, 16385 tokens")
    odd = d_out[:100, 1:]  # rows start 2 bytes off a 16-byte boundary
    assert lib.cw_embed_bwd_ids_supported(100, e - 1, odd.data_ptr(), e, dw.data_ptr(), e, _lib.CW_BF16) == 0


def test_embedding_backward_from_ids_is_offered_only_where_it_pays():
    """Every workgroup of the one-launch kernel scans all ids, so for rows much smaller than the batch's ids
    cw_embed_bwd_ids_supported says no (the wrapper then takes the token order); the entry point itself still
    serves such a call, with the same sums."""
    from cubework_amd import _lib, ops

    lib = _lib.load()
    BF16 = _lib.CW_BF16
    dummy = torch.empty(16, dtype=torch.bfloat16, device=DEV)
    p = dummy.data_ptr()
    assert lib.cw_embed_bwd_ids_supported(8192, 2048, p, 2048, p, 2048, BF16) == 1    # the benchmark's shape
    assert lib.cw_embed_bwd_ids_supported(16384, 2048, p, 2048, p, 2048, BF16) == 1
    assert lib.cw_embed_bwd_ids_supported(16384, 1024, p, 1024, p, 1024, BF16) == 0   # 4 row sizes = 8192 < 16384
    assert lib.cw_embed_bwd_ids_supported(8192, 512, p, 512, p, 512, BF16) == 1       # 8 row sizes up to 8192 tokens
    assert lib.cw_embed_bwd_ids_supported(8192, 256, p, 256, p, 256, BF16) == 0
    assert lib.cw_embed_bwd_ids_supported(8192, 256, p, 256, p, 256, _lib.CW_F32) == 1
    T, e, rows = 4096, 64, 3000
    ids = torch.randint(0, rows, (T,), generator=torch.Generator().manual_seed(3)).to(DEV)
    d_out = randn((T, e), torch.bfloat16, 4).to(DEV)
    assert lib.cw_embed_bwd_ids_supported(T, e, d_out.data_ptr(), e, p, e, BF16) == 0
    auto = ops.embedding_bwd(ids, d_out, rows)
    forced = ops.embedding_bwd(ids, d_out, rows, via_token_order=False)
    order = ops.embedding_bwd(ids, d_out, rows, via_token_order=True)
    torch.cuda.synchronize()
    assert torch.equal(auto, order)
    want = torch.zeros((rows, e), dtype=torch.float64).index_add_(0, ids.cpu(), d_out.double().cpu())
    assert_parity(forced, want, torch.bfloat16, "one launch where it does not pay")
    assert_parity(auto, want, torch.bfloat16, "token order chosen by the wrapper")
