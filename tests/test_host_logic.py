"""Host-side behaviour of the layer API that needs no GPU: shard shapes and
parameter names of every class at the reference's grid sizes, the env side
channels that depend on construction order, error types, the single-process
collectives, initializer bounds, and the refusal to compute on the CPU."""
import math

import pytest
import torch

from cubework_amd import distributed as D
from cubework_amd.distributed import initialize, pm
from cubework_amd.global_vars import NUM_PARTITIONS, env
import cubework_amd.module as cube_nn
from cubework_amd.module import init
from cubework_amd.module.loss import (VocabParallelCrossEntropyLoss1D, VocabParallelCrossEntropyLoss2D,
                                      VocabParallelCrossEntropyLoss3D)
from cubework_amd.module.parallel_1d import (Classifier1D, Linear1D, Linear1D_Col, Linear1D_Row,
                                             VocabParallelClassifier1D)
from cubework_amd.module.parallel_2d import Classifier2D, LayerNorm2D, Linear2D, VocabParallelClassifier2D
from cubework_amd.module.parallel_3d import Classifier3D, LayerNorm3D, Linear3D, VocabParallelClassifier3D


def test_shard_shapes_2d():
    initialize("2d", 4, row=1, col=0)
    assert env.summa_dim == 2 and pm.PARALLEL_2D_ROW.local_rank == 0 and pm.PARALLEL_2D_COL.local_rank == 1
    lin = Linear2D(64, 128)
    assert lin.weight.shape == (32, 64) and lin.bias.shape == (32,)
    assert (lin.row_rank, lin.col_rank) == (1, 0)
    assert getattr(lin.weight, NUM_PARTITIONS) == 4 and getattr(lin.bias, NUM_PARTITIONS) == 4
    ln = LayerNorm2D(64)
    assert ln.weight.shape == (16,) and ln.variance_epsilon == 1e-5
    assert torch.all(ln.weight == 1) and torch.all(ln.bias == 0)
    c = Classifier2D(64, 10)
    assert c.weight.shape == (10, 16) and c.bias.shape == (10,)
    assert not env.vocab_parallel
    v = VocabParallelClassifier2D(64, 40)
    assert v.weight.shape == (20, 32) and v.bias.shape == (10,) and env.vocab_parallel
    shared = torch.nn.Parameter(torch.zeros(20, 32))
    tied = VocabParallelClassifier2D(64, 40, weight=shared)
    assert tied.weight is shared and not tied.has_weight
    assert set(dict(lin.named_parameters())) == {"weight", "bias"}
    assert isinstance(cube_nn.CrossEntropyLoss().loss, VocabParallelCrossEntropyLoss2D)


def test_shard_shapes_1d_and_construction_order():
    initialize("1d", 4, rank=2)
    first, second = cube_nn.Linear(64, 256), cube_nn.Linear(256, 64)
    assert isinstance(first.linear, Linear1D) and isinstance(first.linear.linear, Linear1D_Col)
    assert isinstance(second.linear.linear, Linear1D_Row)  # column-parallel, then row-parallel (Megatron MLP)
    assert first.weight.shape == (64, 64) and first.bias.shape == (64,)
    assert second.weight.shape == (64, 64) and second.bias.shape == (64,)
    assert not env.parallel_input_1d
    c = Classifier1D(64, 10)
    assert c.weight.shape == (10, 16) and c.bias.shape == (10,) and not env.vocab_parallel
    v = VocabParallelClassifier1D(64, 40)
    assert v.weight.shape == (10, 64) and v.bias.shape == (10,) and env.vocab_parallel
    assert isinstance(cube_nn.CrossEntropyLoss().loss, VocabParallelCrossEntropyLoss1D)
    assert isinstance(cube_nn.LayerNorm(64).norm.norm, torch.nn.LayerNorm)
    with pytest.raises(ValueError):
        Linear1D_Col(8, 8, bias=False, skip_bias_add=True)
    with pytest.raises(ValueError):
        Linear1D_Row(8, 8, bias=False, skip_bias_add=True)


def test_shard_shapes_3d_and_group_swap():
    initialize("3d", 8, coords=(1, 0, 1))
    assert env.depth_3d == 2
    before = (env.input_group_3d, env.output_group_3d)
    lin = Linear3D(64, 128)
    assert lin.weight.shape == (32, 32) and lin.bias.shape == (64,)
    assert (env.input_group_3d, env.output_group_3d) == (before[1], before[0])  # swapped by the constructor
    assert getattr(lin.weight, NUM_PARTITIONS) == 8 and getattr(lin.bias, NUM_PARTITIONS) == 2
    ln = LayerNorm3D(64)
    assert ln.weight.shape == (32,) and ln.variance_epsilon == 1e-12
    c = Classifier3D(64, 10)
    assert c.weight.shape == (10, 32) and c.bias.shape == (10,)
    v = VocabParallelClassifier3D(64, 40)
    assert v.weight.shape == (10, 32) and v.bias.shape == (20,) and env.vocab_parallel
    assert isinstance(cube_nn.CrossEntropyLoss().loss, VocabParallelCrossEntropyLoss3D)


def test_mode_none_uses_torch_layers_and_2d_needs_groups():
    initialize(None, 1)
    assert isinstance(cube_nn.Linear(8, 8).linear, torch.nn.Linear)
    assert isinstance(cube_nn.LayerNorm(8).norm, torch.nn.LayerNorm)
    assert isinstance(cube_nn.CrossEntropyLoss().loss, torch.nn.CrossEntropyLoss)
    with pytest.raises(AssertionError):
        Linear2D(8, 8)
    with pytest.raises(ValueError):
        initialize("4d", 16)
    with pytest.raises(AssertionError):
        initialize("2d", 8)  # not a square


def test_dtype_argument_and_cpu_refusal():
    initialize("2d", 1)
    lin = cube_nn.Linear(16, 16, dtype=torch.bfloat16)
    assert lin.weight.dtype == torch.bfloat16 and lin.bias.dtype == torch.bfloat16
    with pytest.raises(RuntimeError, match="GPU only"):
        lin(torch.zeros(4, 16, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="GPU only"):
        cube_nn.LayerNorm(16)(torch.zeros(4, 16))
    env.vocab_parallel = True
    with pytest.raises(RuntimeError, match="GPU only"):
        cube_nn.CrossEntropyLoss()(torch.zeros(4, 16), torch.zeros(4, dtype=torch.long))
    with pytest.raises(ValueError):
        Linear2D(8, 8, skip_bias_add=True, activation="relu")


def test_single_process_collectives():
    mode = D.ParallelMode("TEST")
    mode.init(1, 0)
    t = torch.arange(6.0).reshape(2, 3)
    for fn in (lambda: D.all_gather(t, -1, mode), lambda: D.reduce_scatter(t, -1, mode), lambda: D.all_reduce(t, mode),
               lambda: D.broadcast(t, 0, mode), lambda: D.reduce(t, 0, mode)):
        assert fn() is t  # identities at world size 1, as cubework/distributed/collective.py:8,30,50,67,84
    mode.init(2, 1)
    with pytest.raises(D.MissingPeerData):
        D.all_reduce(t, mode)
    mode.stage("all_reduce", [t * 2])
    assert torch.equal(D.all_reduce(t, mode), t * 3)
    mode.stage("all_reduce", [t * 2])
    assert torch.equal(D.all_reduce(t, mode, op="max"), t * 2)
    mode.stage("all_gather", [t + 10, None])
    assert torch.equal(D.all_gather(t, -1, mode), torch.cat([t + 10, t], -1))
    mode.stage("reduce_scatter", [torch.ones(2, 4)])
    assert torch.equal(D.reduce_scatter(torch.ones(2, 4), -1, mode), torch.full((2, 2), 2.0))
    assert D.broadcast(t, 1, mode) is t
    mode.stage("broadcast", t + 1)
    assert torch.equal(D.broadcast(t, 0, mode), t + 1)
    D.reduce(t, 0, mode)
    assert mode.outbox["reduce"][0][0] == 0
    mode.stage("reduce", [t])
    assert torch.equal(D.reduce(t, 1, mode), 2 * t)


def test_initializer_bounds_use_global_fans():
    """cubework/module/init.py: kaiming_uniform_(a=sqrt(5)) -> U(+-1/sqrt(fan_in));
    xavier_uniform_(a=1, scale=1) -> U(+-sqrt(1/fan_in)); default xavier_uniform_ -> Glorot."""
    w = torch.empty(512, 512)
    init.kaiming_uniform_(a=math.sqrt(5))(w, fan_in=4096, fan_out=64)
    assert w.abs().max() <= 1 / math.sqrt(4096) and w.abs().max() > 0.9 / math.sqrt(4096)
    init.xavier_uniform_(a=1, scale=1)(w, fan_in=1024)
    assert w.abs().max() <= math.sqrt(1 / 1024) and w.abs().max() > 0.9 * math.sqrt(1 / 1024)
    init.xavier_uniform_()(w, fan_in=1024, fan_out=4096)
    bound = math.sqrt(6.0 / 5120)
    assert w.abs().max() <= bound and w.abs().max() > 0.9 * bound
    init.lecun_uniform_()(w, fan_in=300)
    assert w.abs().max() <= math.sqrt(3 / 300)
    init.kaiming_normal_()(w, fan_in=100)
    assert abs(w.std().item() - math.sqrt(2.0) / 10) < 0.01
    with pytest.raises(AssertionError):
        init.xavier_uniform_()(w)
    with pytest.raises(ValueError):
        init.kaiming_uniform_(mode="bad")(w, fan_in=4)
    initialize("2d", 4)
    lin = Linear2D(4096, 64)
    assert lin.weight.abs().max() <= 1 / math.sqrt(4096)  # bound from the global fan_in, not the shard's


def test_partition_batch():
    initialize("2d", 4, row=1, col=0)
    x = torch.arange(8).reshape(4, 2)
    assert torch.equal(cube_nn.partition_batch(x), x[2:])
    out = cube_nn.partition_batch({"a": x, "b": [x][0]})
    assert torch.equal(out["a"], x[2:])
    initialize("1d", 4)
    assert cube_nn.partition_batch(x) is x


def test_bench_refuses_more_than_one_gpu_and_has_no_cpu_path():
    """bench.py measures one rank's share on one GPU: `--gpus 2` (or a WORLD_SIZE above 1) ends with a message and
    status 2 before anything touches a device, and on a host without a GPU the default invocation ends with
    status 3 instead of timing a CPU stand-in."""
    import os
    import subprocess
    import sys

    bench = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
    r = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
    env_two = dict(os.environ, WORLD_SIZE="2")
    r = subprocess.run([sys.executable, bench], capture_output=True, text=True, timeout=120, env=env_two)
    assert r.returncode == 2
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0"], capture_output=True, text=True,
                           timeout=300)
        assert r.returncode == 3 and "no CPU fallback" in r.stderr and r.stdout.strip() == ""


def test_attention_head_padding_is_exact_on_the_host():
    """Head sizes between the kernels' 64 and 128 are zero-padded (cubework_amd.ops._pad_last): the padded q.k
    products equal the unpadded ones, slicing the padded columns away gives the input back, and sizes above
    128 are refused (benchmark/opt/opt.py:419-495 lists 48, 64, 80 and 128)."""
    from cubework_amd import ops

    assert [ops._attn_padded_head(d) for d in (8, 48, 64, 80, 127, 128)] == [64, 64, 64, 128, 128, 128]
    with pytest.raises(NotImplementedError):
        ops._attn_padded_head(160)
    b, s, h, d, dp = 2, 5, 3, 80, 128
    qkv = torch.randn((b, s, h * 3 * d), generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    padded = ops._pad_last(qkv, d, dp)
    assert padded.shape == (b, s, h * 3 * dp)
    t, tp = qkv.view(b, s, h, 3, d), padded.view(b, s, h, 3, dp)
    assert torch.equal(tp[..., :d], t) and torch.count_nonzero(tp[..., d:]) == 0
    q, k = t[..., 0, :].float(), t[..., 1, :].float()
    qp, kp = tp[..., 0, :].float(), tp[..., 1, :].float()
    # zeros add nothing to q.k (compared in float64: the order of a float32 sum may differ with the length)
    assert torch.equal(torch.einsum("bshd,bthd->bhst", q.double(), k.double()),
                       torch.einsum("bshd,bthd->bhst", qp.double(), kp.double()))
