"""Single-process stand-in for cubework.distributed.

This build computes ONE rank's share on one GPU and never communicates. The
ParallelMode objects therefore only carry what the layers read
(cubework/distributed/utils.py:21-101: world_size, local_rank, rank_by_idx,
is_initialized) plus a mailbox: what a collective would deliver from the
peers is *pre-staged* with `mode.stage(op, value)` before the layer runs, and
what the rank would send is left in `mode.outbox`. At world size 1 every
collective is the identity, as in cubework/distributed/collective.py:8,30,50,67,84.

Use `initialize("2d", 4, row=0, col=1)` to make the layers behave as rank
(row 0, column 1) of a 2 x 2 SUMMA grid, or `initialize("2d", 1)` (and "1d",
"3d", None) for the self-contained tensor-parallel-size-1 case.
"""
from collections import defaultdict
from contextlib import contextmanager
from typing import Optional

import torch

from .global_vars import (PARALLEL_3D_INPUT, PARALLEL_3D_INPUT_X_WEIGHT, PARALLEL_3D_OUTPUT,
                          PARALLEL_3D_OUTPUT_X_WEIGHT, PARALLEL_3D_WEIGHT, env)


class MissingPeerData(RuntimeError):
    """A collective needed the peers' contribution and none was pre-staged."""


class ParallelMode:
    def __init__(self, name: str):
        self.name = name
        self.reset()

    def reset(self):
        self.world_size = 1
        self.local_rank = 0
        self._initialized = False
        self.inbox = defaultdict(list)
        self.outbox = defaultdict(list)

    def init(self, world_size: int = 1, local_rank: int = 0):
        assert 0 <= local_rank < world_size
        self.world_size = world_size
        self.local_rank = local_rank
        self._initialized = True
        self.inbox.clear()
        self.outbox.clear()

    def is_initialized(self) -> bool:
        return self._initialized

    def rank_by_idx(self, idx: int) -> int:
        return idx

    @property
    def ranks_in_group(self):
        return list(range(self.world_size))

    @property
    def group(self):
        return None

    # ---- mailbox -------------------------------------------------------
    def stage(self, op: str, value):
        """Pre-stage what collective `op` will deliver next (FIFO per op)."""
        self.inbox[op].append(value)

    def take(self, op: str):
        if not self.inbox[op]:
            raise MissingPeerData(
                "%s: '%s' over %d ranks needs the peers' data; stage it with "
                "pm.%s.stage('%s', ...) before the call (this build never communicates)"
                % (self.name, op, self.world_size, self.name, op))
        return self.inbox[op].pop(0)

    def post(self, op: str, value):
        self.outbox[op].append(value)


class _ParallelManager:
    NAMES = ["GLOBAL", "DATA", "TENSOR", "PARALLEL_1D", "PARALLEL_2D_ROW", "PARALLEL_2D_COL", PARALLEL_3D_INPUT,
             PARALLEL_3D_WEIGHT, PARALLEL_3D_OUTPUT, PARALLEL_3D_INPUT_X_WEIGHT, PARALLEL_3D_OUTPUT_X_WEIGHT]

    def __init__(self):
        for n in self.NAMES:
            setattr(self, n, ParallelMode(n))

    def reset(self):
        for n in self.NAMES:
            getattr(self, n).reset()


ParallelManager = _ParallelManager()
pm = ParallelManager


def initialize(tensor_parallel: Optional[str] = None, tensor_parallel_size: int = 1, *, rank: int = 0,
               row: int = 0, col: int = 0, coords=(0, 0, 0)):
    """Set up the single-rank view (cubework/initialize.py:24-59 without the
    process group).

    1d: `rank` of `tensor_parallel_size`. 2d: grid position (row, col) of a
    q x q grid, q = sqrt(size) (cubework/distributed/utils.py:195). 3d:
    coords = (input, weight, output) ranks in a depth^3 cube, depth =
    round(size^(1/3)) (utils.py:257).
    """
    if tensor_parallel not in (None, "1d", "2d", "3d"):
        raise ValueError("tensor_parallel must be None, '1d', '2d' or '3d'")
    pm.reset()
    env.load(mode=tensor_parallel)
    pm.GLOBAL.init(1, 0)
    pm.DATA.init(1, 0)
    if tensor_parallel is None:
        return
    if tensor_parallel == "1d":
        pm.TENSOR.init(tensor_parallel_size, rank)
        pm.PARALLEL_1D.init(tensor_parallel_size, rank)
    elif tensor_parallel == "2d":
        q = int(round(tensor_parallel_size ** 0.5))
        assert q * q == tensor_parallel_size, "2D tensor parallel size must be a square"
        env.summa_dim = q
        pm.TENSOR.init(tensor_parallel_size, row * q + col)
        # the ROW group holds the ranks of one grid row: its local rank is the column index
        pm.PARALLEL_2D_ROW.init(q, col)
        pm.PARALLEL_2D_COL.init(q, row)
    else:
        d = int(round(tensor_parallel_size ** (1.0 / 3.0)))
        assert d ** 3 == tensor_parallel_size, "3D tensor parallel size must be a cube"
        env.depth_3d = d
        i, w, o = coords
        pm.TENSOR.init(tensor_parallel_size, i + d * (w + d * o))
        getattr(pm, PARALLEL_3D_INPUT).init(d, i)
        getattr(pm, PARALLEL_3D_WEIGHT).init(d, w)
        getattr(pm, PARALLEL_3D_OUTPUT).init(d, o)
        getattr(pm, PARALLEL_3D_INPUT_X_WEIGHT).init(d * d, i * d + w)
        getattr(pm, PARALLEL_3D_OUTPUT_X_WEIGHT).init(d * d, o * d + w)
        env.input_group_3d = PARALLEL_3D_INPUT
        env.weight_group_3d = PARALLEL_3D_WEIGHT
        env.output_group_3d = PARALLEL_3D_OUTPUT
        env.input_x_weight_group_3d = PARALLEL_3D_INPUT_X_WEIGHT
        env.output_x_weight_group_3d = PARALLEL_3D_OUTPUT_X_WEIGHT


# --------------------------------------------------------------------------
# collectives: identity at world size 1, mailbox otherwise
# (signatures of cubework/distributed/collective.py:6-97)
# --------------------------------------------------------------------------
def all_gather(tensor, dim, parallel_mode, async_op=False):
    if parallel_mode.world_size == 1:
        out = tensor
    else:
        peers = list(parallel_mode.take("all_gather"))  # world_size entries, own slot ignored
        peers[parallel_mode.local_rank] = tensor
        out = torch.cat(peers, dim=dim)
    return (out, None) if async_op else out


def reduce_scatter(tensor, dim, parallel_mode, async_op=False):
    if parallel_mode.world_size == 1:
        out = tensor
    else:
        total = tensor
        for t in parallel_mode.take("reduce_scatter"):  # the peers' full tensors
            total = total + t
        out = torch.chunk(total, parallel_mode.world_size, dim=dim)[parallel_mode.local_rank].contiguous()
    return (out, None) if async_op else out


def all_reduce(tensor, parallel_mode, op="sum", async_op=False):
    if parallel_mode.world_size == 1:
        out = tensor
    else:
        out = tensor
        for t in parallel_mode.take("all_reduce"):  # the peers' tensors
            out = torch.maximum(out, t) if op == "max" else out + t
    return (out, None) if async_op else out


def broadcast(tensor, src, parallel_mode, async_op=False):
    if parallel_mode.world_size == 1 or src == parallel_mode.local_rank:
        out = tensor
    else:
        out = parallel_mode.take("broadcast")
    return (out, None) if async_op else out


def reduce(tensor, dst, parallel_mode, async_op=False):
    if parallel_mode.world_size == 1:
        out = tensor
    elif dst == parallel_mode.local_rank:
        out = tensor
        for t in parallel_mode.take("reduce"):
            out = out + t
    else:
        parallel_mode.post("reduce", (dst, tensor))
        out = tensor
    return (out, None) if async_op else out


@contextmanager
def seed(parallel_mode):
    """RNG fork used around parameter initialisation (cubework/utils/common.py:9-18).
    The per-rank generator states of the reference are not reproduced: the
    current generators are used and restored."""
    cpu_state = torch.get_rng_state()
    dev_state = torch.cuda.get_rng_state() if torch.cuda.is_available() else None
    try:
        yield
    finally:
        torch.set_rng_state(cpu_state)
        if dev_state is not None:
            torch.cuda.set_rng_state(dev_state)


def get_current_device():
    """cubework/utils/common.py:32-36."""
    if torch.cuda.is_available():
        return torch.device("cuda", torch.cuda.current_device())
    return torch.device("cpu")
