"""cubework_amd: the per-rank compute of Cubework's tensor-parallel layers
(SUMMA block GEMM + bias + activation, LayerNorm2D/3D, vocab-parallel
cross-entropy) as hand-written gfx950 HIP kernels behind the `cubework.module`
layer API. One rank, one MI355X, no communication: operands a collective
would deliver are pre-staged.

    from cubework_amd.distributed import initialize
    import cubework_amd.module as cube_nn
    initialize("2d", 1)
    layer = cube_nn.Linear(2048, 8192, dtype=torch.bfloat16).cuda()
"""
from .global_vars import env  # noqa: F401
from .distributed import ParallelManager, initialize  # noqa: F401

__version__ = "0.1.0"
