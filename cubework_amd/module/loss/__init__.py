from ._operation import vocab_parallel_cross_entropy  # noqa: F401
from .losses import (CrossEntropyLoss, CrossEntropyLoss2D, CrossEntropyLoss3D,  # noqa: F401
                     VocabParallelCrossEntropyLoss1D, VocabParallelCrossEntropyLoss2D,
                     VocabParallelCrossEntropyLoss3D)
