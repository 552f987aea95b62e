"""Drop-in for the Linear / LayerNorm / Classifier / CrossEntropyLoss part of
`cubework.module` (cubework/module/__init__.py:1-6), and for Embedding.
PatchEmbedding, Dropout, DropPath and the metrics are outside this package's scope."""
from .init import (kaiming_normal_, kaiming_uniform_, lecun_normal_, lecun_uniform_, normal_, ones_,  # noqa: F401
                   trunc_normal_, uniform_, xavier_normal_, xavier_uniform_, zeros_)
from .embedding import (Embedding, Embedding1D, Embedding2D, Embedding3D, VocabParallelEmbedding1D,  # noqa: F401
                        VocabParallelEmbedding2D, VocabParallelEmbedding3D)
from .loss import CrossEntropyLoss  # noqa: F401
from .modules import Classifier, LayerNorm, Linear, partition_batch  # noqa: F401
