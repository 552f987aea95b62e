from ._operation import (add_bias_2d, classifier_2d, layernorm_2d, summa_AB, summa_AB_bias_act, summa_ABT,  # noqa: F401
                         summa_ATB)
from ._utils import reduce_by_batch_2d, split_batch_2d  # noqa: F401
from .module import Classifier2D, LayerNorm2D, Linear2D, VocabParallelClassifier2D  # noqa: F401
