from ._operation import linear_nt  # noqa: F401
from .module import (Classifier1D, LayerNorm1D, Linear1D, Linear1D_Col, Linear1D_Row,  # noqa: F401
                     VocabParallelClassifier1D)
