from ._operation import classifier_3d, layernorm_3d, linear_3d, vocab_parallel_classifier_3d  # noqa: F401
from ._utils import reduce_by_batch_3d, split_batch_3d  # noqa: F401
from .module import Classifier3D, LayerNorm3D, Linear3D, VocabParallelClassifier3D  # noqa: F401
