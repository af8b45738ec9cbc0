"""Cut Cross-Entropy for AMD MI355X (gfx950): the ``cut_cross_entropy`` operator API backed by
hand-written HIP kernels (reference exports: cut_cross_entropy/__init__.py:9-14)."""

from cut_cross_entropy.cce_utils import LinearCrossEntropyImpl
from cut_cross_entropy.linear_cross_entropy import LinearCrossEntropy, linear_cross_entropy
from cut_cross_entropy.vocab_parallel import VocabParallelOptions

__all__ = [
    "LinearCrossEntropy",
    "LinearCrossEntropyImpl",
    "linear_cross_entropy",
    "VocabParallelOptions",
]

__version__ = "0.1.0"
