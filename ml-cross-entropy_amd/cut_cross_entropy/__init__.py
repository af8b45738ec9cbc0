"""Cut Cross-Entropy for AMD MI355X (gfx950).

The ``cut_cross_entropy`` operator API (reference exports: cut_cross_entropy/__init__.py:9-14) backed by
hand-written HIP kernels behind a C ABI (``_lib/libcce_hip.so``, built by ``csrc/Makefile``)::

    from cut_cross_entropy import linear_cross_entropy
    loss = linear_cross_entropy(hidden, lm_head.weight, labels, shift=1)    # impl="cce"
    loss, lse = linear_cross_entropy(e, c, t, softcap=30.0, return_lse=True, impl="cce_exact")

The logit matrix ``e @ c.T`` is never written to memory; see ``linear_cross_entropy`` for the arguments.
There is no CPU fallback: the ``cce*`` implementations raise when the library or a GPU is missing.
"""

__version__ = "0.1.0"

from .cce_utils import LinearCrossEntropyImpl  # noqa: E402
from .linear_cross_entropy import LinearCrossEntropy, linear_cross_entropy  # noqa: E402
from .vocab_parallel import VocabParallelOptions  # noqa: E402

__all__ = ["linear_cross_entropy", "LinearCrossEntropy", "LinearCrossEntropyImpl", "VocabParallelOptions"]
