"""Public operator (reference: cut_cross_entropy/linear_cross_entropy.py:103-255).

``linear_cross_entropy(e, c, targets, ...)`` computes
``F.cross_entropy((e @ c.T).float(), targets)`` without writing the logit matrix to
memory.  Parameters:

:param e: embeddings, shape (..., D)
:param c: classifier, shape (NumClasses, D)
:param targets: target class per input, values in [0, NumClasses) or ``ignore_index``, shape (...)
:param bias: optional (NumClasses,) added to the logits
:param ignore_index: targets with this value do not enter the loss
:param softcap: logit soft-capping value, ``tanh(x / softcap) * softcap``
:param reduction: "mean" (over the non-ignored tokens), "sum" or "none"
:param shift: n-th next token prediction: row t is scored against ``targets[..., t + shift]``;
    ``True`` means 1.  Must be in [0, T).
:param return_lse: also return the log-sum-exp per token (for a z-loss)
:param filter_eps: gradient-filter threshold; "auto" = eps(dtype) / 32, ``None`` = off  (cce only)
:param accum_e_fp32 / accum_c_fp32: accumulate dE / dC in fp32 buffers  (cce only)
:param filter_e_grad / filter_c_grad: apply the gradient filter to dE / dC  (cce only)
:param impl: one of the names of ``LinearCrossEntropyImpl`` (lower case) or the enum itself.
    Every ``cce*`` name other than "cce" fixes the cce options and ignores the caller's.
:param vocab_parallel_options: bounds of the vocabulary shard held in ``c``
"""

import platform
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn

from cut_cross_entropy.cce_utils import CCEPreset, CCEPresets, LinearCrossEntropyImpl, impl_name
from cut_cross_entropy.constants import IGNORE_INDEX
from cut_cross_entropy.torch_compile import torch_compile_linear_cross_entropy
from cut_cross_entropy.vocab_parallel.utils import VocabParallelOptions

LCE_IMPL_DEFAULT = LinearCrossEntropyImpl.CCE

_DTENSOR_MESSAGE = (
    "Received {name} as a torch.distributed.tensor.DTensor. "
    "This is not supported. "
    "If possible, change the sharding strategy such that {name} is already unsharded."
)


def _reject_dtensors(**tensors) -> None:
    try:
        from torch.distributed.tensor import DTensor
    except Exception:  # torch built without distributed
        return
    for name, value in tensors.items():
        if isinstance(value, DTensor):
            raise ValueError(_DTENSOR_MESSAGE.format(name=name))


def _check_arguments(c, targets, bias, shift, vocab_parallel_options) -> None:
    """The argument errors of the reference (linear_cross_entropy.py:131-145), same types and conditions."""
    steps = targets.size(-1)
    if isinstance(shift, int) and not 0 <= shift < steps:
        raise ValueError(f"Shift must be in the range [0, {steps}). Got {shift}.")
    if vocab_parallel_options is not None:
        held = vocab_parallel_options.stop - vocab_parallel_options.start
        if c.size(0) != held:
            raise ValueError(f"Expected c.size(0) to be {held}, got {c.size(0)}.")
    if bias is not None and bias.size(0) != c.size(0):
        raise ValueError(f"Bias has a different number of elements than c. {bias.size(0)} vs. {c.size(0)}.")


def linear_cross_entropy(
    e: torch.Tensor,
    c: torch.Tensor,
    targets: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    ignore_index: int = IGNORE_INDEX,
    softcap: Optional[float] = None,
    reduction: str = "mean",
    shift: Union[bool, int] = 0,
    return_lse: bool = False,
    filter_eps: Union[float, str, None] = "auto",
    accum_e_fp32: bool = False,
    accum_c_fp32: bool = False,
    filter_e_grad: bool = True,
    filter_c_grad: bool = True,
    impl: Union[str, LinearCrossEntropyImpl] = LCE_IMPL_DEFAULT,
    vocab_parallel_options: Optional[VocabParallelOptions] = None,
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    _reject_dtensors(e=e, c=c, targets=targets, bias=bias)
    impl = impl_name(impl)
    _check_arguments(c, targets, bias, shift, vocab_parallel_options)
    common = dict(bias=bias, ignore_index=ignore_index, softcap=softcap, reduction=reduction, shift=shift,
                  vocab_parallel_options=vocab_parallel_options, return_lse=return_lse)

    if impl == "torch_compile":
        loss, lse = torch_compile_linear_cross_entropy(e, c, targets, **common)
    elif impl in CCEPresets.names:
        if platform.system() == "Darwin":
            raise RuntimeError("CCE does not support MacOS. Please use torch_compile when running on MacOS instead.")
        from cut_cross_entropy.cce import cce_linear_cross_entropy  # needs the HIP library: imported on use

        asked = CCEPreset(filter_eps=filter_eps, accum_e_fp32=accum_e_fp32, accum_c_fp32=accum_c_fp32,
                          filter_e_grad=filter_e_grad, filter_c_grad=filter_c_grad)
        loss, lse = cce_linear_cross_entropy(e, c, targets, **common, **CCEPresets.build_for_impl(impl, asked))
    else:
        raise NotImplementedError(f"{impl} is not implemented.")

    if not return_lse:
        return loss
    assert lse is not None
    return loss, lse


linear_cross_entropy.__doc__ = __doc__

_MODULE_OPTIONS = ("ignore_index", "softcap", "reduction", "shift", "filter_eps", "accum_e_fp32", "accum_c_fp32",
                   "filter_e_grad", "filter_c_grad", "impl", "return_lse")


class LinearCrossEntropy(nn.Module):
    """Module form of :func:`linear_cross_entropy` (reference :201-255): the options are fixed at
    construction and kept as attributes of the same names, the tensors arrive in ``forward``."""

    def __init__(
        self,
        ignore_index: int = IGNORE_INDEX,
        softcap: Optional[float] = None,
        reduction: str = "mean",
        shift: Union[bool, int] = 0,
        filter_eps: Union[float, str, None] = "auto",
        accum_e_fp32: bool = False,
        accum_c_fp32: bool = False,
        filter_e_grad: bool = True,
        filter_c_grad: bool = True,
        impl: Union[str, LinearCrossEntropyImpl] = LCE_IMPL_DEFAULT,
        return_lse: bool = False,
    ):
        super().__init__()
        given = locals()
        for name in _MODULE_OPTIONS:
            setattr(self, name, given[name])

    def forward(self, e, c, targets, bias=None):
        return linear_cross_entropy(e, c, targets, bias=bias, **{name: getattr(self, name) for name in _MODULE_OPTIONS})
