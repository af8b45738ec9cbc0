"""Options of a patched model and the call into ``linear_cross_entropy``.

Restates ref: transformers/utils.py:14-78 (``PatchOptions``, ``apply_lce``).
"""

import dataclasses
from typing import Optional, Union

import torch

from cut_cross_entropy.linear_cross_entropy import linear_cross_entropy


@dataclasses.dataclass
class PatchOptions:
    """What ``cce_patch`` was asked for (ref: transformers/utils.py:19-48)."""

    impl: str
    reduction: str
    filter_eps: Union[float, str, None]
    accum_e_fp32: bool
    accum_c_fp32: bool
    filter_e_grad: bool
    filter_c_grad: bool
    train_only: bool

    def to_kwargs(self) -> dict:
        """The fields that are arguments of ``linear_cross_entropy`` (all but ``train_only``)."""
        kwargs = dataclasses.asdict(self)
        del kwargs["train_only"]
        return kwargs

    def use_lce(self, labels: Optional[torch.Tensor], training: bool) -> bool:
        """The fused loss needs labels; with ``train_only`` it is also skipped outside training."""
        return labels is not None and (training or not self.train_only)


def apply_lce(
    e: torch.Tensor,
    c: torch.Tensor,
    labels: torch.Tensor,
    opts: PatchOptions,
    bias: Optional[torch.Tensor] = None,
    softcap: Optional[float] = None,
    **loss_kwargs,
) -> torch.Tensor:
    """Next-token loss of hidden states ``e`` against the classifier ``c`` (ref: transformers/utils.py:51-78).

    ``num_items_in_batch`` (the trainer's gradient-accumulation normaliser) turns a mean into a sum
    divided by that count, as the reference does.  ``softcap`` carries a model's final logit
    soft-capping (Gemma 2) into the fused loss; the reference's patch drops it on this path.
    """
    kwargs = opts.to_kwargs()
    denominator = loss_kwargs.get("num_items_in_batch")
    per_item = denominator is not None and kwargs["reduction"] == "mean"
    if per_item:
        kwargs["reduction"] = "sum"
    loss = linear_cross_entropy(e, c, labels.to(e.device), bias=bias, softcap=softcap, shift=True, **kwargs)
    return loss / denominator if per_item else loss
