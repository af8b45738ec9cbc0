"""Options of a patched model and the call into ``linear_cross_entropy``.

Restates ref: transformers/utils.py:14-78 (``PatchOptions``, ``apply_lce``).
"""

from dataclasses import dataclass
from typing import Optional, Union

import torch

from cut_cross_entropy.linear_cross_entropy import linear_cross_entropy


@dataclass
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
        return dict(
            impl=self.impl,
            reduction=self.reduction,
            filter_eps=self.filter_eps,
            accum_e_fp32=self.accum_e_fp32,
            accum_c_fp32=self.accum_c_fp32,
            filter_e_grad=self.filter_e_grad,
            filter_c_grad=self.filter_c_grad,
        )

    def use_lce(self, labels: Optional[torch.Tensor], training: bool) -> bool:
        """The fused loss runs when there are labels, and in eval mode only unless ``train_only``."""
        if labels is None:
            return False
        if not training and self.train_only:
            return False
        return True


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
    num_items_in_batch = loss_kwargs.get("num_items_in_batch", None)
    cce_kwargs = opts.to_kwargs()
    if num_items_in_batch is not None and cce_kwargs["reduction"] == "mean":
        cce_kwargs["reduction"] = "sum"
    else:
        num_items_in_batch = None

    loss = linear_cross_entropy(
        e,
        c,
        labels.to(e.device),
        bias=bias,
        shift=True,
        softcap=softcap,
        **cce_kwargs,
    )

    if num_items_in_batch is not None:
        loss = loss / num_items_in_batch
    return loss
