"""The dense alternative ``impl="torch_compile"`` (reference: cut_cross_entropy/torch_compile.py).

It materialises the logits with ordinary PyTorch operators on whatever device the inputs
live on.  It is a separate, explicitly selected implementation: the cce implementations
never fall back to it.
"""

from typing import Optional, Tuple, Union

import torch
import torch.nn.functional as F

from cut_cross_entropy.constants import IGNORE_INDEX
from cut_cross_entropy.utils import _build_flat_valids, handle_reduction_none, softcapping
from cut_cross_entropy.vocab_parallel.utils import VocabParallelOptions, require_single_rank


def torch_compile_linear_cross_entropy_apply(
    e, c, targets, bias=None, softcap=None, *, ignore_index=IGNORE_INDEX, reduction="mean",
    return_lse=False,
):
    """Reference: torch_compile.py:18-49 (run eagerly here)."""
    logits = e @ c.T
    if bias is not None:
        logits = logits + bias
    if softcap is not None:
        logits = softcapping(logits, softcap)
    wide = logits.float()
    if not return_lse:
        return F.cross_entropy(wide, targets, ignore_index=ignore_index, reduction=reduction), None
    lse = torch.logsumexp(wide, dim=-1)
    loss = F.nll_loss(wide - lse.unsqueeze(-1), targets, ignore_index=ignore_index, reduction=reduction)
    return loss, lse


def _shard_apply(vp: VocabParallelOptions, e, c, targets, bias, softcap, reduction, return_lse):
    """One vocabulary shard without the exchange steps
    (reference: vocab_parallel/vocab_parallel_torch_compile.py:64-134)."""
    logits = e @ c.T
    if bias is not None:
        logits = logits + bias
    if softcap is not None:
        logits = softcapping(logits, softcap)
    wide = logits.float()
    lse = torch.logsumexp(wide, dim=-1)
    mine = (targets >= vp.start) & (targets < vp.stop)
    local = torch.where(mine, targets - vp.start, torch.zeros_like(targets))
    correct = torch.where(mine, wide.gather(1, local.view(-1, 1)).squeeze(1), wide.new_zeros(()))
    loss = lse - correct
    if reduction == "mean":
        loss = loss.mean()
    elif reduction == "sum":
        loss = loss.sum()
    elif reduction != "none":
        raise ValueError(f"Unknown reduction {reduction!r}")
    return loss, (lse if return_lse else None)


def torch_compile_linear_cross_entropy(
    e: torch.Tensor,
    c: torch.Tensor,
    targets: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    ignore_index: int = IGNORE_INDEX,
    softcap: Optional[float] = None,
    reduction: str = "mean",
    shift: Union[bool, int] = 0,
    vocab_parallel_options: Optional[VocabParallelOptions] = None,
    return_lse: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Reference: torch_compile.py:53-117."""
    assert e.size()[0:-1] == targets.size()
    assert e.size(-1) == c.size(1)
    batch_shape = targets.size()
    e = e.contiguous()
    targets = targets.contiguous()
    shift = int(shift)
    valids = _build_flat_valids(targets, ignore_index, shift)

    e = e.flatten(0, -2)
    targets = targets.flatten()
    if valids is not None:
        rows = valids.long()
        e = e[rows]
        targets = targets[rows + shift]

    if vocab_parallel_options is None:
        loss, lse = torch_compile_linear_cross_entropy_apply(
            e, c, targets, bias, softcap, ignore_index=ignore_index, reduction=reduction,
            return_lse=return_lse,
        )
    else:
        require_single_rank(vocab_parallel_options)
        loss, lse = _shard_apply(
            vocab_parallel_options, e, c, targets, bias, softcap, reduction, return_lse
        )

    if reduction == "none":
        loss = handle_reduction_none(batch_shape, valids, shift, loss)
        if shift != 0:
            loss = loss[..., shift:]
    if return_lse:
        assert lse is not None
        lse = handle_reduction_none(batch_shape, valids, shift, lse)
        if shift != 0:
            lse = lse[..., shift:]
    return loss, lse
