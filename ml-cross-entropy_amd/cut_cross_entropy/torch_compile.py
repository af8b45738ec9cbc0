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


def _wide_logits(e, c, bias, softcap) -> torch.Tensor:
    """fp32 copy of the (biased, soft-capped) logits, computed in the input dtype like the reference does."""
    z = e @ c.T
    if bias is not None:
        z = z + bias
    if softcap is not None:
        z = softcapping(z, softcap)
    return z.float()


def _reduce(per_row: torch.Tensor, reduction: str) -> torch.Tensor:
    if reduction == "none":
        return per_row
    if reduction == "sum":
        return per_row.sum()
    if reduction == "mean":
        return per_row.mean()
    raise ValueError(f"Unknown reduction {reduction!r}")


def torch_compile_linear_cross_entropy_apply(
    e, c, targets, bias=None, softcap=None, *, ignore_index=IGNORE_INDEX, reduction="mean",
    return_lse=False,
):
    """Reference: torch_compile.py:18-49 (run eagerly here)."""
    wide = _wide_logits(e, c, bias, softcap)
    if not return_lse:
        return F.cross_entropy(wide, targets, ignore_index=ignore_index, reduction=reduction), None
    lse = torch.logsumexp(wide, dim=-1)
    log_p = wide - lse.unsqueeze(-1)
    return F.nll_loss(log_p, targets, ignore_index=ignore_index, reduction=reduction), lse


def _shard_apply(vp: VocabParallelOptions, e, c, targets, bias, softcap, reduction, return_lse):
    """One vocabulary shard without the exchange steps (reference:
    vocab_parallel/vocab_parallel_torch_compile.py:64-134): the shard's log-sum-exp, and the correct logit
    only for the rows whose target the shard holds."""
    wide = _wide_logits(e, c, bias, softcap)
    lse = torch.logsumexp(wide, dim=-1)
    local = targets - vp.start
    held = (local >= 0) & (local < c.size(0))
    picked = wide.gather(1, local.clamp(0, c.size(0) - 1).view(-1, 1)).squeeze(1)
    per_row = lse - picked * held
    return _reduce(per_row, reduction), (lse if return_lse else None)


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
    shift = int(shift)
    batch_shape = targets.size()
    targets = targets.contiguous()
    valids = _build_flat_valids(targets, ignore_index, shift)

    rows = e.contiguous().flatten(0, -2)
    labels = targets.flatten()
    if valids is not None:
        rows = rows[valids.long()]
        labels = labels[valids.long() + shift]

    if vocab_parallel_options is None:
        loss, lse = torch_compile_linear_cross_entropy_apply(
            rows, c, labels, bias, softcap, ignore_index=ignore_index, reduction=reduction, return_lse=return_lse)
    else:
        require_single_rank(vocab_parallel_options)
        loss, lse = _shard_apply(vocab_parallel_options, rows, c, labels, bias, softcap, reduction, return_lse)

    def to_batch(per_row):
        full = handle_reduction_none(batch_shape, valids, shift, per_row)
        return full[..., shift:] if shift else full

    if reduction == "none":
        loss = to_batch(loss)
    if return_lse:
        assert lse is not None
        lse = to_batch(lse)
    return loss, lse
