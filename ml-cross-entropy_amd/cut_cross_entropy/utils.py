"""Host-side helpers of the loss path (reference: cut_cross_entropy/utils.py)."""

from dataclasses import dataclass
from typing import Optional, Union

import torch

from cut_cross_entropy.constants import IGNORE_INDEX


def softcapping(logits: torch.Tensor, softcap: float) -> torch.Tensor:
    """tanh(x / softcap) * softcap (reference utils.py:12-14)."""
    return torch.tanh(logits / softcap) * softcap


def _handle_eps(filter_eps: Union[float, str, None], dtype: torch.dtype) -> Optional[float]:
    """Resolve the filter threshold (reference utils.py:17-25): ``None`` and floats
    pass through, "auto" is eps(dtype) / 32, anything else is a RuntimeError."""
    if filter_eps is None:
        return None
    if isinstance(filter_eps, float):
        return filter_eps
    if isinstance(filter_eps, str) and filter_eps == "auto":
        return torch.finfo(dtype).eps / 32
    raise RuntimeError(f"Unknown eps {filter_eps=}")


def _build_flat_valids(
    targets: torch.Tensor, ignore_index: int, shift: int
) -> Optional[torch.Tensor]:
    """int32 indices of the rows of the flattened ``e`` that enter the loss
    (reference utils.py:28-49).

    Without a shift the result is ``None`` when no target is ignored.  With a
    shift, row (b, t) enters iff ``targets[b, t + shift]`` is not ignored, the
    index is relative to the *unsliced* layout, and a tensor is always returned;
    the matching target / upstream-gradient index is ``valid + shift``.
    """
    if shift == 0:
        flat = targets.reshape(-1)
        keep = torch.nonzero(flat != ignore_index).squeeze(1).to(torch.int32)
        return None if keep.numel() == flat.numel() else keep

    assert targets.stride(-1) == 1
    T = targets.size(-1)
    window = targets[..., shift:]
    # positions inside the sliced view, turned into offsets of the unsliced tensor
    pos = torch.nonzero(window.reshape(-1, T - shift) != ignore_index)
    return (pos[:, 0] * T + pos[:, 1]).to(torch.int32)


def handle_reduction_none(
    batch_shape: torch.Size, valids: Optional[torch.Tensor], shift: int, loss: torch.Tensor
) -> torch.Tensor:
    """Per-valid-row values placed at their batch positions (row + shift), zeros elsewhere
    (reference utils.py:52-61)."""
    if valids is None:
        return loss.view(batch_shape)
    out = torch.zeros(batch_shape.numel(), dtype=loss.dtype, device=loss.device)
    out.index_copy_(0, valids.long() + shift, loss)
    return out.view(batch_shape)


def compute_z_loss(
    lse: torch.Tensor,
    targets: Optional[torch.Tensor] = None,
    shift: Union[bool, int] = False,
    ignore_index: int = IGNORE_INDEX,
    reduction: str = "mean",
) -> torch.Tensor:
    """Z loss, the square of the log-sum-exp, zero where the (shifted) target is ignored; "mean" is taken
    over the positions that count (reference utils.py:64-102)."""
    if reduction not in ("mean", "sum", "none"):
        raise ValueError(f"Invalid reduction: {reduction}")
    sq = lse.square()
    counted = sq.numel()
    if targets is not None:
        kept = targets[..., int(shift):] != ignore_index
        sq = sq.masked_fill(~kept, 0.0)
        counted = kept.sum()
    if reduction == "none":
        return sq
    total = sq.sum()
    return total / counted if reduction == "mean" else total


@dataclass
class TensorInfo:
    """dtype / requires_grad of an input as the caller passed it (before autocast)."""

    dtype: torch.dtype
    requires_grad: bool
