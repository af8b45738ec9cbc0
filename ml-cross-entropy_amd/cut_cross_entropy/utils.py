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
    """Scatter per-valid-row values into zeros of the batch shape
    (reference utils.py:52-61)."""
    if valids is None:
        return loss.view(batch_shape)
    full = loss.new_zeros((batch_shape.numel(),))
    full[(valids + shift).long() if shift != 0 else valids.long()] = loss
    return full.view(batch_shape)


def compute_z_loss(
    lse: torch.Tensor,
    targets: Optional[torch.Tensor] = None,
    shift: Union[bool, int] = False,
    ignore_index: int = IGNORE_INDEX,
    reduction: str = "mean",
) -> torch.Tensor:
    """Z loss ``lse ** 2`` with ignored tokens masked out; "mean" averages over the
    tokens that are not ignored (reference utils.py:64-102)."""
    z_loss = lse.pow(2)

    if targets is not None:
        shift = int(shift)
        if shift != 0:
            targets = targets[..., shift:]
        keep = targets != ignore_index
        z_loss = torch.where(keep, z_loss, 0.0)
        if reduction == "mean":
            z_loss = z_loss * (z_loss.numel() / keep.count_nonzero().type_as(z_loss))

    if reduction == "mean":
        return z_loss.mean()
    if reduction == "sum":
        return z_loss.sum()
    if reduction == "none":
        return z_loss
    raise ValueError(f"Invalid reduction: {reduction}")


@dataclass
class TensorInfo:
    """dtype / requires_grad of an input as the caller passed it (before autocast)."""

    dtype: torch.dtype
    requires_grad: bool
