"""Launcher of the fused matmul + log-sum-exp kernel
(reference: cut_cross_entropy/cce_lse_forward.py:170-237)."""

from typing import Optional, Tuple, Union

import torch

from cut_cross_entropy import _hip


def lse_forward(
    e: torch.Tensor,
    c: torch.Tensor,
    bias: Optional[torch.Tensor],
    valids: Optional[torch.Tensor],
    softcap: Optional[float],
    want_logit_avg: bool = False,
    want_tile_max: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Returns ``(lse[B] fp32, logit_avg[V] fp32 | None, tile_max | None)``.

    ``tile_max`` holds the largest soft-capped logit of every 32-row x 32-class cell;
    the backward uses it to drop tiles without recomputing them.
    """
    assert e.ndim == 2 and c.ndim == 2
    assert e.shape[1] == c.shape[1], "Incompatible dimensions"
    assert e.is_contiguous(), "Matrix A must be contiguous"
    _hip.require_gpu_tensor("e", e)
    assert c.device == e.device and c.dtype == e.dtype
    if valids is not None:
        assert valids.ndim == 1 and valids.dtype == torch.int32
        valids = valids.contiguous()
        B = valids.numel()
    else:
        B = e.shape[0]
    if bias is not None:
        assert bias.ndim == 1
        assert c.shape[0] == bias.shape[0]
        bias = bias.to(e.dtype).contiguous()
    V, D = c.shape
    code = _hip.dtype_code(e.dtype)
    lib = _hip.load()

    lse = torch.empty((B,), dtype=torch.float32, device=e.device)
    logit_avg = torch.empty((V,), dtype=torch.float32, device=e.device) if want_logit_avg else None
    tile_max = None
    if want_tile_max:
        tile_max = torch.empty((lib.cce_tile_stat_elems(B, V),), dtype=torch.float32, device=e.device)
    if B == 0:
        if logit_avg is not None:
            logit_avg.zero_()
        return lse, logit_avg, tile_max

    ws_bytes = lib.cce_lse_forward_workspace_bytes(B, V, D)
    workspace = torch.empty((max(ws_bytes, 8) // 8,), dtype=torch.int64, device=e.device)
    with torch.cuda.device(e.device), _hip.timed("lse_forward", e.device):
        status = lib.cce_lse_forward(
            e.data_ptr(), c.data_ptr(), _hip.ptr(bias), _hip.ptr(valids),
            lse.data_ptr(), _hip.ptr(logit_avg), _hip.ptr(tile_max),
            workspace.data_ptr(), workspace.numel() * 8,
            e.shape[0], B, V, D,
            e.stride(0), c.stride(0), c.stride(1),
            float(softcap) if softcap is not None else 0.0, code,
            _hip.current_stream_ptr(e.device),
        )
    _hip.check(status, "cce_lse_forward")
    return lse, logit_avg, tile_max


def cce_lse_forward_kernel(
    e: torch.Tensor,
    c: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    valids: Optional[torch.Tensor] = None,
    softcap: Optional[float] = None,
    return_logit_avg: bool = False,
) -> Union[Tuple[torch.Tensor, torch.Tensor], torch.Tensor]:
    """Same call as the reference launcher: ``lse`` or ``(lse, logit_avg)``."""
    lse, logit_avg, _ = lse_forward(e, c, bias, valids, softcap, want_logit_avg=return_logit_avg)
    if return_logit_avg:
        assert logit_avg is not None
        return lse, logit_avg
    return lse
