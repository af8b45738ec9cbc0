"""Launcher of the gather-dot for the correct-class logit
(reference: cut_cross_entropy/indexed_dot.py:101-158)."""

from typing import Optional

import torch

from cut_cross_entropy import _hip


def indexed_neg_dot_forward_kernel(
    e: torch.Tensor,
    c: torch.Tensor,
    inds: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    shift: int = 0,
    valids: Optional[torch.Tensor] = None,
    softcap: Optional[float] = None,
    out_dtype: Optional[torch.dtype] = None,
    target_offset: int = 0,
) -> torch.Tensor:
    """``softcap(-(e[valid_i] . c[inds[valid_i + shift] - target_offset]) - bias[...])``.

    Rows whose (offset) index falls outside ``[0, c.size(0))`` give exactly 0; that is how
    a vocabulary shard ignores the rows whose target another shard holds.  ``target_offset``
    is an addition to the reference signature (its caller rebases ``inds`` on the host,
    cce.py:113).  The result has ``e.dtype`` unless ``out_dtype`` is given (reference :153-156).
    """
    assert inds.ndim == 1
    assert e.ndim == 2
    assert c.ndim == 2
    assert inds.size(0) == e.size(0)
    assert c.size(1) == e.size(1)
    assert e.is_contiguous()
    _hip.require_gpu_tensor("e", e)
    assert c.device == e.device and c.dtype == e.dtype
    if valids is not None:
        assert valids.ndim == 1 and valids.dtype == torch.int32
        valids = valids.contiguous()
        B = valids.size(0)
    else:
        B = e.size(0)
    inds = inds.to(torch.int64).contiguous()
    if bias is not None:
        bias = bias.to(e.dtype).contiguous()
    code = _hip.dtype_code(e.dtype)
    lib = _hip.load()

    out = torch.empty((B,), dtype=torch.float32, device=e.device)
    if B > 0:
        with torch.cuda.device(e.device):
            status = lib.cce_indexed_neg_dot(
                e.data_ptr(), c.data_ptr(), inds.data_ptr(), _hip.ptr(bias), _hip.ptr(valids),
                out.data_ptr(),
                e.size(0), B, c.size(0), e.size(1),
                e.stride(0), c.stride(0), c.stride(1),
                int(shift), int(target_offset),
                float(softcap) if softcap is not None else 0.0, code,
                _hip.current_stream_ptr(e.device),
            )
        _hip.check(status, "cce_indexed_neg_dot")
    if out_dtype is None:
        out_dtype = e.dtype
    return out.to(out_dtype)
