"""Autograd glue of the Cut Cross-Entropy loss (reference: cut_cross_entropy/cce.py).

Forward: fused matmul + log-sum-exp kernel -> gather-dot for the correct-class logit ->
``nll = lse - correct_logit`` -> reduction.  Backward: one fused kernel that recomputes
logit tiles and accumulates dE / dC / dBias.  All three kernels are hand-written gfx950
HIP code behind the C ABI of ``libcce_hip.so``.
"""

from dataclasses import dataclass
from typing import Optional, Tuple, Union

import torch
import torch.amp

from cut_cross_entropy import _hip, fp32_path
from cut_cross_entropy.cce_backward import cce_backward_kernel
from cut_cross_entropy.cce_lse_forward import lse_forward
from cut_cross_entropy.constants import IGNORE_INDEX
from cut_cross_entropy.indexed_dot import indexed_neg_dot_forward_kernel
from cut_cross_entropy.utils import (
    TensorInfo,
    _build_flat_valids,
    _handle_eps,
    handle_reduction_none,
)
from cut_cross_entropy.vocab_parallel.utils import VocabParallelOptions, require_single_rank


@dataclass
class CCEParams:
    targets: torch.Tensor
    valids: Optional[torch.Tensor]
    softcap: Optional[float]
    reduction: str
    filter_eps: Optional[float]
    shift: int
    batch_shape: torch.Size
    accum_e_fp32: bool
    accum_c_fp32: bool
    filter_e_grad: bool
    filter_c_grad: bool
    vocab_parallel_options: Optional[VocabParallelOptions]
    return_lse: bool


# Device tensor of uint64[4] that, when set, receives the backward tile counters
# (tiles in the grid, recomputed, with a dE product, with a dC product).  Used by the
# benchmark to report the kept-tile fractions of the timed run.
_tile_counters: Optional[torch.Tensor] = None


def set_tile_counters(t: Optional[torch.Tensor]) -> None:
    global _tile_counters
    _tile_counters = t


class LinearCrossEntropyFunction(torch.autograd.Function):
    """Reference: cce.py:48-235."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, e, c, bias, params: CCEParams):
        needs_grad = e.requires_grad or c.requires_grad or (bias is not None and bias.requires_grad)
        # the forward statistic that lets the backward drop tiles is only useful with filtering
        want_tile_max = needs_grad and params.filter_eps is not None

        e_info = TensorInfo(e.dtype, e.requires_grad)
        c_info = TensorInfo(c.dtype, c.requires_grad)
        bias_info = TensorInfo(bias.dtype, bias.requires_grad) if bias is not None else None

        if torch.is_autocast_enabled():
            low = torch.get_autocast_gpu_dtype()
            e = e.to(dtype=low)
            c = c.to(dtype=low)
            if bias is not None:
                bias = bias.to(dtype=low)

        vp = params.vocab_parallel_options
        ctx.fp32 = e.dtype == torch.float32
        if ctx.fp32:
            # fp32 values as three bf16 parts along a six times longer reduction axis: fp32_path.py
            assert c.dtype == torch.float32, "e and c must have the same dtype"
            _hip.require_gpu_tensor("e", e)
            e = e.contiguous()
            lse = fp32_path.fp32_lse(e, c, bias, params.valids, params.softcap)
            tile_max = None
            neg_dot = fp32_path.fp32_indexed_neg_dot(
                e, c, bias, params.targets, params.valids, params.shift, params.softcap,
                vp.start if vp is not None else 0)
        else:
            lse, _, tile_max = lse_forward(
                e, c, bias, params.valids, params.softcap, want_tile_max=want_tile_max
            )
            neg_dot = indexed_neg_dot_forward_kernel(
                e=e,
                c=c,
                inds=params.targets,
                bias=bias,
                shift=params.shift,
                valids=params.valids,
                softcap=params.softcap,
                out_dtype=lse.dtype,
                target_offset=vp.start if vp is not None else 0,
            )
        nll = neg_dot.add_(lse)

        ctx.save_for_backward(e, c, bias, lse, params.targets, params.valids, tile_max)
        ctx.params = params
        ctx.e_info = e_info
        ctx.c_info = c_info
        ctx.bias_info = bias_info

        lse_out = None
        if params.return_lse:
            lse_out = handle_reduction_none(params.batch_shape, params.valids, params.shift, lse)

        reduction = params.reduction
        if reduction == "mean":
            loss = nll.mean()
        elif reduction == "sum":
            loss = nll.sum()
        elif reduction == "none":
            loss = handle_reduction_none(params.batch_shape, params.valids, params.shift, nll)
        else:
            raise ValueError(f"Unknown reduction {reduction}")
        return loss, lse_out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_out, grad_lse_out):
        e, c, bias, lse, targets, valids, tile_max = ctx.saved_tensors
        params: CCEParams = ctx.params

        reduction = params.reduction
        if reduction == "mean":
            # zero valid rows: the forward already returned NaN; give zero gradients
            grad_scale = 1.0 / lse.numel() if lse.numel() > 0 else 0.0
        elif reduction == "sum":
            grad_scale = 1.0
        elif reduction == "none":
            grad_scale = 1.0
            grad_out = grad_out.reshape(-1)
        else:
            raise ValueError(f"Unknown reduction {reduction}")
        if grad_lse_out is not None:
            grad_lse_out = grad_lse_out.reshape(-1)

        vp = params.vocab_parallel_options
        if ctx.fp32:
            de, dc, dbias = fp32_path.fp32_backward(
                e, c, bias, lse, grad_out, grad_lse_out, valids, targets, params.shift,
                vp.start if vp is not None else 0, params.softcap, grad_scale,
                ctx.e_info.requires_grad, ctx.c_info.requires_grad,
                ctx.bias_info is not None and ctx.bias_info.requires_grad)
            if dbias is not None:
                dbias = dbias.to(ctx.bias_info.dtype)
            return de, dc, dbias, None
        de, dc, dbias = cce_backward_kernel(
            do=grad_out,
            dlse=grad_lse_out,
            e=e,
            e_info=ctx.e_info,
            c=c,
            c_info=ctx.c_info,
            bias=bias,
            bias_info=ctx.bias_info,
            lse=lse,
            valids=valids,
            softcap=params.softcap,
            filter_eps=params.filter_eps,
            targets=targets,
            shift=params.shift,
            vocab_ordering=None,
            grad_scale=grad_scale,
            accum_e_fp32=params.accum_e_fp32,
            accum_c_fp32=params.accum_c_fp32,
            filter_e_grad=params.filter_e_grad,
            filter_c_grad=params.filter_c_grad,
            tile_max=tile_max,
            target_offset=vp.start if vp is not None else 0,
            counters=_tile_counters,
        )
        return de, dc, dbias, None


def linear_cross_entropy_apply(e, c, bias, params: CCEParams):
    """Reference: cce.py:238-256.  The slice after the autograd function makes autograd
    zero-pad the upstream gradients back to the full batch shape."""
    loss, lse = LinearCrossEntropyFunction.apply(e, c, bias, params)
    if params.shift != 0 and params.reduction == "none":
        loss = loss[..., params.shift :]
    if params.return_lse and params.shift != 0:
        assert lse is not None
        lse = lse[..., params.shift :]
    return loss, lse


def cce_linear_cross_entropy(
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
    vocab_parallel_options: Optional[VocabParallelOptions] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Reference: cce.py:261-319."""
    assert e.size()[0:-1] == targets.size()
    assert e.size(-1) == c.size(1)
    if not (torch.cuda.is_available() and torch.cuda.is_bf16_supported()):
        raise RuntimeError(
            "Cut Cross Entropy requires a bf16-capable GPU. "
            "Consider using torch_compile_linear_cross_entropy for scenarios where one is not available."
        )
    if vocab_parallel_options is not None:
        require_single_rank(vocab_parallel_options)

    batch_shape = targets.size()
    e = e.contiguous()
    targets = targets.contiguous()
    # The kernels stream 16-byte pieces of C's rows.  A classifier whose unit stride runs along the classes
    # (the transpose of a [D, V] matrix), or whose rows start off 16-byte boundaries although D would allow
    # them not to, takes the element-wise kernels, which are an order of magnitude slower than one packing
    # copy of C (0.3 ms for 1.2 GB); autograd carries the gradient back through the copy.
    per16 = 16 // c.element_size()
    if c.stride(1) != 1 or (c.size(1) % per16 == 0 and (c.stride(0) % per16 != 0 or c.data_ptr() % 16 != 0)):
        c = c.contiguous()

    shift = int(shift)
    valids = _build_flat_valids(targets, ignore_index, shift)

    e = e.flatten(0, -2)
    targets = targets.flatten()

    low = torch.get_autocast_gpu_dtype() if torch.is_autocast_enabled() else e.dtype
    params = CCEParams(
        targets,
        valids,
        softcap,
        reduction,
        _handle_eps(filter_eps, low),
        shift,
        batch_shape,
        accum_e_fp32,
        accum_c_fp32,
        filter_e_grad=filter_e_grad and filter_eps is not None,
        filter_c_grad=filter_c_grad and filter_eps is not None,
        vocab_parallel_options=vocab_parallel_options,
        return_lse=return_lse,
    )
    return linear_cross_entropy_apply(e, c, bias, params)
