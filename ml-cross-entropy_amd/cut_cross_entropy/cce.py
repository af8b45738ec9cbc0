"""Autograd node of the Cut Cross-Entropy loss on gfx950 (reference: cut_cross_entropy/cce.py).

forward    lse[i]  = logsumexp_v softcap(e[row_i] . c[v] + bias[v])      cce_lse_forward   (HIP)
           dot[i]  = -softcap(e[row_i] . c[t_i] + bias[t_i])            cce_indexed_neg_dot (HIP)
           nll     = lse + dot, then mean / sum / scatter to the batch shape
backward   dE, dC, dBias from recomputed logit tiles                    cce_backward / cce_backward_dz (HIP)

fp32 inputs go through ``fp32_path`` (three bf16 parts per value); everything else here is bookkeeping:
which rows count, where their targets sit, what the upstream gradients mean for each reduction.
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
from cut_cross_entropy.utils import TensorInfo, _build_flat_valids, _handle_eps, handle_reduction_none
from cut_cross_entropy.vocab_parallel.utils import VocabParallelOptions, require_single_rank

_REDUCTIONS = ("mean", "sum", "none")
_D_MULTIPLE = 128  # columns per stage of the fast backward kernels


@dataclass(frozen=True)
class CCEParams:
    """Everything about one call that is not a differentiable tensor (reference: cce.py:26-40)."""

    # which rows of the flattened e enter the loss and where their targets are
    targets: torch.Tensor
    valids: Optional[torch.Tensor]
    batch_shape: torch.Size
    shift: int
    # the loss itself
    softcap: Optional[float]
    reduction: str
    return_lse: bool
    # the backward
    filter_eps: Optional[float]
    filter_e_grad: bool
    filter_c_grad: bool
    accum_e_fp32: bool
    accum_c_fp32: bool
    vocab_parallel_options: Optional[VocabParallelOptions] = None

    @property
    def first_class(self) -> int:
        """Global index of the first class of ``c`` (non-zero for a vocabulary shard)."""
        vp = self.vocab_parallel_options
        return 0 if vp is None else vp.start

    def to_batch(self, per_row: torch.Tensor) -> torch.Tensor:
        """Per-valid-row values laid out in the batch shape, zeros where a target is ignored."""
        return handle_reduction_none(self.batch_shape, self.valids, self.shift, per_row)

    def reduce(self, nll: torch.Tensor) -> torch.Tensor:
        if self.reduction == "mean":
            return nll.mean()  # over the valid rows; NaN when there are none, like F.cross_entropy
        if self.reduction == "sum":
            return nll.sum()
        if self.reduction == "none":
            return self.to_batch(nll)
        raise ValueError(f"Unknown reduction {self.reduction}")

    def loss_grad_scale(self, n_valid: int) -> float:
        """Factor between the upstream gradient of the returned loss and that of a row's nll."""
        if self.reduction == "mean":
            return 1.0 / n_valid if n_valid > 0 else 0.0  # no valid row: zero gradients, no exception
        if self.reduction in ("sum", "none"):
            return 1.0
        raise ValueError(f"Unknown reduction {self.reduction}")


# uint64[4] device tensor that, while set, accumulates the backward's sub-tile counters (in the plane,
# recomputed, with a dE product, with a dC product); the benchmark reads the kept fractions from it.
_tile_counters: Optional[torch.Tensor] = None


def set_tile_counters(t: Optional[torch.Tensor]) -> None:
    global _tile_counters
    _tile_counters = t


def _autocast_dtype() -> Optional[torch.dtype]:
    """The GPU autocast dtype while an autocast region is active, else None."""
    if hasattr(torch, "get_autocast_dtype"):
        return torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else None
    return torch.get_autocast_gpu_dtype() if torch.is_autocast_enabled() else None


def _autocast_inputs(*tensors):
    """Inside an autocast region the inputs are taken to the autocast dtype by hand (custom_fwd does not
    cast when the function is entered with autocast on)."""
    low = _autocast_dtype()
    if low is None:
        return tensors
    return tuple(t if t is None else t.to(dtype=low) for t in tensors)


class LinearCrossEntropyFunction(torch.autograd.Function):
    """Reference: cce.py:48-235."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, e, c, bias, params: CCEParams):
        as_given = [None if t is None else TensorInfo(t.dtype, t.requires_grad) for t in (e, c, bias)]
        any_grad = any(info is not None and info.requires_grad for info in as_given)
        e, c, bias = _autocast_inputs(e, c, bias)

        is_fp32 = e.dtype == torch.float32
        tile_max = None
        if is_fp32:
            assert c.dtype == torch.float32, "e and c must have the same dtype"
            _hip.require_gpu_tensor("e", e)
            e = e.contiguous()
            with _hip.timed("forward_fp32", e.device):
                lse = fp32_path.fp32_lse(e, c, bias, params.valids, params.softcap)
            neg_dot = fp32_path.fp32_indexed_neg_dot(e, c, bias, params.targets, params.valids, params.shift,
                                                     params.softcap, params.first_class)
        else:
            # the per-sub-tile maxima let the backward drop sub-tiles unseen; only a filtered backward reads them
            lse, _, tile_max = lse_forward(e, c, bias, params.valids, params.softcap,
                                           want_tile_max=any_grad and params.filter_eps is not None)
            neg_dot = indexed_neg_dot_forward_kernel(e, c, params.targets, bias, params.shift, params.valids,
                                                     params.softcap, lse.dtype, params.first_class)
        nll = neg_dot.add_(lse)

        ctx.save_for_backward(e, c, bias, lse, params.targets, params.valids, tile_max)
        ctx.params, ctx.as_given, ctx.is_fp32 = params, as_given, is_fp32
        return params.reduce(nll), (params.to_batch(lse) if params.return_lse else None)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, d_loss, d_lse):
        e, c, bias, lse, targets, valids, tile_max = ctx.saved_tensors
        params: CCEParams = ctx.params
        e_info, c_info, bias_info = ctx.as_given

        scale = params.loss_grad_scale(lse.numel())
        # "none": one upstream value per batch position, read by the kernels at row + shift; else one scalar
        d_loss = d_loss.reshape(-1)
        if d_lse is not None:
            d_lse = d_lse.reshape(-1)

        if ctx.is_fp32:
            with _hip.timed("backward_fp32", e.device):
                de, dc, dbias = fp32_path.fp32_backward(
                    e, c, bias, lse, d_loss, d_lse, valids, targets, params.shift, params.first_class,
                    params.softcap, scale, e_info.requires_grad, c_info.requires_grad,
                    bias_info is not None and bias_info.requires_grad)
            if dbias is not None:
                dbias = dbias.to(bias_info.dtype)
        else:
            de, dc, dbias = cce_backward_kernel(
                d_loss, d_lse, e, e_info, c, c_info, bias, bias_info, lse, valids, params.softcap, params.filter_eps,
                targets=targets, shift=params.shift, grad_scale=scale,
                accum_e_fp32=params.accum_e_fp32, accum_c_fp32=params.accum_c_fp32,
                filter_e_grad=params.filter_e_grad, filter_c_grad=params.filter_c_grad,
                tile_max=tile_max, target_offset=params.first_class, counters=_tile_counters)
        return de, dc, dbias, None


def linear_cross_entropy_apply(e, c, bias, params: CCEParams):
    """Runs the node and cuts the first ``shift`` positions off batch-shaped outputs (reference:
    cce.py:238-256); slicing outside the node lets autograd pad the upstream gradients back with zeros."""
    loss, lse = LinearCrossEntropyFunction.apply(e, c, bias, params)
    if params.shift:
        if params.reduction == "none":
            loss = loss[..., params.shift:]
        if lse is not None:
            lse = lse[..., params.shift:]
    return loss, lse


def _streamable(c: torch.Tensor) -> bool:
    """Whether the kernels can stream 16-byte pieces of c's rows where its width allows them to."""
    per16 = 16 // c.element_size()
    if c.stride(1) != 1:
        return False
    if c.size(1) % per16 != 0:
        return True  # the element-wise kernels run whatever the layout
    return c.stride(0) % per16 == 0 and c.data_ptr() % 16 == 0


@torch.compiler.disable  # ctypes launches and a host read of the valid rows: a graph break for torch.compile, not a trace
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
    shift = int(shift)

    # A classifier whose unit stride runs along the classes (the transpose of a [D, V] matrix), or whose rows
    # start off 16-byte boundaries although D would allow otherwise, would take the element-wise kernels: an
    # order of magnitude slower than one packing copy (0.3 ms for 1.2 GB); autograd carries dC back through it.
    if not _streamable(c):
        c = c.contiguous()
    # The direct-to-LDS kernels stream whole 128-column stages.  A width that is no multiple of 128 (D = 72,
    # 1000, 123, ...) would take the register-staged generic kernels, several times slower; zero columns change
    # no logit, so e and c are padded once instead (one copy each; autograd cuts the gradients back).
    compute_dtype = _autocast_dtype() or e.dtype
    if compute_dtype != torch.float32 and e.size(-1) % _D_MULTIPLE != 0:
        pad = _D_MULTIPLE - e.size(-1) % _D_MULTIPLE
        e = torch.nn.functional.pad(e, (0, pad))
        c = torch.nn.functional.pad(c, (0, pad))
    targets = targets.contiguous()
    filtering = filter_eps is not None
    params = CCEParams(
        targets=targets.flatten(),
        valids=_build_flat_valids(targets, ignore_index, shift),
        batch_shape=targets.size(),
        shift=shift,
        softcap=softcap,
        reduction=reduction,
        return_lse=return_lse,
        filter_eps=_handle_eps(filter_eps, compute_dtype),
        filter_e_grad=filtering and filter_e_grad,
        filter_c_grad=filtering and filter_c_grad,
        accum_e_fp32=accum_e_fp32,
        accum_c_fp32=accum_c_fp32,
        vocab_parallel_options=vocab_parallel_options,
    )
    if reduction not in _REDUCTIONS:
        raise ValueError(f"Unknown reduction {reduction}")
    return linear_cross_entropy_apply(e.contiguous().flatten(0, -2), c, bias, params)
