"""Vocabulary sharding on one GPU: shard bounds and per-shard partial results.

``shard_forward`` / ``shard_backward`` expose what one vocab-parallel rank of the
reference computes before and after its exchange steps
(reference: cut_cross_entropy/cce.py:94-137 and :193-208), so that the shards of a
vocabulary can be run one after another on a single device and combined on the host.
"""

from typing import Optional, Tuple

import torch

from cut_cross_entropy.vocab_parallel.utils import VocabParallelOptions, partition_n_into_range

__all__ = [
    "VocabParallelOptions",
    "partition_n_into_range",
    "shard_forward",
    "shard_backward",
    "combine_shards",
]


def shard_forward(
    e: torch.Tensor,
    c_shard: torch.Tensor,
    targets: torch.Tensor,
    opts: VocabParallelOptions,
    bias_shard: Optional[torch.Tensor] = None,
    softcap: Optional[float] = None,
    valids: Optional[torch.Tensor] = None,
    shift: int = 0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(correct_logit[B], lse_shard[B])`` of the classes ``[opts.start, opts.stop)``: the
    log-sum-exp over the shard's classes, and the (soft-capped) logit of the target for the
    rows whose target lies in the shard, 0 for the others.  ``e`` is [N, D], ``targets`` [N]."""
    from cut_cross_entropy.cce_lse_forward import lse_forward
    from cut_cross_entropy.indexed_dot import indexed_neg_dot_forward_kernel

    assert c_shard.size(0) == opts.stop - opts.start
    lse, _, _ = lse_forward(e, c_shard, bias_shard, valids, softcap)
    neg = indexed_neg_dot_forward_kernel(
        e, c_shard, targets, bias=bias_shard, shift=shift, valids=valids, softcap=softcap,
        out_dtype=torch.float32, target_offset=opts.start,
    )
    return -neg, lse


def combine_shards(correct_logits, shard_lses) -> Tuple[torch.Tensor, torch.Tensor]:
    """Host-side stand-in for the reference's all-reduces (vocab_parallel/utils.py:47-65):
    returns ``(nll[B], lse[B])`` of the whole vocabulary."""
    lse = torch.logsumexp(torch.stack(list(shard_lses), 0), dim=0)
    correct = torch.stack(list(correct_logits), 0).sum(0)
    return lse - correct, lse


def shard_backward(
    e: torch.Tensor,
    c_shard: torch.Tensor,
    targets: torch.Tensor,
    opts: VocabParallelOptions,
    global_lse: torch.Tensor,
    d_out: torch.Tensor,
    d_lse: Optional[torch.Tensor] = None,
    bias_shard: Optional[torch.Tensor] = None,
    softcap: Optional[float] = None,
    valids: Optional[torch.Tensor] = None,
    shift: int = 0,
    grad_scale: float = 1.0,
    filter_eps: Optional[float] = None,
    accum_fp32: bool = True,
):
    """``(dE_partial, dC_shard, dBias_shard)`` of one shard given the LSE of the whole
    vocabulary; summing ``dE_partial`` over the shards gives dE."""
    from cut_cross_entropy.cce_backward import cce_backward_kernel
    from cut_cross_entropy.utils import TensorInfo

    info = TensorInfo(torch.float32 if accum_fp32 else e.dtype, True)
    return cce_backward_kernel(
        do=d_out, dlse=d_lse, e=e, e_info=info, c=c_shard, c_info=info,
        bias=bias_shard, bias_info=info if bias_shard is not None else None,
        lse=global_lse, valids=valids, softcap=softcap, filter_eps=filter_eps,
        targets=targets, shift=shift, grad_scale=grad_scale,
        accum_e_fp32=accum_fp32, accum_c_fp32=accum_fp32,
        target_offset=opts.start,
    )
