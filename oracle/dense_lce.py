"""CPU oracle for the linear-cross-entropy loss path.  TEST INFRASTRUCTURE ONLY.

This module is a dense (logits-materialising) restatement of the reference
algorithm.  It exists so that the HIP kernels can be checked against it; it is
never imported by the shipped package.  Only the test-suite, the smoke check
and the CPU-baseline leg of the benchmark may import it.

Every function cites the reference source it follows (paths are relative to the
upstream apple/ml-cross-entropy checkout).

How each function is pinned (see tests/test_oracle_*.py):

* ``compute_z_loss``            known-answer test of the reference
                                (tests/test_compute_z_loss.py:13-44)
* ``partition_n_into_range``    exact invariant test of the reference
                                (tests/test_vocab_parallel.py:153-165)
* ``build_flat_valids``         brute-force Python loops on small tensors
* ``handle_reduction_none``     brute-force scatter
* ``softcapping``               library ``tanh``; softcap -> inf reduces to identity
* ``dense_lse``                 ``scipy.special.logsumexp`` in float64
* ``dense_indexed_neg_dot``     explicit Python loops
* ``dense_linear_cross_entropy`` ``torch.nn.functional.cross_entropy`` on the
                                gathered rows (what the reference's own tests use
                                as ground truth, tests/test_cce_loss_forward.py:12-41)
* ``dense_grads``               autograd through the float64 dense formulation and
                                central finite differences
* ``vp_shard_partials``         logsumexp over shard LSEs == full LSE; sum of shard
                                correct logits == full correct logit

No function here is "parity unpinned".
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

IGNORE_INDEX = -100  # cut_cross_entropy/constants.py:2


# ---------------------------------------------------------------------------
# small helpers
# ---------------------------------------------------------------------------


def softcapping(logits: torch.Tensor, softcap: float) -> torch.Tensor:
    """tanh(x / softcap) * softcap  (cut_cross_entropy/utils.py:12-14)."""
    return torch.tanh(logits / softcap) * softcap


def handle_eps(filter_eps, dtype: torch.dtype):
    """"auto" -> finfo(dtype).eps / 32  (cut_cross_entropy/utils.py:17-25)."""
    if filter_eps is None:
        return None
    if isinstance(filter_eps, float):
        return filter_eps
    if filter_eps == "auto":
        return torch.finfo(dtype).eps / 32
    raise RuntimeError(f"Unknown eps {filter_eps=}")


def partition_n_into_range(n: int, rank: int, world_size: int) -> Tuple[int, int]:
    """Contiguous split of [0, n); the first n % world_size ranks get one more
    (cut_cross_entropy/vocab_parallel/utils.py:9-13)."""
    base, rem = divmod(n, world_size)
    start = rank * base + min(rank, rem)
    stop = start + base + (1 if rank < rem else 0)
    return start, stop


def build_flat_valids(
    targets: torch.Tensor, ignore_index: int, shift: int
) -> Optional[torch.Tensor]:
    """Flat row indices (into the flattened ``e``) of the rows that take part in
    the loss (cut_cross_entropy/utils.py:28-49).

    shift == 0: indices of ``targets.flatten() != ignore_index`` as int32, or
    ``None`` when nothing is ignored.
    shift > 0: row ``(b, t)`` takes part iff ``targets[b, t + shift] != ignore``;
    its flat index is ``b * T + t`` with ``T`` the unsliced length, and the
    result is always a tensor.  The matching target lives at ``index + shift``.
    """
    targets = targets.contiguous()
    if shift == 0:
        flat = targets.reshape(-1)
        keep = (flat != ignore_index).nonzero().reshape(-1).to(torch.int32)
        return None if keep.numel() == flat.numel() else keep

    T = targets.size(-1)
    lead = targets.reshape(-1, T)
    rows = []
    tt = torch.arange(T - shift, device=targets.device)
    for b in range(lead.size(0)):
        ok = lead[b, shift:] != ignore_index
        rows.append(b * T + tt[ok])
    if not rows:
        return torch.zeros((0,), dtype=torch.int32, device=targets.device)
    return torch.cat(rows).to(torch.int32)


def handle_reduction_none(
    batch_shape, valids: Optional[torch.Tensor], shift: int, loss: torch.Tensor
) -> torch.Tensor:
    """Scatter per-valid-row values back into the full batch shape, zeros at the
    ignored positions (cut_cross_entropy/utils.py:52-61)."""
    batch_shape = torch.Size(batch_shape)
    if valids is None:
        return loss.view(batch_shape)
    full = loss.new_zeros((batch_shape.numel(),))
    full[(valids.long() + shift)] = loss
    return full.view(batch_shape)


def compute_z_loss(
    lse: torch.Tensor,
    targets: Optional[torch.Tensor] = None,
    shift: int = 0,
    ignore_index: int = IGNORE_INDEX,
    reduction: str = "mean",
) -> torch.Tensor:
    """lse**2, zeroed at ignored tokens; "mean" averages over the valid tokens
    (cut_cross_entropy/utils.py:64-102)."""
    z = lse.pow(2)
    if targets is not None:
        shift = int(shift)
        if shift != 0:
            targets = targets[..., shift:]
        keep = targets != ignore_index
        z = torch.where(keep, z, torch.zeros((), dtype=z.dtype, device=z.device))
        if reduction == "mean":
            z = z * (z.numel() / keep.count_nonzero().to(z.dtype))
    if reduction == "mean":
        return z.mean()
    if reduction == "sum":
        return z.sum()
    if reduction == "none":
        return z
    raise ValueError(f"Invalid reduction: {reduction}")


# ---------------------------------------------------------------------------
# dense forward pieces
# ---------------------------------------------------------------------------


def _dense_logits(e, c, bias, softcap, compute_dtype):
    """e @ c.T (+ bias) (softcap) in ``compute_dtype``, then float
    (cut_cross_entropy/torch_compile.py:29-37)."""
    if compute_dtype is not None:
        e = e.to(compute_dtype)
        c = c.to(compute_dtype)
        bias = bias.to(compute_dtype) if bias is not None else None
    logits = e @ c.T
    if bias is not None:
        logits = logits + bias
    if softcap is not None:
        logits = softcapping(logits, softcap)
    return logits


def dense_lse(e, c, bias=None, softcap=None, compute_dtype=torch.float32) -> torch.Tensor:
    """logsumexp over the vocabulary of the (soft-capped) logits, in float32 or
    wider (what cut_cross_entropy/cce_lse_forward.py:170-237 returns; ground truth
    as in tests/test_cce_lse.py:11-20)."""
    logits = _dense_logits(e, c, bias, softcap, compute_dtype)
    if logits.dtype in (torch.float16, torch.bfloat16):
        logits = logits.float()
    return torch.logsumexp(logits, dim=-1)


def dense_indexed_neg_dot(e, c, inds, bias=None, softcap=None, compute_dtype=torch.float32):
    """-(e_i . c[inds_i]) - bias[inds_i], soft-capped
    (cut_cross_entropy/indexed_dot.py:101-158; ground truth as in
    tests/test_cce_indexed_dot.py:43-48)."""
    ee = e.to(compute_dtype)
    cc = c.to(compute_dtype)[inds]
    out = -(ee * cc).sum(-1)
    if bias is not None:
        out = out - bias.to(compute_dtype)[inds]
    if softcap is not None:
        out = softcapping(out, softcap)
    return out


def dense_linear_cross_entropy(
    e: torch.Tensor,
    c: torch.Tensor,
    targets: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    ignore_index: int = IGNORE_INDEX,
    softcap: Optional[float] = None,
    reduction: str = "mean",
    shift: int = 0,
    return_lse: bool = False,
    compute_dtype: Optional[torch.dtype] = None,
):
    """Dense restatement of ``torch_compile_linear_cross_entropy``
    (cut_cross_entropy/torch_compile.py:53-117): gather the valid rows, form the
    logits in the input (or ``compute_dtype``) precision, upcast, cross-entropy,
    then scatter ("none") and drop the first ``shift`` positions.

    Returns ``(loss, lse_or_None)``; both are differentiable w.r.t. e, c, bias.
    """
    assert e.size()[0:-1] == targets.size()
    assert e.size(-1) == c.size(1)
    batch_shape = targets.size()
    shift = int(shift)
    e = e.contiguous()
    targets = targets.contiguous()
    valids = build_flat_valids(targets, ignore_index, shift)

    e2 = e.flatten(0, -2)
    t1 = targets.flatten()
    if valids is not None:
        e2 = e2[valids.long()]
        t1 = t1[valids.long() + shift]

    logits = _dense_logits(e2, c, bias, softcap, compute_dtype)
    if logits.dtype in (torch.float16, torch.bfloat16):
        logits = logits.float()

    lse = torch.logsumexp(logits, dim=-1)
    if t1.numel() > 0:
        nll = lse - logits.gather(1, t1.view(-1, 1)).squeeze(1)
    else:
        nll = lse
    # equivalent to F.cross_entropy(logits, t1, reduction=...) once the ignored
    # rows are gathered away (torch_compile.py:78-80): checked in the tests.
    if reduction == "mean":
        loss = nll.mean()
    elif reduction == "sum":
        loss = nll.sum()
    elif reduction == "none":
        loss = handle_reduction_none(batch_shape, valids, shift, nll)
        if shift != 0:
            loss = loss[..., shift:]
    else:
        raise ValueError(f"Unknown reduction {reduction}")

    lse_out = None
    if return_lse:
        lse_out = handle_reduction_none(batch_shape, valids, shift, lse)
        if shift != 0:
            lse_out = lse_out[..., shift:]
    return loss, lse_out


# ---------------------------------------------------------------------------
# closed-form gradients (row-chunked so that large shapes fit in memory)
# ---------------------------------------------------------------------------


def dense_grads(
    e: torch.Tensor,  # [N, D]
    c: torch.Tensor,  # [V, D]
    targets: torch.Tensor,  # [N] int64 (full batch, flattened)
    valids: Optional[torch.Tensor],  # [B] int32 or None
    d_out: torch.Tensor,  # [N] per-row dLoss/dnll (already multiplied by grad_scale), or 0-dim
    d_lse: Optional[torch.Tensor] = None,  # [N] per-row dLoss/dlse
    bias: Optional[torch.Tensor] = None,
    softcap: Optional[float] = None,
    shift: int = 0,
    compute_dtype: torch.dtype = torch.float32,
    chunk: int = 2048,
):
    """Closed-form dE, dC, dBias of ``sum_i d_out_i * nll_i + d_lse_i * lse_i``.

    With z the raw logit, s = softcap(z), p = exp(s - lse_i), y = [v == t_i],
    g = d_out_i, h = d_lse_i:   dz = (p (g + h) - y g) (1 - (s / softcap)^2);
    dE[row_i] = sum_v dz C[v];  dC[v] = sum_i dz E[row_i];  dBias[v] = sum_i dz
    (the math of cut_cross_entropy/cce_backward.py:190-310 without filtering,
    rounding of dz, or locks).  Targets outside [0, V) never match a column.
    """
    N, D = e.shape
    V = c.shape[0]
    dev = e.device
    rows = torch.arange(N, device=dev) if valids is None else valids.long()
    B = rows.numel()
    cc = c.to(compute_dtype)
    bb = bias.to(compute_dtype) if bias is not None else None
    dE = torch.zeros((N, D), dtype=compute_dtype, device=dev)
    dC = torch.zeros((V, D), dtype=compute_dtype, device=dev)
    dB = torch.zeros((V,), dtype=compute_dtype, device=dev) if bias is not None else None
    for s0 in range(0, B, chunk):
        r = rows[s0 : s0 + chunk]
        ee = e[r].to(compute_dtype)
        z = ee @ cc.T
        if bb is not None:
            z = z + bb
        s = softcapping(z, softcap) if softcap is not None else z
        lse = torch.logsumexp(s, dim=-1, keepdim=True)
        p = torch.exp(s - lse)
        t = targets[r + shift]
        g = (d_out[r + shift] if d_out.ndim > 0 and d_out.numel() > 1 else d_out.reshape(())).to(
            compute_dtype
        )
        g = g.reshape(-1, 1) if g.ndim > 0 else g
        if d_lse is not None:
            h = d_lse[r + shift].to(compute_dtype).reshape(-1, 1)
            dz = p * (g + h)
        else:
            dz = p * g
        inb = (t >= 0) & (t < V)
        tt = torch.where(inb, t, torch.zeros_like(t))
        onehot_g = torch.zeros_like(dz)
        gv = g.expand(r.numel(), 1) if g.ndim > 0 else g.expand(r.numel()).reshape(-1, 1)
        onehot_g.scatter_(1, tt.view(-1, 1), torch.where(inb.view(-1, 1), gv, torch.zeros_like(gv)))
        dz = dz - onehot_g
        if softcap is not None:
            dz = dz * (1 - (s / softcap) ** 2)
        dE.index_add_(0, r, dz @ cc)
        dC += dz.T @ ee
        if dB is not None:
            dB += dz.sum(0)
    return dE, dC, dB


# ---------------------------------------------------------------------------
# vocab shard partials (no collective)
# ---------------------------------------------------------------------------


def vp_shard_partials(e, c_shard, targets, start, stop, bias_shard=None, softcap=None,
                      compute_dtype=torch.float32):
    """Per-shard (correct_logit, lse) over the vocab slice [start, stop)
    (cut_cross_entropy/vocab_parallel/vocab_parallel_torch_compile.py:64-92):
    rows whose target is outside the shard contribute a correct logit of 0."""
    logits = _dense_logits(e, c_shard, bias_shard, softcap, compute_dtype)
    if logits.dtype in (torch.float16, torch.bfloat16):
        logits = logits.float()
    lse = torch.logsumexp(logits, dim=-1)
    inside = (targets >= start) & (targets < stop)
    local = torch.where(inside, targets - start, torch.zeros_like(targets))
    picked = logits.gather(1, local.view(-1, 1)).squeeze(1)
    correct = torch.where(inside, picked, torch.zeros_like(picked))
    return correct, lse


def vp_combine(shard_correct, shard_lse):
    """Host-side stand-in for the two all-reduces
    (cut_cross_entropy/vocab_parallel/utils.py:47-65): lse = logsumexp over the
    shard LSEs, correct logit = sum over shards; nll = lse - correct."""
    lse = torch.logsumexp(torch.stack(shard_lse, 0), dim=0)
    correct = torch.stack(shard_correct, 0).sum(0)
    return lse - correct, lse
