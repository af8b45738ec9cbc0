"""Shared input builders and the accuracy criterion of the parity tests."""

import torch

IGNORE_INDEX = -100


def make_inputs(N, V, D, dtype=torch.bfloat16, seed=0, invalid_frac=0.0, bias=False, planted=True,
                c_std=1.0):
    """Inputs in the style of the reference tests (tests/test_cce_loss_backward.py:110-133):
    e ~ N(0,1)/sqrt(D), c ~ N(0,1), the first rows of c copied from e so that some logits are
    large, uniform targets, optionally a fraction set to ignore_index.  Generated on the CPU
    from a seeded generator and rounded to ``dtype`` so CPU oracle and GPU kernels see the
    same values."""
    g = torch.Generator().manual_seed(seed)
    e = (torch.randn((N, D), generator=g) / (D**0.5)).to(dtype)
    c = (torch.randn((V, D), generator=g) * c_std).to(dtype)
    if planted:
        k = min(N, V) // 2
        c[:k] = e[:k]
    targets = torch.randint(0, V, (N,), generator=g)
    if invalid_frac > 0:
        idx = torch.randperm(N, generator=g)[: int(invalid_frac * N)]
        targets[idx] = IGNORE_INDEX
    b = (torch.randn((V,), generator=g) * 0.02).to(dtype) if bias else None
    return e, c, targets, b


def assert_no_worse(gt, ref, got, tol, what="", rel=0.0):
    """The reference's criterion (tests/test_cce_loss_forward.py:103-108): elementwise
    |gt - got| <= |gt - ref| + tol, gt = fp32/fp64 dense result, ref = dense result in the
    low-precision input type.  ``rel`` adds rel * |gt| to the allowance (gradients whose
    scale is not 1/N: the kernel rounds dz to the 16-bit input type before the dE / dC
    products, as the reference does, cce_backward.py:256)."""
    gt = gt.double().cpu().flatten()
    ref = ref.double().cpu().flatten()
    got = got.double().cpu().flatten()
    assert gt.shape == got.shape, f"{what}: shape {got.shape} vs {gt.shape}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    excess = ((gt - got).abs() - (gt - ref).abs() - tol - rel * gt.abs()).clamp_min(0)
    if (excess > 0).any():
        i = int(excess.argmax())
        raise AssertionError(
            f"{what}: excess error {excess.max().item():.3e} at {i}: got {got[i].item():.6e}, "
            f"gt {gt[i].item():.6e}, ref {ref[i].item():.6e}"
        )


def autograd_grads(e, c, targets, valids, d_out, d_lse, bias, softcap, shift, compute_dtype):
    """Gradients of sum_i d_out_i * nll_i + d_lse_i * lse_i by autograd through the dense
    formulation with the logits formed in ``compute_dtype`` and the soft-max in fp32 or wider:
    with a 16-bit ``compute_dtype`` this is the "naive low-precision implementation" the
    reference's tests measure against (tests/test_cce_loss_backward.py:12-76)."""
    from oracle import dense_lce

    N = e.shape[0]
    rows = torch.arange(N) if valids is None else valids.long()
    el = e.detach().to(compute_dtype).requires_grad_(True)
    cl = c.detach().to(compute_dtype).requires_grad_(True)
    bl = bias.detach().to(compute_dtype).requires_grad_(True) if bias is not None else None
    logits = dense_lce._dense_logits(el[rows], cl, bl, softcap, None)
    wide = logits.float() if logits.dtype in (torch.float16, torch.bfloat16) else logits
    lse = torch.logsumexp(wide, -1)
    t = targets[rows + shift]
    inb = (t >= 0) & (t < c.shape[0])
    tt = torch.where(inb, t, torch.zeros_like(t))
    picked = torch.where(inb, wide.gather(1, tt.view(-1, 1)).squeeze(1), torch.zeros_like(lse))
    nll = lse - picked
    g = d_out[rows + shift] if d_out.numel() > 1 else d_out.reshape(())
    total = (nll * g.to(nll.dtype)).sum()
    if d_lse is not None:
        total = total + (lse * d_lse[rows + shift].to(lse.dtype)).sum()
    total.backward()
    return el.grad, cl.grad, (bl.grad if bl is not None else None)
