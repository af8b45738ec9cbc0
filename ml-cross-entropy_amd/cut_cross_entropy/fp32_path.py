"""fp32 inputs on matrix cores that multiply 16-bit numbers.

gfx950 has no fast fp32 matrix path (the reference leans on Triton's tf32x3 / ieee dot for fp32
inputs, cce_lse_forward.py:81, constants via tl_utils).  An fp32 value is therefore split into three
bfloat16 parts, x = hi + mid + lo (8 + 8 + 8 significant bits), and the product of two such sums is
taken as the six leading terms

    hi*hi + hi*mid + mid*hi + mid*mid + hi*lo + lo*hi          (what is left is below 2^-24 relative)

which is ONE 16-bit contraction over a six times longer reduction axis: E' = [hi hi mid mid hi lo] and
C' = [hi mid hi mid lo hi] side by side along D.  The unchanged bf16 kernels then produce logits of fp32
accuracy (their accumulators are fp32).  A bias rides along as three more columns (ones in E', the
three parts of the bias in C').  The vocabulary is walked in chunks so that the widened copy of the
classifier stays small; chunk log-sum-exps are merged with logaddexp.

Backward: the gradient filter threshold of fp32 is far below anything a soft-max produces, so the
backward is the unfiltered one: the dz kernel runs on the widened matrices and writes the dz of a vocabulary
chunk as fp32; dz, the classifier chunk and the rows of e are split into the same three parts, and the two
products dE += dz . C and dC = dz^T . E are summed over the same cross terms, one call of the library's 16-bit
product kernels per term (``cce_backward_products``: fp32 accumulators, dE and dC added to in fp32).  No copy
of an operand is widened for this: a term pairs part i of dz with part j of C and of E as they lie.

``torch.set_float32_matmul_precision``: "highest" (the default) takes the six terms above; with "high" or
"medium" the caller has asked for fast fp32 products (the reference then lets Triton use tf32, 10 mantissa
bits, cce_lse_forward.py:129-131) and logits and gradient products are formed from the three leading terms
hi*hi + hi*mid + mid*hi (16 bits), half the work.
"""

from typing import Optional, Tuple

import torch

from cut_cross_entropy import _hip
from cut_cross_entropy.cce_lse_forward import lse_forward

_WIDE_C_BYTES = 1 << 29   # widened classifier chunk
_DZ_ELEMS = 1 << 25       # fp32 dz chunk (128 MB)


def split3(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    hi = x.to(torch.bfloat16)
    r = x - hi.to(torch.float32)
    mid = r.to(torch.bfloat16)
    lo = (r - mid.to(torch.float32)).to(torch.bfloat16)
    return hi, mid, lo


def n_terms() -> int:
    """Cross terms per product: all six under "highest" float32 matmul precision, the leading three otherwise."""
    return 6 if torch.get_float32_matmul_precision() == "highest" else 3


# which part (0 hi, 1 mid, 2 lo) of e and of c meets in term k; the first three are the 16-bit product
_E_PARTS = (0, 0, 1, 1, 0, 2)
_C_PARTS = (0, 1, 0, 1, 2, 0)


def _padded_width(d: int, has_bias: bool, terms: int) -> int:
    w = terms * d + (3 if has_bias else 0)
    return (w + 63) // 64 * 64


def widen_e(e: torch.Tensor, has_bias: bool, terms: int = 6) -> torch.Tensor:
    """[N, D] fp32 -> [N, Dp] bf16 = [hi hi mid (mid hi lo) (1 1 1) 0 ...]."""
    n, d = e.shape
    parts = split3(e)
    out = torch.zeros((n, _padded_width(d, has_bias, terms)), dtype=torch.bfloat16, device=e.device)
    for k in range(terms):
        out[:, k * d : (k + 1) * d] = parts[_E_PARTS[k]]
    if has_bias:
        out[:, terms * d : terms * d + 3] = 1.0
    return out


def widen_c(c: torch.Tensor, bias: Optional[torch.Tensor], terms: int = 6) -> torch.Tensor:
    """[V, D] fp32 (+ [V] bias) -> [V, Dp] bf16 = [hi mid hi (mid lo hi) (b_hi b_mid b_lo) 0 ...]."""
    v, d = c.shape
    parts = split3(c)
    out = torch.zeros((v, _padded_width(d, bias is not None, terms)), dtype=torch.bfloat16, device=c.device)
    for k in range(terms):
        out[:, k * d : (k + 1) * d] = parts[_C_PARTS[k]]
    if bias is not None:
        for k, part in enumerate(split3(bias.to(torch.float32))):
            out[:, terms * d + k] = part
    return out


def _chunk(v: int, per_class_bytes: int, budget: int) -> int:
    return max(256, min(v, (budget // max(per_class_bytes, 1)) // 256 * 256))


def fp32_lse(e, c, bias, valids, softcap) -> torch.Tensor:
    """Log-sum-exp of the valid rows over the whole vocabulary, fp32 accurate."""
    terms = n_terms()
    e6 = widen_e(e, bias is not None, terms)
    n_valid = valids.numel() if valids is not None else e.size(0)
    lse = torch.full((n_valid,), float("-inf"), dtype=torch.float32, device=e.device)
    vc = _chunk(c.size(0), e6.size(1) * 2, _WIDE_C_BYTES)
    for v0 in range(0, c.size(0), vc):
        c6 = widen_c(c[v0 : v0 + vc], bias[v0 : v0 + vc] if bias is not None else None, terms)
        part, _, _ = lse_forward(e6, c6, None, valids, softcap)
        lse = torch.logaddexp(lse, part)
    return lse


def fp32_indexed_neg_dot(e, c, bias, targets, valids, shift, softcap, target_offset) -> torch.Tensor:
    """-(soft-capped logit of the target) per valid row, 0 where the target is not a class of this
    shard (the semantics of the indexed-dot kernel).  O(rows x D) work: plain fp32 arithmetic."""
    n = e.size(0)
    rows = valids.to(torch.int64) if valids is not None else torch.arange(n, device=e.device)
    tpos = rows + int(shift)
    ok = tpos < n
    t = torch.where(ok, targets[tpos.clamp_max(n - 1)] - int(target_offset), torch.full_like(tpos, -1))
    ok = ok & (t >= 0) & (t < c.size(0))
    tc = t.clamp(0, c.size(0) - 1)
    logit = (e[rows] * c[tc]).sum(dim=1)
    if bias is not None:
        logit = logit + bias[tc].to(torch.float32)
    if softcap is not None:
        logit = torch.tanh(logit / softcap) * softcap
    return torch.where(ok, -logit, torch.zeros_like(logit))


def _pad_cols(x: torch.Tensor, width: int) -> torch.Tensor:
    return x if x.size(1) == width else torch.nn.functional.pad(x, (0, width - x.size(1)))


def fp32_backward(e, c, bias, lse, do, dlse, valids, targets, shift, target_offset, softcap, grad_scale,
                  want_de, want_dc, want_dbias):
    """(dE, dC, dBias) in fp32: dz of a vocabulary chunk from the HIP kernel (fp32 output), then the two
    products as sums of 16-bit cross terms on the library's product kernels."""
    lib = _hip.load()
    dev = e.device
    n, d = e.shape
    v = c.size(0)
    rows = valids.to(torch.int64) if valids is not None else None
    n_valid = rows.numel() if rows is not None else n
    de = torch.zeros_like(e) if want_de else None
    dc = torch.zeros_like(c) if want_dc else None
    dbias = torch.zeros((v,), dtype=torch.float32, device=dev) if want_dbias else None
    if n_valid == 0 or not (want_de or want_dc or want_dbias):
        return de, dc, dbias
    terms = n_terms()
    bf16 = _hip.DTYPE_CODES[torch.bfloat16]
    e6 = widen_e(e, bias is not None, terms)
    d8 = (d + 7) // 8 * 8  # the product kernels move 16-byte pieces
    e_parts = None
    if want_dc:
        e_rows = e if rows is None else e.index_select(0, rows)
        e_parts = [_pad_cols(part, d8).contiguous() for part in split3(e_rows)]
    de_acc = torch.zeros((n_valid, d8), dtype=torch.float32, device=dev) if want_de else None
    vc = min(_chunk(v, e6.size(1) * 2, _WIDE_C_BYTES), _chunk(v, n_valid * 4, _DZ_ELEMS * 4))
    ldz_full = (min(vc, v) + 63) // 64 * 64
    # fp32 dz of a chunk; its padding columns are never written by the kernel and have to read as zeros
    dz_buf = torch.zeros((n_valid * ldz_full,), dtype=torch.float32, device=dev)
    dc_direct = dc is not None and d8 == d and dc.is_contiguous()
    dc_tmp = None if (dc is None or dc_direct) else torch.empty((min(vc, v), d8), dtype=torch.float32, device=dev)
    do = do.to(torch.float32).contiguous().view(-1)
    dlse = dlse.to(torch.float32).contiguous().view(-1) if dlse is not None else None
    targets = targets.to(torch.int64).contiguous()
    stream = _hip.current_stream_ptr(dev)
    for v0 in range(0, v, vc):
        m = min(vc, v - v0)
        ldz = (m + 63) // 64 * 64
        if ldz != ldz_full:
            dz_buf.zero_()  # the last, shorter chunk lays the buffer out anew
        dz = dz_buf[: n_valid * ldz].view(n_valid, ldz)
        c_chunk = c[v0 : v0 + m]
        c6 = widen_c(c_chunk, bias[v0 : v0 + m] if bias is not None else None, terms)
        with torch.cuda.device(dev):
            status = lib.cce_backward_dz(
                e6.data_ptr(), c6.data_ptr(), None,
                lse.data_ptr(), do.data_ptr(), 1 if do.numel() == 1 else 0, _hip.ptr(dlse),
                _hip.ptr(valids), targets.data_ptr(),
                dz.data_ptr(), ldz, 1,
                n, n_valid, m, e6.size(1),
                e6.stride(0), c6.stride(0), c6.stride(1),
                float(grad_scale), int(shift), int(target_offset) + v0,
                float(softcap) if softcap is not None else 0.0, bf16, stream,
            )
        _hip.check(status, "cce_backward_dz")
        del c6
        if dbias is not None:
            dbias[v0 : v0 + m] = dz[:, :m].sum(dim=0)
        if de_acc is None and dc is None:
            continue
        dz_parts = split3(dz)
        c_parts = [_pad_cols(part, d8).contiguous() for part in split3(c_chunk)] if de_acc is not None else None
        dc_out = None
        if dc is not None:
            dc_out = dc[v0 : v0 + m] if dc_direct else dc_tmp[:m]
        for k in range(terms):
            a, b = dz_parts[_E_PARTS[k]], _C_PARTS[k]
            with torch.cuda.device(dev):
                status = lib.cce_backward_products(
                    a.data_ptr(), ldz,
                    c_parts[b].data_ptr() if c_parts is not None else None, d8,
                    e_parts[b].data_ptr() if e_parts is not None else None, d8, None,
                    _hip.ptr(de_acc), d8, _hip.ptr(dc_out), d8, 1 if k > 0 else 0,
                    n_valid, m, d8, bf16, stream,
                )
            _hip.check(status, "cce_backward_products")
        if dc is not None and not dc_direct:
            dc[v0 : v0 + m] = dc_tmp[:m, :d]
    if de is not None:
        if rows is None:
            de.copy_(de_acc[:, :d])
        else:
            de.index_copy_(0, rows, de_acc[:, :d].contiguous())
    return de, dc, dbias
