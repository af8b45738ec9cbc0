"""Launcher of the fused backward kernel
(reference: cut_cross_entropy/cce_backward.py:346-521)."""

import threading
from typing import Optional, Tuple

import torch

from cut_cross_entropy import _hip
from cut_cross_entropy.cce_utils import filter_eps_or_none
from cut_cross_entropy.utils import TensorInfo


# Upper bound of the dz chunk buffer of the unfiltered backward (bytes).  The chunk is [B, vc] in the input type
# with vc a multiple of 256 classes, at most 16384; the library picks the vc that fits and fills the 256 compute
# units most evenly.  A smaller buffer means more, smaller chunks: less memory, more launches and more passes over
# the dE accumulator (measured, backward of E [15356, 4096] x C [128256, 4096]: 44.1 ms with 128 MB, 40.4 with
# 256; E [8192, 2048] x C [256000, 2048]: 21.5 / 21.5; E [8192, 2304] x C [256000, 2304]: 24.4 / 24.0; with 32 MB
# the last one takes 29.7).  On top of it comes, when dE is wanted in a 16-bit type, a [B, D] 16-bit
# compensation buffer (dE is summed over the chunks as a pair of 16-bit numbers).
DENSE_DZ_BYTES = 256 << 20

# ... but never so small that a chunk holds fewer classes than this (a block fewer rows, where the library walks by
# blocks of rows: 16-bit gradients and at least twice as many rows as classes): the tiles of the gradient that is
# carried between the launches then have a short reduction, their fetch and read-modify-write weigh as much as their
# products, and that gradient is passed over once per launch.  The buffer then grows with the problem like its
# operands do (E [32768, 4096] x C [128256, 4096], by classes: 256 MB hold 4096 classes; E [65536, 3584] x
# C [19008, 3584], by rows: 256 MB hold 6912 rows, 22.6 ms, against 27.9 ms with 55 MB).
DENSE_DZ_MIN_CLASSES = 4096


def _dz_budget(lib, B: int, V: int, D: int, de_16bit: bool) -> int:
    return max(int(DENSE_DZ_BYTES),
               lib.cce_backward_dense_dz_bytes(B, V, D, 1 if de_16bit else 0, int(DENSE_DZ_MIN_CLASSES)))

# With the gradient filter on, the ownership kernels pay per surviving sub-tile and the dense path pays for
# the whole plane once.  Measured on MI355X the two cross where 0.177 of the 32 x 32 cells of the forward
# statistic can hold a probability above filter_eps for E [8192, 2304] x C [256000, 2304], and at 0.083 for
# E [16384, 4096] x C [128256, 4096], where a workgroup of the ownership kernels covers D in two slices and
# recomputes its logits for each.  Above DENSE_WHEN_FLAGGED_ABOVE / slices a FILTERED backward runs unfiltered; an
# unfiltered gradient is the exact one, so nothing is lost.  None switches the test off.
#
# The fraction is measured on the device (cce_count_flagged_cells over the forward's statistic) and the choice is
# a function of the data alone, the same on every run: every filtered backward enqueues the count of ITS cells and
# an asynchronous copy of it to pinned host memory; the FIRST backward of a (device, V, D, dtype) waits for its own
# count (once per shape and process, as the reference's first call waits for its autotuner), every later one uses
# the count of the backward before it, which has long arrived (a soft-max distribution moves slowly, so a decision
# that lags one step is as good).  Identical inputs therefore take the same path, and give the same bits, on the
# first call and on the tenth.  While a HIP graph is being captured nothing is measured or read: the capture
# takes the path of the last backward of that shape outside a capture (the ownership kernels if there was none),
# and the graph replays that path.  FILTERED_BACKWARD_PATH pins the choice: "sparse" or "dense" instead of "auto".
DENSE_WHEN_FLAGGED_ABOVE = 0.17
FILTERED_BACKWARD_PATH = "auto"
# A filtered backward that changes to the unfiltered path BY ITSELF may take at most
#     max(DENSE_WORKSPACE_LIMIT_BYTES, DENSE_WORKSPACE_LIMIT_OPERANDS x (bytes of E + bytes of C))
# of workspace (the dz buffer, plus the 16-bit compensation buffer of the gradient that is carried between launches:
# [B, D] for dE, or [V, D] for dC where rows outnumber classes two to one): the ownership kernels need well
# under 16 MB, and a caller who picked a filtered preset did not ask for more.  The defaults, 256 MB and 1.0, say:
# never more than the operands the caller already holds take themselves, and 256 MB where they are smaller (the
# second term matters when rows are many: at E [65536, 3584] x C [19008, 3584] the compensation buffer alone is
# 448 MB and the operands are 578 MB; the ownership kernels take 167 ms there, the unfiltered path 22 - 30).  The dz chunk
# shrinks to fit (more, smaller chunks: slower); if no plan with chunks of AUTO_DENSE_MIN_CLASSES classes fits, the
# backward stays on the ownership kernels.  DENSE_WORKSPACE_LIMIT_BYTES = None: no limit;
# DENSE_WORKSPACE_LIMIT_OPERANDS = 0: the byte limit alone.  The presets that ask for unfiltered gradients
# (cce_exact, cce_kahan_full_*) are not bound by either: their dz chunk is DENSE_DZ_BYTES (the reference's own
# unfiltered presets take fp32 copies of dE and dC, 2.3 GB at E [8192, 2304] x C [256000, 2304]).
DENSE_WORKSPACE_LIMIT_BYTES: Optional[int] = 256 << 20
DENSE_WORKSPACE_LIMIT_OPERANDS: float = 1.0
AUTO_DENSE_MIN_CLASSES = 1024
_OWNERSHIP_SLICE_COLS = 2304  # columns of D one ownership workgroup accumulates


class _FlaggedMonitor:
    """Fraction of flagged cells of the latest backward of one (device, V, D, dtype), and the path it chose."""

    def __init__(self, device: torch.device):
        self.counter = torch.zeros((1,), dtype=torch.int64, device=device)
        self.host = torch.zeros((1,), dtype=torch.int64, pin_memory=True)
        self.event = torch.cuda.Event()
        self.pending_cells = 0   # cells of the measurement in flight (0: none)
        self.fraction: Optional[float] = None
        self.dense: bool = False  # the last choice made outside a capture

    def collect(self) -> None:
        """Takes in the measurement in flight, waiting for it if it has not arrived."""
        if self.pending_cells:
            if not self.event.query():
                self.event.synchronize()
            self.fraction = int(self.host[0]) / self.pending_cells  # pinned host memory: a plain read
            self.pending_cells = 0

    def measure(self, lib, tile_max, lse, B: int, V: int, filter_eps: float, dev: torch.device) -> None:
        self.counter.zero_()
        with torch.cuda.device(dev):
            status = lib.cce_count_flagged_cells(tile_max.data_ptr(), lse.data_ptr(), B, V, float(filter_eps),
                                                 self.counter.data_ptr(), _hip.current_stream_ptr(dev))
        _hip.check(status, "cce_count_flagged_cells")
        self.host.copy_(self.counter, non_blocking=True)
        self.event.record(torch.cuda.current_stream(dev))
        self.pending_cells = lib.cce_tile_stat_elems(B, V)


_monitors: dict = {}
_monitors_lock = threading.Lock()


def reset_backward_path_memory() -> None:
    """Forgets every measured fraction: the next filtered backward of each shape waits for its own count again."""
    with _monitors_lock:
        _monitors.clear()


def _auto_dense_dz_budget(lib, B: int, V: int, D: int, de_16bit: bool, operand_bytes: int) -> Optional[int]:
    """dz chunk bytes a filtered backward may use when it changes to the unfiltered path by itself, or None when
    the workspace limit leaves no room for chunks of a useful size."""
    budget = _dz_budget(lib, B, V, D, de_16bit)
    if DENSE_WORKSPACE_LIMIT_BYTES is None:
        return budget
    limit = max(int(DENSE_WORKSPACE_LIMIT_BYTES), int(DENSE_WORKSPACE_LIMIT_OPERANDS * operand_bytes))
    # what the unfiltered backward keeps for the whole call (the compensation term of the gradient it carries from
    # launch to launch: [B, D], or [V, D] where it walks by blocks of rows)
    fixed = lib.cce_backward_dense_fixed_bytes(B, V, D, 1 if de_16bit else 0)
    # dz buffers of fewer than AUTO_DENSE_MIN_CLASSES classes per chunk (rows per block) are not worth having: every
    # launch passes over all of the carried gradient, and its products reduce over a handful of stages (measured,
    # backward of E [15356, 4096] x C [128256, 4096]: 226 ms with 256 classes per chunk, 45 ms with 2048, 39 ms with
    # 8192, against 168 ms on the ownership kernels).
    room = limit - fixed
    if room < lib.cce_backward_dense_dz_bytes(B, V, D, 1 if de_16bit else 0, int(AUTO_DENSE_MIN_CLASSES)):
        return None
    return min(budget, room)


def _filtered_backward_runs_dense(lib, tile_max, lse, B: int, V: int, D: int, filter_eps: float, dtype, dev) -> bool:
    """The dense / sparse choice of a filtered backward."""
    if FILTERED_BACKWARD_PATH != "auto":
        return FILTERED_BACKWARD_PATH == "dense"
    if DENSE_WHEN_FLAGGED_ABOVE is None:
        return False
    key = (dev.index, V, D, dtype)
    capturing = torch.cuda.is_current_stream_capturing()
    with _monitors_lock:
        mon = _monitors.get(key)
        if capturing:
            # nothing may be allocated, measured or waited for inside a capture
            return mon.dense if mon is not None else False
        if mon is None:
            mon = _monitors[key] = _FlaggedMonitor(dev)
        first = mon.fraction is None and not mon.pending_cells
        if first:
            mon.measure(lib, tile_max, lse, B, V, filter_eps, dev)  # this backward's own cells ...
        mon.collect()                                              # ... or those of the backward before
        fraction = mon.fraction
        mon.measure(lib, tile_max, lse, B, V, filter_eps, dev)      # for the next backward of this shape
        mon.dense = fraction is not None and fraction > DENSE_WHEN_FLAGGED_ABOVE / -(-D // _OWNERSHIP_SLICE_COLS)
        return mon.dense


def _dense_layout_ok(e, c) -> bool:
    """Whether the layout suits the direct-to-LDS kernels of the unfiltered backward (cce_backward_dense: dz chunks
    and the two products as MFMA kernels)."""
    return (
        e.size(1) % 64 == 0
        and e.stride(0) % 8 == 0
        and c.stride(1) == 1
        and c.stride(0) % 8 == 0
        and e.data_ptr() % 16 == 0
        and c.data_ptr() % 16 == 0
    )


def _dense_backward(lib, code, dev, e, c, bias, lse, do, dlse, valids, targets, de, dc, dbias, B, grad_scale,
                    shift, target_offset, softcap, dz_budget):
    """dE, dC, dBias of the unfiltered backward: one call into the library, which walks the vocabulary in
    chunks (dz of the chunk -> workspace, then the two products as hand-written MFMA kernels; reference:
    cce_backward.py:170-302, there one kernel with atomics).  The workspace -- the dz chunk, plus a 16-bit
    [B, D] compensation term when dE is accumulated in the 16-bit input type -- is a torch allocation, so the
    allocator's peak statistic sees it."""
    V, D = c.size(0), e.size(1)
    de_in_ws = de is not None and de.dtype != torch.float32
    ws_bytes = lib.cce_backward_dense_workspace_bytes(B, V, D, 1 if de_in_ws else 0, int(dz_budget))
    workspace = torch.empty((ws_bytes + 256,), dtype=torch.uint8, device=dev)
    ws_ptr = (workspace.data_ptr() + 255) // 256 * 256
    with torch.cuda.device(dev), _hip.timed("backward_dense", dev):
        status = lib.cce_backward_dense(
            e.data_ptr(), c.data_ptr(), _hip.ptr(bias),
            lse.data_ptr(), do.data_ptr(), 1 if do.numel() == 1 else 0, _hip.ptr(dlse),
            _hip.ptr(valids), targets.data_ptr(),
            _hip.ptr(de), _hip.ptr(dc), _hip.ptr(dbias),
            ws_ptr, ws_bytes,
            e.size(0), B, V, D,
            e.stride(0), c.stride(0), c.stride(1),
            float(grad_scale), 1 if (de is not None and de.dtype == torch.float32) else 0,
            1 if (dc is not None and dc.dtype == torch.float32) else 0,
            int(shift), int(target_offset),
            float(softcap) if softcap is not None else 0.0, code, _hip.current_stream_ptr(dev),
        )
    _hip.check(status, "cce_backward_dense")


def cce_backward_kernel(
    do: torch.Tensor,
    dlse: Optional[torch.Tensor],
    e: torch.Tensor,
    e_info: TensorInfo,
    c: torch.Tensor,
    c_info: TensorInfo,
    bias: Optional[torch.Tensor],
    bias_info: Optional[TensorInfo],
    lse: torch.Tensor,
    valids: Optional[torch.Tensor],
    softcap: Optional[float],
    filter_eps: Optional[float],
    targets: Optional[torch.Tensor] = None,
    shift: int = 0,
    vocab_ordering: Optional[torch.Tensor] = None,
    grad_scale: float = 1.0,
    accum_e_fp32: bool = False,
    accum_c_fp32: bool = False,
    filter_e_grad: bool = True,
    filter_c_grad: bool = True,
    reduce_e_grad: bool = False,
    pg=None,
    tile_max: Optional[torch.Tensor] = None,
    target_offset: int = 0,
    counters: Optional[torch.Tensor] = None,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Returns ``(de, dc, dbias)`` in the dtypes recorded in the ``*_info`` arguments; an
    entry is ``None`` when that input does not require a gradient (reference :391-403,
    :511-519).

    ``do`` is one element (mean / sum reductions) or the per-position upstream gradient of
    the whole batch, read at ``row + shift``; ``dlse`` likewise.  ``lse`` must be the global
    log-sum-exp when ``c`` is a vocabulary shard.

    Additions to the reference signature: ``tile_max`` (statistic of the forward pass that
    lets whole tiles be dropped before their logits are recomputed), ``target_offset``
    (first class of a vocabulary shard; the reference rebases ``targets`` on the host,
    cce.py:193-205) and ``counters`` (uint64[4] device tensor accumulating 32 x 32 sub-tiles in the
    plane / recomputed by the dE pass / with a dE product / with a dC product).  ``reduce_e_grad`` and
    ``pg`` belong to the reference's all-reduce of dE and must be left unset here.
    """
    assert do.numel() in (e.size(0), 1)
    assert c.size(1) == e.size(1)
    assert lse.size(0) == e.size(0) or (valids is not None and lse.size(0) == valids.size(0))
    assert e.ndim == 2 and c.ndim == 2 and e.is_contiguous()
    if reduce_e_grad:
        raise NotImplementedError("summing dE over vocabulary-parallel ranks is not part of this build")
    _hip.require_gpu_tensor("e", e)
    code = _hip.dtype_code(e.dtype)
    lib = _hip.load()
    dev = e.device

    if targets is None:
        # no one-hot term at all: every row gets a target that matches no class
        targets = torch.full((e.size(0),), -1, dtype=torch.int64, device=dev)
    targets = targets.to(torch.int64).contiguous()
    assert targets.numel() == e.size(0)

    do = do.to(torch.float32).contiguous().view(-1)
    lse = lse.to(torch.float32).contiguous()
    if dlse is not None:
        dlse = dlse.to(torch.float32).contiguous().view(-1)
        assert dlse.numel() == e.size(0)
        if do.numel() > 1:
            assert dlse.size() == do.size()

    n_valid_rows = valids.size(0) if valids is not None else e.size(0)
    want_de = e_info.requires_grad
    want_dc = c_info.requires_grad
    want_dbias = bias is not None and bias_info is not None and bias_info.requires_grad
    # dBias follows dC: filtered with it, unfiltered with it
    filtering = filter_eps_or_none(filter_eps) >= 0.0
    e_filtered = filtering and filter_e_grad
    c_filtered = filtering and filter_c_grad

    # Which kernels form which gradient.  An unfiltered gradient is a dense matrix product and goes to
    # cce_backward_dense; a filtered one goes to the ownership kernels (cce_backward), which pay per surviving
    # sub-tile.  The reference decides per side inside one kernel (cce_backward.py:211-216, 258-310); here the two
    # sides of a preset that filters only one of them (cce_kahan_full_c / _full_e) are two library calls.
    layout_ok = _dense_layout_ok(e, c)
    de_dense = want_de and layout_ok and not e_filtered
    dc_dense = (want_dc or want_dbias) and layout_ok and not c_filtered
    dz_budget = _dz_budget(lib, n_valid_rows, c.size(0), e.size(1), de_dense and e_info.dtype != torch.float32)
    some_filtered = (want_de and not de_dense) or ((want_dc or want_dbias) and not dc_dense)
    if (some_filtered and layout_ok and tile_max is not None and filter_eps is not None and filter_eps > 0
            and lse.numel() > 0):
        # ... unless so many cells are flagged that filtering cannot pay: then everything runs unfiltered (exact)
        de_16bit = want_de and e_info.dtype != torch.float32
        auto_budget = dz_budget if (de_dense or dc_dense) else _auto_dense_dz_budget(
            lib, n_valid_rows, c.size(0), e.size(1), de_16bit,
            n_valid_rows * e.size(1) * e.element_size() + c.numel() * c.element_size())
        if auto_budget is not None and _filtered_backward_runs_dense(
                lib, tile_max, lse, n_valid_rows, c.size(0), e.size(1), float(filter_eps), e.dtype, dev):
            de_dense, dc_dense, dz_budget = want_de, (want_dc or want_dbias), auto_budget
    de_sparse = want_de and not de_dense
    dc_sparse = (want_dc or want_dbias) and not dc_dense

    # Every kernel accumulates in fp32 registers and writes an element of dC and dBias once; dE is written once by
    # the ownership kernels and carried from chunk to chunk with a 16-bit compensation term by the unfiltered path.
    # Gradient buffers in fp32 (what accum_e_fp32 / accum_c_fp32 ask the reference for, cce_backward.py:390-394)
    # would hold the same values before the final cast, so the buffers take the dtype the caller gets back.
    de_dtype = torch.float32 if e_info.dtype == torch.float32 else e.dtype
    dc_dtype = torch.float32 if c_info.dtype == torch.float32 else c.dtype
    de = None
    if want_de:
        # the unfiltered path writes every valid row of a 16-bit dE; rows outside `valids` and every other case
        # (the ownership kernels, an fp32 accumulator) start from zeros
        de_written_whole = de_dense and valids is None and de_dtype != torch.float32 and n_valid_rows > 0
        de = torch.empty_like(e, dtype=de_dtype) if de_written_whole else torch.zeros_like(e, dtype=de_dtype)
    dc = None
    if want_dc:
        # both paths write every element of dC (the ownership kernel stores zeros for a class group nothing
        # survived for); only with no valid row at all is nothing launched
        dc = torch.empty_like(c, dtype=dc_dtype) if n_valid_rows > 0 else torch.zeros_like(c, dtype=dc_dtype)
        if dc.stride() != c.stride():
            # a view with gaps between its rows or columns (empty_like packs those): the kernels address C and
            # dC with one pair of strides, so dC gets the layout of c, or c is packed if its elements overlap
            (s_small, n_small), (s_large, _) = sorted(zip(c.stride(), c.size()))
            if s_small >= 1 and s_large >= s_small * n_small:
                dc = torch.empty_strided(c.size(), c.stride(), dtype=dc_dtype, device=dev)
                if n_valid_rows == 0:
                    dc.zero_()
            else:
                c = c.contiguous()
                dc = dc.contiguous()
    dbias = None
    if bias is not None:
        assert bias_info is not None
        bias = bias.to(e.dtype).contiguous()
        if bias_info.requires_grad:
            dbias = torch.zeros((bias.numel(),), dtype=torch.float32, device=dev)
    if de is not None:
        assert de.stride() == e.stride()
    if dc is not None:
        assert dc.stride() == c.stride()

    if valids is not None:
        assert valids.ndim == 1 and valids.dtype == torch.int32
        valids = valids.contiguous()
        B = valids.size(0)
    else:
        B = e.size(0)

    if vocab_ordering is not None:
        assert vocab_ordering.ndim == 1
        assert vocab_ordering.numel() == c.size(0)
        assert vocab_ordering.stride(0) == 1
        vocab_ordering = vocab_ordering.to(torch.int32)
    if tile_max is not None:
        assert tile_max.dtype == torch.float32 and tile_max.is_contiguous()
        assert tile_max.numel() == lib.cce_tile_stat_elems(B, c.size(0))
    if counters is not None:
        assert counters.dtype in (torch.int64, torch.uint64) and counters.numel() >= _hip.NUM_COUNTERS
        assert counters.is_contiguous() and counters.device == dev

    if B > 0 and (de_sparse or dc_sparse):
        ws_bytes = lib.cce_backward_workspace_bytes(B, c.size(0), e.size(1))
        workspace = torch.empty((max(ws_bytes, 8) // 8 + 1,), dtype=torch.int64, device=dev)
        with torch.cuda.device(dev), _hip.timed("backward_sparse", dev):
            status = lib.cce_backward(
                e.data_ptr(), c.data_ptr(), _hip.ptr(bias),
                lse.data_ptr(), do.data_ptr(), 1 if do.numel() == 1 else 0, _hip.ptr(dlse),
                _hip.ptr(valids), _hip.ptr(vocab_ordering), targets.data_ptr(),
                _hip.ptr(tile_max),
                _hip.ptr(de if de_sparse else None), _hip.ptr(dc if dc_sparse else None),
                _hip.ptr(dbias if dc_sparse else None),
                workspace.data_ptr(), workspace.numel() * 8, _hip.ptr(counters),
                e.size(0), B, c.size(0), e.size(1),
                e.stride(0), c.stride(0), c.stride(1),
                float(grad_scale), filter_eps_or_none(filter_eps),
                1 if filter_e_grad else 0, 1 if filter_c_grad else 0,
                1 if de_dtype == torch.float32 else 0, 1 if dc_dtype == torch.float32 else 0,
                int(shift), int(target_offset),
                float(softcap) if softcap is not None else 0.0, code,
                _hip.current_stream_ptr(dev),
            )
        _hip.check(status, "cce_backward")
    if B > 0 and (de_dense or dc_dense):
        _dense_backward(lib, code, dev, e, c, bias, lse, do, dlse, valids, targets,
                        de if de_dense else None, dc if dc_dense else None, dbias if dc_dense else None,
                        B, grad_scale, shift, target_offset, softcap, dz_budget)
        if counters is not None:
            # every 32 x 32 sub-tile is recomputed (once: a recompute the ownership kernels did for the other
            # side of a one-sided preset is on top and not counted) and enters the products of this call
            tiles = ((B + 31) // 32) * ((c.size(0) + 31) // 32)
            sparse_too = de_sparse or dc_sparse
            view = counters.view(torch.int64)
            if sparse_too:
                view[1] = view[0]  # recomputed = the whole plane, whatever the ownership kernels added
                view[2:4] += torch.tensor([tiles if de_dense else 0, tiles if dc_dense else 0],
                                          dtype=torch.int64, device=dev)
            else:
                view[:4] += torch.tensor([tiles, tiles, tiles if de_dense else 0, tiles if dc_dense else 0],
                                         dtype=torch.int64, device=dev)

    if dbias is not None:
        assert bias_info is not None
        dbias = dbias.to(dtype=bias_info.dtype)
    if dc is not None:
        dc = dc.to(dtype=c_info.dtype)
    if de is not None:
        de = de.to(dtype=e_info.dtype)
    return de, dc, dbias
