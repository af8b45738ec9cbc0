"""The C-ABI library loads and exports every symbol include/cce_hip.h declares; the host-only
queries answer without a GPU.  No compute entry point is called here."""

import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cce_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cce_[a-z_0-9]+)\s*\(", text)))


def _lib():
    from cut_cross_entropy import _hip

    if not os.path.exists(_hip.lib_path()):
        pytest.fail(f"{_hip.lib_path()} is missing: run __graft_entry__.build() first")
    return _hip.load()


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for want in ("cce_version", "cce_error_string", "cce_tile_stat_elems", "cce_lse_forward_workspace_bytes",
                 "cce_lse_forward", "cce_indexed_neg_dot", "cce_backward_workspace_bytes", "cce_backward",
                 "cce_backward_dz", "cce_lse_forward_static", "cce_lse_forward_static_init", "cce_backward_dense",
                 "cce_backward_dense_workspace_bytes", "cce_backward_dense_fixed_bytes", "cce_backward_dense_dz_bytes",
                 "cce_count_flagged_cells", "cce_backward_products"):
        assert want in names


def test_library_exports_every_declared_symbol():
    lib = _lib()
    for name in _declared_functions():
        assert hasattr(lib, name), f"libcce_hip.so does not export {name}"


def test_binding_covers_every_declared_symbol():
    from cut_cross_entropy import _hip

    assert sorted(_hip._SIGNATURES) == _declared_functions()


def test_host_only_queries():
    lib = _lib()
    from cut_cross_entropy import _hip

    assert lib.cce_version() == _hip.ABI_VERSION
    assert lib.cce_error_string(0) == b"success"
    assert lib.cce_source_hash().decode() == _hip._hash_of_sources()  # the library matches the sources beside it
    assert b"workspace" in lib.cce_error_string(10003)
    # ceil(8192 / 32) * ceil(256000 / 32)
    assert lib.cce_tile_stat_elems(8192, 256000) == 256 * 8000
    assert lib.cce_tile_stat_elems(33, 129) == 2 * 5
    assert lib.cce_tile_stat_elems(0, 100) == 0
    ws = lib.cce_lse_forward_workspace_bytes(8192, 256000, 2304)
    assert ws > 0 and ws % 8 == 0 and ws <= 16 * 2**20
    # one bit per 32 x 32 sub-tile, rows padded to 32-bit words
    # survivor bits (256 row groups x 250 words) + a count and one id per class group for the second dC pass
    assert lib.cce_backward_workspace_bytes(8192, 256000, 2304) == 256 * 250 * 4 + (1 + 8000) * 4
    assert lib.cce_backward_workspace_bytes(0, 5, 5) == 0


def test_header_constants_match_binding():
    from cut_cross_entropy import _hip

    text = open(HEADER).read()
    assert int(re.search(r"#define CCE_STAT_ROWS (\d+)", text).group(1)) == _hip.STAT_ROWS
    assert int(re.search(r"#define CCE_STAT_COLS (\d+)", text).group(1)) == _hip.STAT_COLS
    assert int(re.search(r"#define CCE_NUM_COUNTERS (\d+)", text).group(1)) == _hip.NUM_COUNTERS
    assert int(re.search(r"#define CCE_DTYPE_BF16 (\d+)", text).group(1)) == 0
    assert int(re.search(r"#define CCE_DTYPE_F16 (\d+)", text).group(1)) == 1
    m = re.search(r"#define CCE_STATIC_SCRATCH_BYTES \((\d+) \* (\d+) \* (\d+)\)", text)
    assert int(m.group(1)) * int(m.group(2)) * int(m.group(3)) == _hip.STATIC_SCRATCH_BYTES


def test_dense_backward_plans_by_classes_or_by_rows():
    """Host-only size queries of the unfiltered backward: with 16-bit gradients and at least twice as many rows as
    classes the walk goes by blocks of rows and the compensation term in the workspace is [v, d], else [b, d]."""
    lib = _lib()
    a256 = lambda x: (x + 255) // 256 * 256
    # rows few against classes: by classes; fixed part = compensation term of dE
    assert lib.cce_backward_dense_fixed_bytes(8192, 256000, 2304, 1) == a256(8192 * 2304 * 2)
    assert lib.cce_backward_dense_fixed_bytes(8192, 256000, 2304, 0) == 0
    assert lib.cce_backward_dense_dz_bytes(8192, 256000, 2304, 1, 1024) == 8192 * 1024 * 2
    # a vocabulary shard: by rows; fixed part = compensation term of dC; a dz unit is 256 rows of all classes
    B, V, D = 65536, 19008, 3584
    v_pad = a256(V)
    assert lib.cce_backward_dense_fixed_bytes(B, V, D, 1) == a256(V * D * 2)
    assert lib.cce_backward_dense_fixed_bytes(B, V, D, 0) == 0           # fp32 gradients: by classes, nothing fixed
    assert lib.cce_backward_dense_dz_bytes(B, V, D, 1, 1024) == 1024 * v_pad * 2
    assert lib.cce_backward_dense_dz_bytes(B, V, D, 0, 1024) == B * 1024 * 2
    # the whole workspace: fixed part + a dz buffer inside the budget, never below one 256-row block
    for budget in (0, 64 << 20, 256 << 20, 1 << 32):
        total = lib.cce_backward_dense_workspace_bytes(B, V, D, 1, budget)
        dz = total - a256(V * D * 2)
        assert dz % (256 * v_pad * 2) == 0 and dz >= 256 * v_pad * 2
        assert dz <= max(budget, 256 * v_pad * 2)
        assert dz <= a256(B) * v_pad * 2
