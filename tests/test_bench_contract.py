"""Host-side contract of bench.py and of the workspace rule of the self-chosen unfiltered backward (no GPU)."""

import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""  # no JSON line for a run that did not happen


def test_traffic_figure_is_reported_only_for_the_sources_it_was_measured_with():
    import re

    import bench

    text = open(os.path.join(ROOT, "profiles", "lse_forward_c2_hbm_traffic.txt")).read()
    m = re.search(r"traffic_bytes=(\S+) workload=(\S+) source_hash=(\S+)", text)
    assert m, "the counter summary carries the line bench.py reads"
    value, source = bench.measured_traffic(m.group(2), m.group(3))
    assert value == float(m.group(1)) and value > 1e9
    assert source == "profiles/lse_forward_c2_hbm_traffic.txt"
    assert bench.measured_traffic(m.group(2), "0" * 16) == (None, None)   # another build: no figure
    assert bench.measured_traffic("c4", m.group(3)) == (None, None)       # another workload: no figure


def test_workloads_name_the_configurations_of_the_baseline():
    import bench

    assert set(bench.WORKLOADS) == {"c1", "c2", "c3", "c4", "c5", "c5shard"}
    c2 = bench.WORKLOADS["c2"]
    assert (c2["N"], c2["D"], c2["V"], c2["softcap"], c2["impl"]) == (8192, 2304, 256000, 30.0, "cce")
    assert bench.PEAK_BF16_TFLOPS == 2516.6


class _FakeLib:
    """The two size queries of the library the rule uses, restated for the walk by classes."""

    @staticmethod
    def cce_backward_dense_fixed_bytes(b, v, d, de_16bit):
        return 2 * b * d if de_16bit else 0

    @staticmethod
    def cce_backward_dense_dz_bytes(b, v, d, de_16bit, units):
        return 2 * b * min((units + 255) // 256 * 256, (v + 255) // 256 * 256)


@pytest.mark.parametrize(
    "B,V,D,limit_bytes,operands,expect",
    [
        # c3-like: 120 MB compensation buffer; 128 MB leaves 8 MB (< 30 MB for 1024 classes): ownership kernels
        (15356, 128256, 4096, 128 << 20, 0.0, None),
        # 192 MB leaves 66 MB: chunks of 1024 classes fit
        (15356, 128256, 4096, 192 << 20, 0.0, "room"),
        # the operand rule: E + C = 1122 MB, so the 256 MB floor does not bind and the budget is DENSE_DZ_BYTES
        (15356, 128256, 4096, 256 << 20, 1.0, "budget"),
        # many rows, walked by classes: the compensation buffer alone (448 MB) exceeds 256 MB; the operands (578 MB)
        # leave 130 MB >= 128 MB
        (65536, 19008, 3584, 256 << 20, 0.0, None),
        (65536, 19008, 3584, 256 << 20, 1.0, "room"),
        # a vocabulary smaller than 1024 classes needs room for itself only
        (512, 300, 128, 1 << 20, 0.0, "room"),
    ],
)
def test_workspace_rule_of_the_self_chosen_unfiltered_backward(monkeypatch, B, V, D, limit_bytes, operands, expect):
    sys.path.insert(0, os.path.join(ROOT, "ml-cross-entropy_amd"))
    from cut_cross_entropy import cce_backward as bw

    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", limit_bytes)
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_OPERANDS", operands)
    operand_bytes = 2 * (B * D + V * D)
    got = bw._auto_dense_dz_budget(_FakeLib, B, V, D, True, operand_bytes)
    limit = max(limit_bytes, int(operands * operand_bytes))
    room = limit - 2 * B * D
    if expect is None:
        assert got is None
    elif expect == "room":
        assert got == room and got < bw._dz_budget(_FakeLib, B, V, D, True)
        assert got >= 2 * B * min(bw.AUTO_DENSE_MIN_CLASSES, (V + 255) // 256 * 256)
    else:
        assert got == bw._dz_budget(_FakeLib, B, V, D, True) and got <= room
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", None)
    assert bw._auto_dense_dz_budget(_FakeLib, B, V, D, True, operand_bytes) == bw._dz_budget(_FakeLib, B, V, D, True)
