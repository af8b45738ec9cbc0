"""Host-side behaviour of the operator that needs no GPU: argument validation and exception
types (reference linear_cross_entropy.py:125-192, cce.py:278-284), the preset table
(cce_utils.py:32-70), and the dense impl="torch_compile" path against the oracle."""

import pytest
import torch

from _util import IGNORE_INDEX, make_inputs
from oracle import dense_lce


def _small():
    e, c, t, bias = make_inputs(24, 32, 16, torch.float32, seed=1, bias=True)
    return e.view(2, 12, 16), c, t.view(2, 12), bias


def test_exports():
    import cut_cross_entropy as cce

    for name in ("LinearCrossEntropy", "LinearCrossEntropyImpl", "linear_cross_entropy", "VocabParallelOptions"):
        assert hasattr(cce, name)
    from cut_cross_entropy.cce_backward import cce_backward_kernel  # noqa: F401
    from cut_cross_entropy.cce_lse_forward import cce_lse_forward_kernel  # noqa: F401
    from cut_cross_entropy.constants import IGNORE_INDEX as pkg_ignore
    from cut_cross_entropy.indexed_dot import indexed_neg_dot_forward_kernel  # noqa: F401
    from cut_cross_entropy.utils import compute_z_loss  # noqa: F401

    assert pkg_ignore == -100


@pytest.mark.parametrize("shift", [-1, 12, 40])
def test_shift_out_of_range_is_value_error(shift):
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = _small()
    with pytest.raises(ValueError, match="Shift must be in the range"):
        linear_cross_entropy(e, c, t, shift=shift, impl="torch_compile")


def test_bias_length_and_shard_size_are_value_errors():
    from cut_cross_entropy import VocabParallelOptions, linear_cross_entropy

    e, c, t, bias = _small()
    with pytest.raises(ValueError, match="Bias has a different number of elements"):
        linear_cross_entropy(e, c, t, bias=bias[:-1], impl="torch_compile")
    with pytest.raises(ValueError, match="Expected c.size"):
        linear_cross_entropy(e, c, t, impl="torch_compile", vocab_parallel_options=VocabParallelOptions(0, 31))


def test_unknown_impl_and_reduction():
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = _small()
    with pytest.raises(NotImplementedError):
        linear_cross_entropy(e, c, t, impl="does_not_exist")
    with pytest.raises(ValueError):
        linear_cross_entropy(e, c, t, impl="torch_compile", reduction="median")


def test_cce_without_gpu_fails_loudly():
    """No silent fallback: the cce implementations need the HIP kernels and a GPU."""
    from cut_cross_entropy import linear_cross_entropy

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    e, c, t, _ = _small()
    with pytest.raises(RuntimeError):
        linear_cross_entropy(e, c, t, impl="cce")


def test_shape_asserts():
    from cut_cross_entropy.torch_compile import torch_compile_linear_cross_entropy

    e, c, t, _ = _small()
    with pytest.raises(AssertionError):
        torch_compile_linear_cross_entropy(e, c, t[:, :-1])
    with pytest.raises(AssertionError):
        torch_compile_linear_cross_entropy(e, c[:, :-1], t)


def test_preset_table():
    from cut_cross_entropy.cce_utils import CCEPreset, CCEPresets, LinearCrossEntropyImpl

    user = CCEPreset(filter_eps=0.25, accum_e_fp32=False, accum_c_fp32=False, filter_e_grad=False, filter_c_grad=True)
    assert CCEPresets.build_for_impl("cce", user) == user
    for name in ("cce_exact", "cce_kahan_full", "cce_kahan_full_c_full_e"):
        got = CCEPresets.build_for_impl(name, user)
        assert got["filter_eps"] is None and got["accum_e_fp32"] and got["accum_c_fp32"]
        assert got["filter_e_grad"] is False and got["filter_c_grad"] is True  # untouched
    got = CCEPresets.build_for_impl("cce_kahan_full_c", user)
    assert got == dict(filter_eps="auto", accum_e_fp32=True, accum_c_fp32=True, filter_e_grad=True, filter_c_grad=False)
    got = CCEPresets.build_for_impl("cce_kahan_full_e", user)
    assert got == dict(filter_eps="auto", accum_e_fp32=True, accum_c_fp32=True, filter_e_grad=False, filter_c_grad=True)
    with pytest.raises(ValueError):
        CCEPresets.build_for_impl("torch_compile", user)
    names = {v.name.lower() for v in LinearCrossEntropyImpl}
    assert names == {"cce", "torch_compile", "cce_kahan_full_c", "cce_kahan_full_e", "cce_exact",
                     "cce_kahan_full_c_full_e", "cce_kahan_full"}
    assert (names - {"torch_compile"}) <= CCEPresets.names


def test_handle_eps_package():
    from cut_cross_entropy.utils import _handle_eps

    assert _handle_eps("auto", torch.bfloat16) == 2.44140625e-4
    assert _handle_eps(None, torch.bfloat16) is None
    assert _handle_eps(1e-3, torch.bfloat16) == 1e-3
    with pytest.raises(RuntimeError):
        _handle_eps(3, torch.bfloat16)
    with pytest.raises(RuntimeError):
        _handle_eps("never", torch.bfloat16)


@pytest.mark.parametrize("reduction", ["none", "mean", "sum"])
@pytest.mark.parametrize("shift", [0, 2])
@pytest.mark.parametrize("softcap", [None, 10.0])
@pytest.mark.parametrize("invalids", [False, True])
def test_torch_compile_impl_matches_oracle(reduction, shift, softcap, invalids):
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, bias = make_inputs(48, 40, 12, torch.float64, seed=2, bias=True, invalid_frac=0.25 if invalids else 0.0)
    e, t = e.view(4, 12, 12), t.view(4, 12)
    got, got_lse = linear_cross_entropy(e, c, t, bias=bias, softcap=softcap, reduction=reduction, shift=shift,
                                        impl="torch_compile", return_lse=True)
    want, want_lse = dense_lce.dense_linear_cross_entropy(e, c, t, bias, IGNORE_INDEX, softcap, reduction, shift, True)
    # the dense path upcasts to float32 like the reference (torch_compile.py:38-46)
    assert got.shape == want.shape and got.dtype == torch.float32
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-5)
    assert torch.allclose(got_lse.double(), want_lse, rtol=1e-5, atol=1e-5)


def test_torch_compile_shard_matches_oracle():
    from cut_cross_entropy import VocabParallelOptions, linear_cross_entropy

    e, c, t, _ = make_inputs(30, 44, 10, torch.float64, seed=3)
    loss = linear_cross_entropy(e, c[11:33], t, impl="torch_compile", reduction="none",
                                vocab_parallel_options=VocabParallelOptions(11, 33))
    corr, lse = dense_lce.vp_shard_partials(e, c[11:33], t, 11, 33, None, None, torch.float64)
    assert torch.allclose(loss.double(), lse - corr, rtol=1e-5, atol=1e-5)


def test_vocab_parallel_options_and_dtensor_message():
    from cut_cross_entropy import VocabParallelOptions

    o = VocabParallelOptions(3, 9)
    assert (o.start, o.stop, o.group, o.reduce_e_grad) == (3, 9, None, True)
