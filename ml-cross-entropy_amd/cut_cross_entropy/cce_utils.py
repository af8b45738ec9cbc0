"""Implementation names and the option presets behind them.

Mirrors the reference table in cut_cross_entropy/cce_utils.py:8-70:

=========================  ==========  ============  ============  =============  =============
impl                       filter_eps  accum_e_fp32  accum_c_fp32  filter_e_grad  filter_c_grad
=========================  ==========  ============  ============  =============  =============
cce                        (caller's)  (caller's)    (caller's)    (caller's)     (caller's)
cce_exact                  None        True          True          (caller's)     (caller's)
cce_kahan_full             None        True          True          (caller's)     (caller's)
cce_kahan_full_c_full_e    None        True          True          (caller's)     (caller's)
cce_kahan_full_c           "auto"      True          True          True           False
cce_kahan_full_e           "auto"      True          True          False          True
=========================  ==========  ============  ============  =============  =============

``cce_kahan`` (named in the reference README but absent from its enum) is
accepted here as an extension: "auto" filtering on both gradients with fp32
accumulation of both.
"""

import enum
from typing import Optional, TypedDict, Union


class LinearCrossEntropyImpl(enum.IntEnum):
    CCE = 1
    TORCH_COMPILE = 2
    CCE_KAHAN_FULL_C = 3
    CCE_KAHAN_FULL_E = 4
    CCE_EXACT = 5
    CCE_KAHAN_FULL_C_FULL_E = 6
    CCE_KAHAN_FULL = 7


class CCEPreset(TypedDict):
    filter_eps: Union[float, str, None]
    accum_e_fp32: bool
    accum_c_fp32: bool
    filter_e_grad: bool
    filter_c_grad: bool


_EXACT = dict(filter_eps=None, accum_e_fp32=True, accum_c_fp32=True)
_OVERRIDES = {
    "cce": {},
    "cce_exact": _EXACT,
    "cce_kahan_full": _EXACT,
    "cce_kahan_full_c_full_e": _EXACT,
    "cce_kahan_full_c": dict(
        filter_eps="auto", accum_e_fp32=True, accum_c_fp32=True,
        filter_e_grad=True, filter_c_grad=False,
    ),
    "cce_kahan_full_e": dict(
        filter_eps="auto", accum_e_fp32=True, accum_c_fp32=True,
        filter_e_grad=False, filter_c_grad=True,
    ),
    # extension, see module docstring
    "cce_kahan": dict(
        filter_eps="auto", accum_e_fp32=True, accum_c_fp32=True,
        filter_e_grad=True, filter_c_grad=True,
    ),
}


class CCEPresets:
    names = set(_OVERRIDES)

    @classmethod
    def build_for_impl(cls, impl: str, opts: CCEPreset) -> CCEPreset:
        if impl not in cls.names:
            raise ValueError(f"{impl!r} not in {cls.names}")
        merged = dict(opts)
        merged.update(_OVERRIDES[impl])
        return merged  # type: ignore[return-value]


def impl_name(impl: Union[str, LinearCrossEntropyImpl]) -> str:
    if isinstance(impl, LinearCrossEntropyImpl):
        return impl.name.lower()
    return impl


def filter_eps_or_none(x: Optional[float]) -> float:
    """Encoding used at the C boundary: a negative value switches filtering off."""
    return -1.0 if x is None else float(x)
