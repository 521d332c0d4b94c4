"""Deterministic fp32 exp / sigmoid built from IEEE add, sub, mul, div, rint only.

The reference calls ``exp`` through whatever libm its backend has
(``tl.exp`` in mmfreelm/ops/hgrn/chunk.py:79, ``::exp`` in
mmfreelm/modules/activations.py:115-119, ``tl.sigmoid`` in
mmfreelm/modules/fused_norm_gate.py:126-128, ``Tensor.sigmoid`` in
mmfreelm/layers/hgrn_bit.py:113).  Those differ by an ulp between devices, so
the spec fixes one evaluation order that a CPU and a GPU both reproduce
exactly: Cody-Waite reduction by ln2 (hi = 0.693359375, lo = -2.12194440e-4),
a degree-5 polynomial in Horner form with every multiply and add rounded
separately (no FMA), and a two-step power-of-two scaling.  Max error against
float64 exp is < 2 ulp (tests/test_oracle_detmath.py).
"""
import torch

_F = torch.float32


def _c(v):
    return torch.tensor(v, dtype=_F)


_LOG2E = _c(1.44269504088896341)
_LN2_HI = _c(0.693359375)
_LN2_LO = _c(-2.12194440e-4)
_P = [_c(1.9875691500e-4), _c(1.3981999507e-3), _c(8.3334519073e-3),
      _c(4.1665795894e-2), _c(1.6666665459e-1), _c(5.0000001201e-1)]
_ONE = _c(1.0)
_XMAX = _c(89.0)
_XMIN = _c(-104.0)


def _pow2(n_i32):
    """2**n for int32 n in [-126, 127], built from the exponent bits."""
    return ((n_i32 + 127) << 23).view(_F)


def det_exp(x):
    """exp(x) for an fp32 tensor, one IEEE-rounded operation at a time."""
    assert x.dtype == _F
    xc = torch.minimum(torch.maximum(x, _XMIN), _XMAX)   # NaN propagates through min/max
    n = torch.round(xc * _LOG2E)                          # half-to-even, like rintf
    r = xc - n * _LN2_HI
    r = r - n * _LN2_LO
    z = r * r
    p = _P[0]
    for c in _P[1:]:
        p = p * r
        p = p + c
    y = p * z
    y = y + r
    y = y + _ONE
    ni = torch.nan_to_num(n, nan=0.0).to(torch.int32)
    n1 = ni >> 1                                          # floor(n/2)
    n2 = ni - n1
    y = y * _pow2(n1)
    y = y * _pow2(n2)
    return y


def det_sigmoid(x):
    """1 / (1 + exp(-x)) with det_exp; fp32 in, fp32 out."""
    return _ONE / (_ONE + det_exp(-x))
