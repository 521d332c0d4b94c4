"""RMSNorm, RMSNorm * swish-gate, swiglu and the fused norm + int8 quantiser."""
import numpy as np
import torch

from .detmath import det_exp
from .quant import activation_codes

_F = torch.float32
_ONE = torch.tensor(1.0, dtype=_F)


# ----------------------------------------------------------------------------- literal
def rms_norm_literal(x, weight, bias=None, residual=None, eps=1e-6, prenorm=False, upcast=False):
    """mmfreelm/modules/layernorm.py:73-87 (``rms_norm_ref``)."""
    dtype = x.dtype
    if upcast:
        weight = weight.float()
        bias = bias.float() if bias is not None else None
        x = x.float()
        residual = residual.float() if residual is not None else residual
    if residual is not None:
        x = (x + residual).to(x.dtype)
    rstd = 1 / torch.sqrt((x.square()).mean(dim=-1, keepdim=True) + eps)
    out = (x * rstd * weight) + bias if bias is not None else (x * rstd * weight)
    out = out.to(dtype)
    return out if not prenorm else (out, x)


def swiglu_literal(x, y):
    """mmfreelm/modules/activations.py:115-119: float(x)*float(y)/(1+exp(-float(x))) -> T."""
    xf, yf = x.float(), y.float()
    return (xf * yf / (1.0 + torch.exp(-xf))).to(x.dtype)


def rms_norm_swish_gate_literal(x, o, weight, eps=1e-6):
    """mmfreelm/modules/fused_norm_gate.py:101-131 in fp32, with torch's sigmoid."""
    xf = x.float()
    rstd = 1 / torch.sqrt(xf.square().mean(dim=-1, keepdim=True) + eps)
    y = xf * rstd * weight.float()
    of = o.float()
    return (y * of * torch.sigmoid(of)).to(x.dtype)


# ----------------------------------------------------------------------------- spec
def _rstd(xf, eps):
    """1/sqrt(mean(x^2)+eps): squares and their sum in fp64, one rounding to fp32."""
    k = xf.shape[-1]
    ss = (xf.to(torch.float64) ** 2).sum(dim=-1, keepdim=True)
    var = (ss / k).to(_F)
    # numpy's fp32 sqrt is the correctly rounded hardware one; torch.sqrt on CPU is a
    # vectorised approximation that is off by an ulp for ~0.7 % of inputs.
    root = torch.from_numpy(np.sqrt((var + torch.tensor(eps, dtype=_F)).numpy()))
    return _ONE / root


def _sum_with_residual(x, residual):
    xf = x.to(_F)
    if residual is not None:
        xf = xf + residual.to(_F)
    return xf


def rms_norm_spec(x, weight, residual=None, eps=1e-6, prenorm=False, residual_in_fp32=False):
    """mmfreelm/modules/layernorm.py:104-165 (fused kernel data flow), 445-482 (dtype rules).

    x, residual: [..., N].  fp32 math; y rounded to x.dtype; the summed residual is
    stored in residual.dtype (or fp32 if residual_in_fp32, else x.dtype) while the
    un-rounded fp32 sum feeds the norm, exactly as the fused kernel does.
    """
    xf = _sum_with_residual(x, residual)
    rstd = _rstd(xf, eps)
    y = xf * rstd
    if weight is not None:
        y = y * weight.to(_F)
    y = y.to(x.dtype)
    if not prenorm:
        return y
    res_dtype = residual.dtype if residual is not None else (_F if residual_in_fp32 else x.dtype)
    return y, xf.to(res_dtype)


def rms_norm_swish_gate_spec(x, o, weight, eps=1e-6):
    """mmfreelm/modules/fused_norm_gate.py:101-131: ((x*rstd)*w) * o * sigmoid(o)."""
    xf = x.to(_F)
    rstd = _rstd(xf, eps)
    y = (xf * rstd) * weight.to(_F)
    of = o.to(_F)
    sig = _ONE / (_ONE + det_exp(-of))
    return ((y * of) * sig).to(x.dtype)


def swiglu_spec(x, y):
    """mmfreelm/modules/activations.py:115-119 with det_exp: (x*y) / (1 + exp(-x))."""
    xf, yf = x.to(_F), y.to(_F)
    return ((xf * yf) / (_ONE + det_exp(-xf))).to(x.dtype)


def rms_norm_quant_spec(x, weight, residual=None, eps=1e-8):
    """mmfreelm/ops/fusedbitnet.py:93-128: RMSNorm then per-row absmax int8 codes.

    x [M, K] (any float dtype).  Returns (q int8, deq fp32 [M], qsum int32 [M], xsum fp32)
    where xsum is the fp32 x (+ residual) that the norm saw.
    """
    xf = _sum_with_residual(x, residual)
    rstd = _rstd(xf, eps)
    y = xf * rstd
    if weight is not None:
        y = y * weight.to(_F)
    q, deq, qsum = activation_codes(y)
    return q, deq, qsum, xf


def layer_norm_quant_literal(x, weight, bias=None, residual=None, eps=1e-8):
    """mmfreelm/ops/fusedbitnet.py:95-128 with IS_RMS_NORM false, as written there (fp32, torch reductions):
    mean, variance of x - mean, (x - mean) * rstd * w + b, then the fake quantiser; returns the de-quantised y."""
    xf = _sum_with_residual(x, residual)
    mean = xf.sum(dim=-1, keepdim=True) / xf.shape[-1]
    xbar = xf - mean
    var = (xbar * xbar).sum(dim=-1, keepdim=True) / xf.shape[-1]
    rstd = 1 / torch.sqrt(var + eps)
    y = xbar * rstd
    if weight is not None:
        y = y * weight.to(_F)
    if bias is not None:
        y = y + bias.to(_F)
    scale = 127.0 / y.abs().amax(dim=-1, keepdim=True).clamp(min=1e-5)
    return (y * scale).round().clamp(-128, 127) / scale


def layer_norm_quant_spec(x, weight, bias=None, residual=None, eps=1e-8):
    """The same branch in the device's arithmetic: sum of x in fp64 -> mean in fp32; differences in fp32; their
    squares and sum in fp64; codes as rms_norm_quant_spec.  Returns (q, deq, qsum, xsum)."""
    xf = _sum_with_residual(x, residual)
    k = xf.shape[-1]
    mean = (xf.to(torch.float64).sum(dim=-1, keepdim=True) / k).to(_F)
    xbar = xf - mean
    rstd = _rstd(xbar, eps)
    y = xbar * rstd
    if weight is not None:
        y = y * weight.to(_F)
    if bias is not None:
        y = y + bias.to(_F)
    q, deq, qsum = activation_codes(y)
    return q, deq, qsum, xf
