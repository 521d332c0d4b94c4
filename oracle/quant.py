"""Activation (int8, per token) and weight (ternary, per tensor) quantisers.

``*_literal`` restate mmfreelm/ops/fusedbitnet.py:15-46 (identical copies at
mmfreelm/ops/bitnet.py:10-41) and return fake-quantised floats as the
reference does.  ``*_codes`` return the integer codes and the de-quantisation
multipliers the device kernels emit; on the same fp32 input the codes are the
integers the literal functions round to.
"""
import torch

_F = torch.float32


def activation_quant_literal(x):
    """mmfreelm/ops/fusedbitnet.py:15-29.  Arithmetic runs in ``x.dtype``."""
    scale = 127.0 / x.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    y = (x * scale).round().clamp_(-128, 127) / scale
    return y


def weight_quant_literal(w):
    """mmfreelm/ops/fusedbitnet.py:32-46.  Arithmetic runs in ``w.dtype``."""
    scale = 1.0 / w.abs().mean().clamp_(min=1e-5)
    u = (w * scale).round().clamp_(-1, 1) / scale
    return u


def activation_codes(y):
    """Per-row int8 codes of an fp32 matrix ``y`` [M, K].

    Follows the fused kernel's fp32 arithmetic (mmfreelm/ops/fusedbitnet.py:
    124-128) with torch's round-half-to-even (fusedbitnet.py:28):
        scale = 127 / max(max|y|, 1e-5);  q = clamp(rint(y * scale), -128, 127)
    Returns (q int8 [M,K], deq fp32 [M] = 1/scale, qsum int32 [M] = sum_k q).
    """
    assert y.dtype == _F and y.dim() == 2
    amax = y.abs().max(dim=-1, keepdim=True).values
    amax = torch.clamp(amax, min=torch.tensor(1e-5, dtype=_F))
    scale = torch.tensor(127.0, dtype=_F) / amax
    q = torch.round(y * scale).clamp_(-128, 127)
    deq = (torch.tensor(1.0, dtype=_F) / scale).reshape(-1)
    qi = q.to(torch.int8)
    return qi, deq, qi.to(torch.int32).sum(dim=-1, dtype=torch.int32)


def ternary_codes(w):
    """Per-tensor ternary codes of a latent weight ``w`` [N, K] (fp32/bf16/fp16).

    mmfreelm/ops/fusedbitnet.py:43-45 with every op rounded to ``w.dtype`` as
    torch eager does; the mean of |w| is accumulated in fp64 and rounded once
    (torch accumulates in fp32 in a backend-dependent order; fp64 makes the
    result order independent):
        mean  = dtype( fp32( sum64|w| / numel ) );  mean = max(mean, dtype(1e-5))
        scale = dtype( 1 / mean )
        t     = clamp(rint(dtype(w * scale)), -1, 1)
        deq   = dtype( 1 / scale )        # value of  t / scale  for t = 1
    Returns (t int8 [N,K], deq fp32 scalar tensor).
    """
    dt = w.dtype
    s64 = w.to(torch.float64).abs().sum()
    mean = (s64 / w.numel()).to(_F).to(dt)
    mean = torch.clamp(mean, min=torch.tensor(1e-5, dtype=dt))
    scale = (torch.tensor(1.0, dtype=_F) / mean.to(_F)).to(dt)
    prod = (w.to(_F) * scale.to(_F)).to(dt)      # exact fp32 product, one rounding to dt
    t = torch.round(prod.to(_F)).clamp_(-1, 1).to(torch.int8)
    deq = (torch.tensor(1.0, dtype=_F) / scale.to(_F)).to(dt).to(_F)
    return t, deq
