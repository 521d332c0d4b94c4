"""BitLinear forward: RMSNorm -> int8 activation codes -> ternary contraction."""
import torch
import torch.nn.functional as F

from .norms import layer_norm_quant_spec, rms_norm_literal, rms_norm_quant_spec
from .quant import activation_quant_literal, ternary_codes, weight_quant_literal

_F = torch.float32


def bitlinear_literal(x, weight, norm_weight, bias=None, eps=1e-8):
    """mmfreelm/ops/fusedbitnet.py:558-581 (BitLinear.forward, forward value only):
    RMSNorm -> activation_quant -> weight_quant -> F.linear, all in x.dtype."""
    x_norm = rms_norm_literal(x, norm_weight, eps=eps, upcast=True)
    x_q = activation_quant_literal(x_norm)
    w_q = weight_quant_literal(weight).to(x.dtype)
    return F.linear(x_q, w_q, bias)


def bitlinear_fused_literal(x, weight, norm_weight, bias=None, eps=1e-6):
    """mmfreelm/ops/fusedbitnet.py:93-131 + 454-458 (the fused path's data flow):
    fp32 norm + fake-quant, y stored in x.dtype, then F.linear with weight_quant(W)."""
    xf = x.float()
    rstd = 1 / torch.sqrt(xf.square().mean(dim=-1, keepdim=True) + eps)
    y = xf * rstd * norm_weight.float()
    y = activation_quant_literal(y).to(x.dtype)
    w_q = weight_quant_literal(weight).to(x.dtype)
    return F.linear(y, w_q, bias)


def contract_exact(q, deq, t, wdeq, out_dtype, bias=None):
    """out[m,n] = dtype( fp32(acc[m,n]) * deq[m] * wdeq (+ bias[n]) ),
    acc = sum_k q[m,k] * t[n,k] in exact integers (|acc| <= 128*K < 2**24)."""
    # BLAS matmul of small integers held as floats: every product and partial sum is an integer of magnitude
    # <= 128 * K, exactly representable below 2**53 in fp64 (and below 2**24 in fp32), so whatever the summation
    # order the result is the exact integer accumulator (and fast).  t may come in already converted (fp32 or
    # fp64, the caller's choice under that bound); int8 codes are converted to fp64 here.
    ft = t.dtype if t.is_floating_point() else torch.float64
    assert 128 * q.shape[-1] < (2 ** 24 if ft == torch.float32 else 2 ** 53)
    acc = (q.to(ft) @ t.to(ft).t())
    out = (acc.to(_F) * deq.reshape(-1, 1)) * wdeq
    if bias is not None:
        out = out + bias.to(_F)
    return out.to(out_dtype), acc.to(torch.int32)


def bitlinear_spec(x, weight, norm_weight, bias=None, eps=1e-8, residual=None, norm_bias=None, is_rms_norm=True):
    """Integer-exact BitLinear on x [..., K], weight [N, K] -> [..., N] in x.dtype (is_rms_norm=False: the LayerNorm
    form of mmfreelm/ops/fusedbitnet.py:513-536)."""
    shp = x.shape
    x2 = x.reshape(-1, shp[-1])
    r2 = residual.reshape(-1, shp[-1]) if residual is not None else None
    if is_rms_norm:
        q, deq, _, _ = rms_norm_quant_spec(x2, norm_weight, residual=r2, eps=eps)
    else:
        q, deq, _, _ = layer_norm_quant_spec(x2, norm_weight, norm_bias, residual=r2, eps=eps)
    t, wdeq = ternary_codes(weight)
    out, _ = contract_exact(q, deq, t, wdeq, x.dtype, bias)
    return out.reshape(*shp[:-1], weight.shape[0])
