"""ShortConvolution (mmfreelm/modules/convolution.py:45-162): CPU restatement, test infrastructure only.

``short_conv_literal`` is the reference's non-causal-conv1d branch as written (nn.Conv1d with padding W - 1, truncated to the
sequence length, then SiLU); ``short_conv_spec`` / ``short_conv_step_spec`` are the device's arithmetic: fp32, one rounding
per operation, taps added oldest first, the sum rounded to the activation dtype before pre / (1 + exp(-pre)) with the
deterministic exp.
"""
import torch
import torch.nn.functional as F

from .detmath import det_exp

_F = torch.float32
_ONE = torch.tensor(1.0, dtype=_F)


def short_conv_literal(x, weight, bias=None, activation=True):
    """x [B, T, D], weight [D, 1, W] -> [B, T, D] (convolution.py:116-131, use_causal_conv False)."""
    w = weight.shape[-1]
    y = F.conv1d(x.transpose(1, 2), weight, bias, padding=w - 1, groups=x.shape[-1])[..., :x.shape[1]]
    if activation:
        y = F.silu(y)
    return y.transpose(1, 2)


def _finish(acc, bias, dtype, activation):
    if bias is not None:
        acc = acc + bias.to(_F)
    pre = acc.to(dtype).to(_F)
    y = pre / (_ONE + det_exp(-pre)) if activation else pre
    return y.to(dtype)


def short_conv_spec(x, weight, bias=None, activation=True):
    """Returns (y [B, T, D], cache [B, D, W]: the last W inputs, oldest first, zero filled)."""
    b, t, d = x.shape
    w2 = weight.reshape(d, -1).to(x.dtype).to(_F)
    wn = w2.shape[1]
    xf = x.to(_F)
    pad = torch.cat([torch.zeros(b, wn - 1, d), xf], dim=1)          # pad[:, j] = x[:, j - (W - 1)]
    acc = torch.zeros(b, t, d)
    for w in range(wn):
        term = w2[:, w] * pad[:, w:w + t]
        valid = (torch.arange(t) - (wn - 1) + w >= 0).view(1, t, 1)
        acc = torch.where(valid, acc + term, acc)
    y = _finish(acc, bias.to(x.dtype) if bias is not None else None, x.dtype, activation)
    cache = torch.cat([torch.zeros(b, wn, d, dtype=x.dtype), x], dim=1)[:, -wn:].transpose(1, 2).contiguous()
    return y, cache


def short_conv_step_spec(x, weight, bias, cache, activation=True):
    """x [B, D], cache [B, D, W] -> (y [B, D], new cache)."""
    d = x.shape[-1]
    w2 = weight.reshape(d, -1).to(x.dtype).to(_F)
    new = torch.cat([cache[:, :, 1:], x.unsqueeze(-1)], dim=-1)
    acc = torch.zeros(x.shape)
    for w in range(w2.shape[1]):
        acc = acc + w2[:, w] * new[:, :, w].to(_F)
    return _finish(acc, bias.to(x.dtype) if bias is not None else None, x.dtype, activation), new
