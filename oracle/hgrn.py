"""HGRN recurrence h_t = g_t * h_{t-1} + x_t: sequential, chunked, and the gate math."""
import torch

from .detmath import det_exp

_F = torch.float32
_ONE = torch.tensor(1.0, dtype=_F)


def naive_recurrent_hgrn_literal(x, g, initial_state=None, output_final_state=False):
    """mmfreelm/ops/hgrn/naive.py:8-31.  g is the decay in the linear domain."""
    dtype = x.dtype
    x, g = x.float(), g.float()
    B, H, T, D = x.shape
    h = torch.zeros(B, H, D, dtype=torch.float)
    o = torch.zeros_like(x)
    if initial_state is not None:
        h = h + initial_state.detach().float()
    for i in range(T):
        h = g[:, :, i] * h + x[:, :, i]
        o[:, :, i] = h
    return o.to(dtype), (h if output_final_state else None)


def recurrent_hgrn_spec(x, g, initial_state=None, output_final_state=False):
    """mmfreelm/ops/hgrn/recurrent_fuse.py:32-68: fp32 state, multiply then add
    (two roundings), o_t = dtype(h_t).  The final state is returned in fp32
    (the reference rounds it to x.dtype, recurrent_fuse.py:143-145)."""
    return naive_recurrent_hgrn_literal(x, g, initial_state, output_final_state)


def chunk_hgrn_spec(x, g, initial_state=None, output_final_state=False, chunk=128):
    """mmfreelm/ops/hgrn/chunk.py:49-116, 223-254.  g is the LOG decay.

    Pass 1 (per chunk, from zero state; chunk 0 starts from h0):
        h = exp(g_t) * h + x_t ;  gc_t = gc_{t-1} + g_t           (fp32)
    Pass 2 (chunks c >= 1 in order):  o_t += exp(gc_t) * o[c*chunk - 1]
    o rounded to x.dtype at the end; final state = fp32 o[T-1].
    """
    dtype = x.dtype
    xf, gf = x.to(_F), g.to(_F)
    B, H, T, D = xf.shape
    o = torch.empty_like(xf)
    gc = torch.empty_like(xf)
    for c0 in range(0, T, chunk):
        h = torch.zeros(B, H, D, dtype=_F)
        acc = torch.zeros(B, H, D, dtype=_F)
        if c0 == 0 and initial_state is not None:
            h = h + initial_state.detach().to(_F)
        for t in range(c0, min(c0 + chunk, T)):
            h = det_exp(gf[:, :, t]) * h + xf[:, :, t]
            acc = acc + gf[:, :, t]
            o[:, :, t] = h
            gc[:, :, t] = acc
    for c0 in range(chunk, T, chunk):
        h0 = o[:, :, c0 - 1].clone()
        c1 = min(c0 + chunk, T)
        o[:, :, c0:c1] = o[:, :, c0:c1] + det_exp(gc[:, :, c0:c1]) * h0.unsqueeze(2)
    final = o[:, :, -1].clone() if output_final_state else None
    return o.to(dtype), final


def hgrn_gate_literal(i, f, lower_bound=None, layer_idx=0, attention_mask=None):
    """mmfreelm/layers/hgrn_bit.py:113-120 in the tensors' dtype, op by op."""
    from .norms import swiglu_literal
    f = f.sigmoid()
    if lower_bound is not None and layer_idx > 0:
        f = lower_bound + (1 - lower_bound) * f
    i = swiglu_literal(i, 1 - f)
    if attention_mask is not None:
        i = i * attention_mask.unsqueeze(-1)
    return i, f


def hgrn_gate_spec(i, f, lower_bound=None, layer_idx=0, attention_mask=None):
    """Fused form of mmfreelm/layers/hgrn_bit.py:113-120 (fp32 inside, two outputs rounded):
        s  = 1 / (1 + exp(-f))
        fg = lb + (1 - lb) * s          (layer_idx > 0 and lb given; else fg = s)
        g  = dtype(fg)                  # the decay tensor the scan loads
        u  = 1 - fp32(g)
        x  = dtype( (i * u) / (1 + exp(-i)) ) ; x = 0 where the mask is 0
    lower_bound: fp32 [D].  Returns (x, g) in i.dtype.
    """
    dt = i.dtype
    fi, ff = i.to(_F), f.to(_F)
    s = _ONE / (_ONE + det_exp(-ff))
    if lower_bound is not None and layer_idx > 0:
        lb = lower_bound.to(_F)
        s = lb + (_ONE - lb) * s
    g = s.to(dt)
    u = _ONE - g.to(_F)
    xo = ((fi * u) / (_ONE + det_exp(-fi))).to(dt)
    if attention_mask is not None:
        xo = torch.where(attention_mask.unsqueeze(-1) != 0, xo, torch.zeros_like(xo))
    return xo, g
