"""HGRNBit language model assembled from the oracle's ops.

The reference model cannot run on a CPU as shipped (its RMSNorm, swiglu and loss are
GPU-only kernels), so the forward is assembled here from the pure-torch pieces, wired as
mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py wires the fused ones:
  HGRNBitModel.forward :182-278, HGRNBitBlock.forward :87-113, HGRNBitMLP.forward :55-59,
  HGRNBitAttention.forward mmfreelm/layers/hgrn_bit.py:83-142, lm_head :386,
  lower bounds :231-238 (softmax over layers, cumsum, minus first row).

``mode="literal_ste"`` is the literal mode with the straight-through estimators of mmfreelm/ops/fusedbitnet.py:571-573 on
both quantisers, so that torch.autograd differentiates it as the reference's training path does.

``forward(..., mode="spec")`` uses the *_spec ops (what the HIP path must reproduce bit for
bit); ``mode="literal"`` uses the *_literal ops in the parameters' dtype (the reference's
PyTorch formulation: fake-quantised floats, F.linear, torch sigmoid/exp, recurrent state
kept in the activation dtype as mmfreelm/ops/hgrn/recurrent_fuse.py:143-145 does).
"""
import math

import torch

from . import bitlinear as ob
from . import hgrn as oh
from . import norms as on

_F = torch.float32


def intermediate_size(hidden_size, hidden_ratio=4, intermediate=None):
    """mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:43-47."""
    if intermediate is not None:
        return intermediate
    i = int(hidden_size * hidden_ratio * 2 / 3)
    return 256 * ((i + 256 - 1) // 256)


def init_params(vocab_size, hidden_size, num_layers, seed=0, dtype=torch.float32, std=0.02, hidden_ratio=4,
                intermediate=None):
    """Random-init state dict with the reference's parameter names: every BitLinear latent
    weight and the embedding ~ N(0, std), norm weights 1, lower_bounds 0."""
    g = torch.Generator().manual_seed(seed)
    H, I = hidden_size, intermediate_size(hidden_size, hidden_ratio, intermediate)

    def w(n, k):
        return (torch.randn(n, k, generator=g) * std).to(dtype)

    def ones(n):
        return torch.ones(n, dtype=dtype)

    p = {"model.embeddings.weight": w(vocab_size, H), "model.lower_bounds": torch.zeros(num_layers, H, dtype=dtype)}
    for i in range(num_layers):
        b = f"model.layers.{i}."
        p[b + "attn_norm.weight"] = ones(H)
        for name in ("i_proj", "f_proj", "g_proj", "o_proj"):
            p[b + f"attn.{name}.weight"] = w(H, H)
            p[b + f"attn.{name}.norm.weight"] = ones(H)
        p[b + "attn.g_norm.weight"] = ones(H)
        p[b + "mlp_norm.weight"] = ones(H)
        p[b + "mlp.gate_proj.weight"] = w(2 * I, H)
        p[b + "mlp.gate_proj.norm.weight"] = ones(H)
        p[b + "mlp.down_proj.weight"] = w(H, I)
        p[b + "mlp.down_proj.norm.weight"] = ones(I)
    p["model.norm.weight"] = ones(H)
    p["lm_head.weight"] = w(vocab_size, H)
    p["lm_head.norm.weight"] = ones(H)
    return p


def lower_bound_rows(lower_bounds):
    lb = lower_bounds.to(_F).softmax(0)
    return lb.cumsum(0) - lb[0]


class _Ops:
    def __init__(self, mode, bl_eps):
        self.mode, self.bl_eps = mode, bl_eps
        self._tern = {}

    def bitlinear(self, x, params, prefix, residual_add=None):
        w, nw = params[prefix + ".weight"], params[prefix + ".norm.weight"]
        if self.mode == "spec":
            key = prefix
            if key not in self._tern:
                from .quant import ternary_codes
                t, wdeq = ternary_codes(w)
                # kept as floats for the BLAS contraction (exact: see contract_exact); fp32 holds every partial sum
                # of a row of K codes exactly while 128 * K < 2**24
                self._tern[key] = (t.to(_F if 128 * t.shape[1] < 2 ** 24 else torch.float64), wdeq)
            t, wdeq = self._tern[key]
            shp = x.shape
            q, deq, _, _ = on.rms_norm_quant_spec(x.reshape(-1, shp[-1]), nw, eps=self.bl_eps)
            out, _ = ob.contract_exact(q, deq, t, wdeq, x.dtype)
            out = out.reshape(*shp[:-1], w.shape[0])
            if residual_add is not None:
                out = (out.to(_F) + residual_add.to(_F)).to(x.dtype)
            return out
        if self.mode == "literal_ste":
            from .backward import bitlinear_ste
            out = bitlinear_ste(x, w, nw, eps=self.bl_eps)
        else:
            out = ob.bitlinear_literal(x, w, nw, eps=self.bl_eps)
        return out if residual_add is None else residual_add + out

    def rmsnorm(self, x, w, eps, residual=None, prenorm=False):
        if self.mode == "spec":
            return on.rms_norm_spec(x, w, residual=residual, eps=eps, prenorm=prenorm)
        return on.rms_norm_literal(x, w, residual=residual, eps=eps, prenorm=prenorm, upcast=True) if not prenorm else \
            _literal_prenorm(x, w, residual, eps)

    def gated_norm(self, x, o, w, eps):
        return on.rms_norm_swish_gate_spec(x, o, w, eps) if self.mode == "spec" else on.rms_norm_swish_gate_literal(x, o, w, eps)

    def swiglu(self, a, b):
        return on.swiglu_spec(a, b) if self.mode == "spec" else on.swiglu_literal(a, b)

    def gate(self, i, f, lb, layer_idx, mask):
        if self.mode == "spec":
            return oh.hgrn_gate_spec(i, f, lb, layer_idx, mask)
        return oh.hgrn_gate_literal(i, f, lb.to(i.dtype) if lb is not None else None, layer_idx,
                                    mask.to(i.dtype) if mask is not None else None)

    def scan(self, x, g, h0):
        o, ht = oh.recurrent_hgrn_spec(x, g, h0, True)
        if self.mode != "spec":
            ht = ht.to(x.dtype)      # the reference hands the state back in the activation dtype
        return o, ht


def _literal_prenorm(x, w, residual, eps):
    dtype = x.dtype
    s = (x.float() + residual.float())
    out = on.rms_norm_literal(s, w.float(), eps=eps).to(dtype)
    return out, s.to(residual.dtype)


def forward(params, input_ids, num_layers, states=None, attention_mask=None, mode="spec", rms_norm_eps=1e-6,
            bitlinear_eps=1e-6, use_lower_bound=True, last_only=False, ops=None):
    """input_ids [B, T] -> (logits [B, T or 1, V], states list of [B, D])."""
    ops = ops or _Ops(mode, bitlinear_eps)
    h = params["model.embeddings.weight"][input_ids]
    B, T, H = h.shape
    lbs = lower_bound_rows(params["model.lower_bounds"]) if use_lower_bound else None
    new_states = []
    for i in range(num_layers):
        b = f"model.layers.{i}."
        residual = h
        hn = ops.rmsnorm(h, params[b + "attn_norm.weight"], rms_norm_eps)
        ii = ops.bitlinear(hn, params, b + "attn.i_proj")
        ff = ops.bitlinear(hn, params, b + "attn.f_proj")
        gg = ops.bitlinear(hn, params, b + "attn.g_proj")
        x_in, gate = ops.gate(ii, ff, lbs[i] if lbs is not None else None, i, attention_mask)
        h0 = states[i].reshape(B, 1, H) if states is not None else None
        o, ht = ops.scan(x_in.reshape(B, 1, T, H), gate.reshape(B, 1, T, H), h0)
        new_states.append(ht.reshape(B, H))
        o2 = ops.gated_norm(gg, o.reshape(B, T, H), params[b + "attn.g_norm.weight"], rms_norm_eps)
        a = ops.bitlinear(o2, params, b + "attn.o_proj")
        hn2, residual = ops.rmsnorm(a, params[b + "mlp_norm.weight"], rms_norm_eps, residual=residual, prenorm=True)
        y = ops.bitlinear(hn2, params, b + "mlp.gate_proj")
        g1, y1 = y.chunk(2, -1)
        z = ops.swiglu(g1, y1)
        h = ops.bitlinear(z, params, b + "mlp.down_proj", residual_add=residual)
    hN = ops.rmsnorm(h, params["model.norm.weight"], rms_norm_eps)
    if last_only:
        hN = hN[:, -1:, :]
    logits = ops.bitlinear(hN, params, "lm_head")
    return logits, new_states


def argmax_lowest(logits):
    """Greedy choice with the lowest index on exact ties (BitLinear logits tie exactly)."""
    m = logits.max(dim=-1, keepdim=True).values
    idx = torch.arange(logits.shape[-1]).expand_as(logits)
    return torch.where(logits == m, idx, torch.full_like(idx, logits.shape[-1])).min(dim=-1).values


def greedy(params, input_ids, num_layers, max_new_tokens, mode="spec", **kw):
    """Prefill + greedy decode with carried state; returns ([B, new] tokens, list of per-step logits [B, V])."""
    ops = _Ops(mode, kw.get("bitlinear_eps", 1e-6))
    logits, states = forward(params, input_ids, num_layers, mode=mode, last_only=True, ops=ops, **kw)
    toks, all_logits = [], []
    for _ in range(max_new_tokens):
        lg = logits[:, -1, :]
        all_logits.append(lg)
        nxt = argmax_lowest(lg.float())
        toks.append(nxt)
        logits, states = forward(params, nxt.reshape(-1, 1), num_layers, states=states, mode=mode, ops=ops, **kw)
    return torch.stack(toks, dim=1), all_logits
