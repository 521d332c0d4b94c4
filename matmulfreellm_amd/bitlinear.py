"""BitLinear / FusedBitLinear (interface of mmfreelm/ops/fusedbitnet.py:513-610).

The latent weight stays an ``nn.Linear`` parameter [out, in]; its ternary codes are packed
2 bits per weight on first use and re-packed only when the parameter changes (the
reference re-quantises it on every forward, fusedbitnet.py:456).
"""
import torch
import torch.nn as nn

from . import functional as F_
from .layernorm import RMSNorm


def activation_quant(x):
    """Per-token int8 fake quantisation, the torch expression of mmfreelm/ops/fusedbitnet.py:15-29."""
    scale = 127.0 / x.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    return (x * scale).round().clamp_(-128, 127) / scale


def weight_quant(w):
    """Per-tensor ternary fake quantisation, the torch expression of mmfreelm/ops/fusedbitnet.py:32-46."""
    scale = 1.0 / w.abs().mean().clamp_(min=1e-5)
    return (w * scale).round().clamp_(-1, 1) / scale


class _PackCache:
    """Packed codes of one weight tensor, invalidated when the tensor is written or replaced."""

    def __init__(self):
        self.key, self.pw, self.frozen = None, None, False

    def freeze(self, pw):
        """Pin codes loaded from a packed checkpoint: there is no latent weight to re-pack from."""
        self.key, self.pw, self.frozen = None, pw, True

    def get(self, weight):
        if self.frozen:
            if not weight.is_meta:
                raise RuntimeError("this BitLinear holds packed codes only; assigning a latent weight to it is not supported")
            return self.pw
        key = (weight.data_ptr(), weight._version, weight.dtype, weight.device, tuple(weight.shape))
        if key != self.key:
            self.pw = F_.ternarize_pack(weight)
            self.key = key
        return self.pw


def layer_norm_linear_quant_fn(x, norm_weight, norm_bias, linear_weight, linear_bias, residual=None, eps=1e-6,
                               prenorm=False, residual_in_fp32=False, is_rms_norm=False, packed=None):
    """Same positional signature as mmfreelm/ops/fusedbitnet.py:513-536.

    is_rms_norm=False selects the LayerNorm form (row mean subtracted, optional norm_bias): forward only, the
    MatMul-free LM never takes it (FusedBitLinear passes is_rms_norm=True, fusedbitnet.py:602-610).  A norm bias on the
    RMSNorm form raises.  ``packed`` (a functional.PackedWeight) skips the ternarise+pack pass.
    """
    from .autograd import BitLinearFn, needs_grad
    if not is_rms_norm:
        if needs_grad(x, norm_weight, norm_bias, linear_weight, linear_bias, residual):
            raise NotImplementedError("the LayerNorm form of layer_norm_linear_quant_fn has no backward here "
                                      "(call it under torch.no_grad(); the model path is RMSNorm)")
        pw = packed if packed is not None else F_.ternarize_pack(linear_weight)
        return F_.bitlinear(x, norm_weight, pw, bias=linear_bias, eps=eps, residual=residual, prenorm=prenorm,
                            residual_in_fp32=residual_in_fp32, norm_bias=norm_bias, is_rms_norm=False)
    if norm_bias is not None:
        raise NotImplementedError("a norm bias exists for the LayerNorm form only (is_rms_norm=False)")
    if needs_grad(x, norm_weight, linear_weight, linear_bias, residual):
        if linear_weight.is_meta:
            raise RuntimeError("this BitLinear holds packed codes only: there is no latent weight to train")
        return BitLinearFn.apply(x, norm_weight, linear_weight, linear_bias, eps, residual, prenorm, residual_in_fp32, packed)
    pw = packed if packed is not None else F_.ternarize_pack(linear_weight)
    return F_.bitlinear(x, norm_weight, pw, bias=linear_bias, eps=eps, residual=residual, prenorm=prenorm,
                        residual_in_fp32=residual_in_fp32)


class BitLinear(nn.Linear):
    """nn.Linear whose forward is RMSNorm -> int8 absmax activations -> ternary weights.

    mmfreelm/ops/fusedbitnet.py:539-581.  eps of the inner norm is 1e-8 as there."""

    def __init__(self, in_features, out_features, bias=False):
        super().__init__(in_features, out_features, bias=bias)
        self.norm = RMSNorm(in_features, eps=1e-8)
        self._pack = _PackCache()

    def packed_weight(self):
        return self._pack.get(self.weight)

    def run_eps(self):
        """eps of the inner norm as forward() uses it (FusedBitLinear may override it)."""
        fe = getattr(self, "fused_eps", None)
        return self.norm.eps if fe is None else fe

    def forward_fused(self, x, prologue, addend=None, epilogue=None):
        """forward() with the elementwise op that produces x folded into the same launch(es);
        ``prologue`` / ``epilogue`` as functional.bitlinear takes them."""
        return F_.bitlinear(x, self.norm.weight, self.packed_weight(), bias=self.bias, eps=self.run_eps(), addend=addend,
                            prologue=prologue, epilogue=epilogue)

    def forward(self, x):
        return layer_norm_linear_quant_fn(x, self.norm.weight, self.norm.bias, self.weight, self.bias,
                                          eps=self.norm.eps, is_rms_norm=True, packed=self.packed_weight())


class FusedBitLinear(BitLinear):
    """mmfreelm/ops/fusedbitnet.py:584-610.  Same math as BitLinear here: both run the fused kernels.

    ``eps``: the reference's fused forward does not pass the norm's eps and so runs with
    layer_norm_linear_quant_fn's default 1e-6 (fusedbitnet.py:602-610 vs :520), while its un-fused
    BitLinear uses the norm's 1e-8.  HGRNBitAttention, HGRNBitMLP and the lm_head are FusedBitLinear there
    (layers/hgrn_bit.py:19, modeling_hgrn_bit.py:24), so 1e-6 is what a reference checkpoint was trained and runs
    with: it is the default here.  ``fused_eps=None`` falls back to the inner norm's own eps."""

    def __init__(self, in_features, out_features, bias=False, fused_eps=1e-6):
        super().__init__(in_features, out_features, bias=bias)
        self.fused_eps = fused_eps

    def forward(self, x):
        eps = self.norm.eps if self.fused_eps is None else self.fused_eps
        return layer_norm_linear_quant_fn(x, self.norm.weight, self.norm.bias, self.weight, self.bias, eps=eps,
                                          is_rms_norm=True, packed=self.packed_weight())
