"""FusedRMSNormSwishGate (interface of mmfreelm/modules/fused_norm_gate.py:510-536)."""
import torch
import torch.nn as nn

from . import functional as F_


def rms_norm_swish_gate_fn(x, o, weight, bias, residual=None, prenorm=False, residual_in_fp32=False, eps=1e-6):
    """mmfreelm/modules/fused_norm_gate.py:510 (there named rms_norm_fn)."""
    if bias is not None:
        raise NotImplementedError("bias is not on the MatMul-free LM path (reference registers bias=None)")
    from .autograd import RMSNormSwishGateFn, needs_grad
    if needs_grad(x, o, weight, residual):
        if residual is not None or prenorm:
            raise NotImplementedError("the gated norm's backward takes no residual (the model never gives it one)")
        return RMSNormSwishGateFn.apply(x, o, weight, eps)
    return F_.rmsnorm_swishgate(x, o, weight, residual=residual, eps=eps, prenorm=prenorm,
                                residual_in_fp32=residual_in_fp32)


class FusedRMSNormSwishGate(nn.Module):
    """y = RMSNorm(x) * weight * o * sigmoid(o)."""

    def __init__(self, hidden_size, eps=1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.empty(hidden_size))
        self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        nn.init.ones_(self.weight)

    def forward(self, x, o, residual=None, prenorm=False, residual_in_fp32=False):
        return rms_norm_swish_gate_fn(x, o, self.weight, self.bias, residual=residual, eps=self.eps, prenorm=prenorm,
                                      residual_in_fp32=residual_in_fp32)
