"""RMSNorm module and functional form (interface of mmfreelm/modules/layernorm.py:534-543, 586-623)."""
import torch
import torch.nn as nn

from . import functional as F_


def rms_norm_fn(x, weight, bias, residual=None, prenorm=False, residual_in_fp32=False, eps=1e-6):
    """Same signature as mmfreelm/modules/layernorm.py:534.  bias must be None (the model never sets one)."""
    if bias is not None:
        raise NotImplementedError("RMSNorm bias is not on the MatMul-free LM path (reference registers bias=None)")
    from .autograd import RMSNormFn, needs_grad
    if needs_grad(x, weight, residual):
        return RMSNormFn.apply(x, weight, residual, eps, prenorm, residual_in_fp32)
    return F_.rmsnorm(x, weight, residual=residual, eps=eps, prenorm=prenorm, residual_in_fp32=residual_in_fp32)


class RMSNorm(nn.Module):
    """mmfreelm/modules/layernorm.py:586-623."""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5):
        super().__init__()
        self.hidden_size = hidden_size
        self.elementwise_affine = elementwise_affine
        self.eps = eps
        if elementwise_affine:
            self.weight = nn.Parameter(torch.ones(hidden_size))
        else:
            self.register_parameter("weight", None)
        self.register_parameter("bias", None)

    def __repr__(self) -> str:
        s = f"{self.__class__.__name__}({self.hidden_size}"
        if not self.elementwise_affine:
            s += f", elementwise_affine={self.elementwise_affine}"
        return s + f", eps={self.eps})"

    def forward(self, x, residual=None, prenorm=False, residual_in_fp32=False):
        return rms_norm_fn(x, self.weight, self.bias, residual=residual, eps=self.eps, prenorm=prenorm,
                           residual_in_fp32=residual_in_fp32)
