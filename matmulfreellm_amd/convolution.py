"""ShortConvolution: causal depthwise convolution with an optional SiLU (mmfreelm/modules/convolution.py:45-162).

Same constructor, parameters (``weight`` [D, 1, W], optional ``bias``) and methods as the reference's nn.Conv1d subclass;
the arithmetic runs in the HIP kernels of csrc/conv.hip.  ``use_causal_conv`` is accepted and ignored (there is one
implementation here).  Unlike the reference's forward, which leaves a given cache untouched when it sees more than one
token, a cache passed with a whole sequence receives the last ``kernel_size`` inputs, so that decoding can continue
from a prefill.
"""
from typing import Optional

import torch
import torch.nn as nn

from . import functional as F_


class ShortConvolution(nn.Conv1d):

    def __init__(self, hidden_size: int, kernel_size: int, bias: bool = False, activation: Optional[str] = "silu",
                 use_causal_conv: Optional[bool] = True):
        super().__init__(in_channels=hidden_size, out_channels=hidden_size, kernel_size=kernel_size, groups=hidden_size,
                         bias=bias, padding=kernel_size - 1)
        self.hidden_size = hidden_size
        self.activation = None
        if activation is not None:
            assert activation in ["silu", "swish"], f"Activation `{activation}` not supported yet."
            self.activation = activation
        self.use_causal_conv = use_causal_conv

    def extra_repr(self):
        s = super().extra_repr()
        return s + (f", activation={self.activation}" if self.activation is not None else "")

    def forward(self, x: torch.Tensor, cache: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x [batch_size, seq_len, hidden_size] -> same shape; cache [batch_size, hidden_size, kernel_size], updated in place."""
        if cache is not None and x.shape[1] == 1:
            return self.step(x, cache)
        from .autograd import ShortConvFn, needs_grad
        if needs_grad(x, self.weight, self.bias):
            y = ShortConvFn.apply(x, self.weight, self.bias, self.activation is not None)
            if cache is not None:
                with torch.no_grad():
                    F_.short_conv(x.detach(), self.weight, self.bias, self.activation is not None, cache=cache)
            return y
        return F_.short_conv(x, self.weight, self.bias, self.activation is not None, cache=cache)

    def step(self, x: torch.Tensor, cache: torch.Tensor):
        assert x.shape[1] == 1, "Only support decoding with 1 token at a time for now"
        return F_.short_conv_step(x.squeeze(1), self.weight, self.bias, cache, self.activation is not None).unsqueeze(1)

    @property
    def state_size(self) -> int:
        return self.hidden_size * self.kernel_size[0]
