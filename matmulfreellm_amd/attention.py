"""HGRNBitAttention: the HGRN token mixer built from BitLinear projections.

Interface of mmfreelm/layers/hgrn_bit.py:22-162.  Data flow of forward (:83-142):
    i, f, g = i_proj(h), f_proj(h), g_proj(h)           three BitLinear H -> H
    f = sigmoid(f); f = lb + (1 - lb) * f  (layer > 0)   gate math, one fused kernel
    i = swiglu(i, 1 - f); i *= mask
    o, state = recurrence(i, f, state)                   h_t = f_t * h_{t-1} + i_t
    o = g_norm(g, o)                                     RMSNorm(g) * o * sigmoid(o)
    o = o_proj(o)
The three input projections run as one contraction over the stacked packed weights when
their inner norm weights are equal (they then share the int8 codes of h).
"""
from typing import Optional, Tuple

import torch
import torch.nn as nn

from . import functional as F_
from .autograd import module_needs_grad
from .bitlinear import FusedBitLinear as BitLinear
from .fused_norm_gate import FusedRMSNormSwishGate


class HGRNBitAttention(nn.Module):

    def __init__(self, mode: str = "fused_recurrent", hidden_size: int = 1024, num_heads: Optional[int] = None,
                 expand_ratio: Optional[int] = 1, use_short_conv: bool = False, conv_size: int = 4,
                 conv_bias: bool = False, share_conv_kernel: bool = True, layernorm_eps: float = 1e-5,
                 layer_idx: int = None, bitlinear_eps: Optional[float] = 1e-6):
        super().__init__()
        if num_heads is None:
            num_heads = 1
        self.mode = mode
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.expand_ratio = expand_ratio
        self.input_dim = int(hidden_size * expand_ratio)
        self.head_dim = self.input_dim // self.num_heads
        self.use_short_conv = use_short_conv
        self.conv_size = conv_size
        self.conv_bias = conv_bias
        self.share_conv_kernel = share_conv_kernel
        self.layer_idx = layer_idx

        assert mode in ["fused_recurrent", "chunk"], f"Not supported mode `{mode}`."
        assert self.hidden_size % num_heads == 0, f"hidden size must be divisible by num_heads of {num_heads}"

        self.i_proj = BitLinear(hidden_size, self.input_dim, bias=False, fused_eps=bitlinear_eps)
        self.f_proj = BitLinear(hidden_size, self.input_dim, bias=False, fused_eps=bitlinear_eps)
        self.g_proj = BitLinear(hidden_size, self.input_dim, bias=False, fused_eps=bitlinear_eps)
        if use_short_conv:
            # mmfreelm/layers/hgrn_bit.py:60-67.  The reference's forward cannot run with this option (it hands
            # ShortConvolution.forward(x, cache) three positionals, :101/:107-108); here the evident intent runs:
            # conv(x, conv_state).  States of a layer: (conv_state, recurrent_state) with a shared kernel, else
            # (conv_state_i, conv_state_f, recurrent_state) - the tuples the reference's forward writes back (:131-134).
            from .convolution import ShortConvolution
            if share_conv_kernel:
                self.h_conv1d = ShortConvolution(hidden_size, conv_size, activation="silu")
            else:
                self.q_conv1d = ShortConvolution(self.input_dim, conv_size, activation="silu")
                self.f_conv1d = ShortConvolution(self.input_dim, conv_size, activation="silu")
                self.i_conv1d = ShortConvolution(self.input_dim, conv_size, activation="silu")
        self.g_norm = FusedRMSNormSwishGate(self.input_dim, layernorm_eps)
        self.o_proj = BitLinear(self.input_dim, hidden_size, bias=False, fused_eps=bitlinear_eps)
        self.apply(self._initialize_weights)
        self._ifg_key, self._ifg = None, None

    def _initialize_weights(self, module):
        if getattr(module, "_is_hf_initialized", False):
            return
        if isinstance(module, nn.Linear):
            nn.init.xavier_uniform_(module.weight, gain=2 ** -2.5)
            if module.bias is not None:
                nn.init.zeros_(module.bias)
        module._is_hf_initialized = True

    # ---- stacked i/f/g projection ------------------------------------------------------
    def _stacked_ifg(self):
        """PackedWeight of [i; f; g] if the three inner norms are identical, else None."""
        projs = (self.i_proj, self.f_proj, self.g_proj)
        key = tuple((p.weight.data_ptr(), p.weight._version, p.norm.weight.data_ptr(), p.norm.weight._version,
                     p.weight.dtype, p.weight.device) for p in projs)
        if key != self._ifg_key:
            self._ifg_key = key
            same = (self.input_dim % 32 == 0 and all(p.bias is None for p in projs)
                    and all(p.norm.eps == projs[0].norm.eps and p.fused_eps == projs[0].fused_eps for p in projs)
                    and torch.equal(self.i_proj.norm.weight, self.f_proj.norm.weight)
                    and torch.equal(self.i_proj.norm.weight, self.g_proj.norm.weight))
            self._ifg = F_.stack_packed([p.packed_weight() for p in projs]) if same else None
        return self._ifg

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_values=None, use_cache: Optional[bool] = False, output_attentions: Optional[bool] = False,
                lower_bound: Optional[torch.Tensor] = None, input_norm=None, **kwargs) -> Tuple[torch.Tensor, None, object]:
        """``input_norm``: the block's RMSNorm in front of this layer; given here, it is folded into the
        stacked i/f/g projection instead of running as a launch of its own."""
        B, T, _ = hidden_states.shape
        D = self.input_dim
        if self.use_short_conv:
            return self._forward_short_conv(hidden_states, attention_mask, past_key_values, use_cache, lower_bound, input_norm)
        if module_needs_grad(self, hidden_states, lower_bound):
            return self._forward_train(hidden_states, attention_mask, lower_bound, input_norm), None, past_key_values
        last_state = past_key_values[self.layer_idx] if use_cache else None

        stacked = self._stacked_ifg()
        if stacked is not None:
            p = self.i_proj
            eps = p.norm.eps if p.fused_eps is None else p.fused_eps
            pro = ("norm", input_norm.weight, input_norm.eps) if input_norm is not None else None
            ifg = F_.bitlinear(hidden_states, p.norm.weight, stacked, eps=eps, prologue=pro)
            i, f, g = ifg[..., :D], ifg[..., D:2 * D], ifg[..., 2 * D:]
        else:
            if input_norm is not None:
                hidden_states = input_norm(hidden_states)
            i, f, g = self.i_proj(hidden_states), self.f_proj(hidden_states), self.g_proj(hidden_states)

        lb = lower_bound if (lower_bound is not None and self.layer_idx > 0) else None
        recurrent_state = last_state[-1] if use_cache else None

        if T == 1 and recurrent_state is not None and recurrent_state.dtype == torch.float32 \
                and recurrent_state.is_contiguous():
            # decode: gate math and the single recurrence step in one kernel, state updated in place
            o = F_.hgrn_step(i, f, recurrent_state.view(B, D), lb, attention_mask)
        else:
            x_in, gate = F_.hgrn_gate(i, f, lb, attention_mask)
            x4, g4 = x_in.view(B, 1, T, D), gate.view(B, 1, T, D)      # heads are independent channels
            h0 = recurrent_state.reshape(B, 1, D) if recurrent_state is not None else None
            self._check_mode(T)
            o, new_state = F_.hgrn_recurrent(x4, g4, initial_state=h0, output_final_state=bool(use_cache))
            o = o.view(B, T, D)
            if use_cache:
                recurrent_state = new_state.view(B, self.num_heads, self.head_dim)

        if past_key_values is not None:
            past_key_values.update((recurrent_state,), self.layer_idx, T)

        # g_norm (layers/hgrn_bit.py:138) folded into o_proj
        o = self.o_proj.forward_fused(g, ("gatednorm", o.reshape(g.shape), self.g_norm.weight, self.g_norm.eps))
        return o, None, past_key_values

    def _check_mode(self, T):
        """mmfreelm/layers/hgrn_bit.py:130-134 runs fused_recurrent only and raises for any other mode; the same here, in every
        path (inference, training, short convolutions): chunk_hgrn takes log-domain gates, which this layer does not form."""
        if self.mode != "fused_recurrent" and T > 1:
            raise NotImplementedError(f"Not supported mode `{self.mode}`: the model path uses fused_recurrent")

    def _forward_train(self, hidden_states, attention_mask, lower_bound, input_norm):
        """The layer as the reference composes it (mmfreelm/layers/hgrn_bit.py:110-140), one autograd Function per op;
        no state cache (training runs whole sequences)."""
        from .autograd import HGRNGateFn
        from .hgrn import fused_recurrent_hgrn
        B, T, _ = hidden_states.shape
        D = self.input_dim
        if input_norm is not None:
            hidden_states = input_norm(hidden_states)
        i, f, g = self.i_proj(hidden_states), self.f_proj(hidden_states), self.g_proj(hidden_states)
        lb = lower_bound if (lower_bound is not None and self.layer_idx > 0) else None
        x_in, gate = HGRNGateFn.apply(i, f, lb, attention_mask)
        self._check_mode(T)
        o, _ = fused_recurrent_hgrn(x_in.view(B, 1, T, D), gate.view(B, 1, T, D))
        o = self.g_norm(g, o.view(B, T, D))
        return self.o_proj(o)

    def _forward_short_conv(self, hidden_states, attention_mask, past_key_values, use_cache, lower_bound, input_norm):
        """The layer with the short convolutions in front of the projections (mmfreelm/layers/hgrn_bit.py:97-139), one
        launch per op (no folding), differentiable; see __init__ for how it departs from the reference's call."""
        from .autograd import HGRNGateFn, needs_grad
        from .hgrn import fused_recurrent_hgrn
        B, T, _ = hidden_states.shape
        D = self.input_dim
        if input_norm is not None:
            hidden_states = input_norm(hidden_states)
        last_state = past_key_values[self.layer_idx] if use_cache else None
        # Left padding: what enters a convolution (and its cache) at a padded position is zeroed, so that a pad token cannot
        # leak into the first real positions through the convolution window.  The reference cannot run this path (its call
        # passes the mask where the cache belongs), so there is nothing to compare with: parity unpinned.
        keep = attention_mask.reshape(B, T).to(hidden_states.dtype).unsqueeze(-1) if attention_mask is not None else None
        if self.share_conv_kernel:
            conv_state = last_state[0] if use_cache else None
            conv_in = hidden_states if keep is None else hidden_states * keep
            hidden_states = self.h_conv1d(conv_in, conv_state)                # the conv state is updated in place
            i, f = self.i_proj(hidden_states), self.f_proj(hidden_states)
        else:
            conv_state_i = last_state[0] if use_cache else None
            conv_state_f = last_state[1] if use_cache else None
            pi, pf = self.i_proj(hidden_states), self.f_proj(hidden_states)
            if keep is not None:
                pi, pf = pi * keep, pf * keep
            i = self.i_conv1d(pi, conv_state_i)
            f = self.f_conv1d(pf, conv_state_f)
        lb = lower_bound if (lower_bound is not None and self.layer_idx > 0) else None
        if needs_grad(i, f, lb):
            x_in, gate = HGRNGateFn.apply(i, f, lb, attention_mask)
        else:
            x_in, gate = F_.hgrn_gate(i, f, lb, attention_mask)
        recurrent_state = last_state[-1] if use_cache else None
        h0 = recurrent_state.reshape(B, 1, D) if recurrent_state is not None else None
        self._check_mode(T)
        o, new_state = fused_recurrent_hgrn(x_in.view(B, 1, T, D), gate.view(B, 1, T, D), initial_state=h0,
                                            output_final_state=bool(use_cache))
        if past_key_values is not None and use_cache:
            recurrent_state = new_state.view(B, self.num_heads, self.head_dim)
            state = (conv_state, recurrent_state) if self.share_conv_kernel else (conv_state_i, conv_state_f, recurrent_state)
            past_key_values.update(state, self.layer_idx, T)
        o = self.g_norm(self.g_proj(hidden_states), o.view(B, T, D))
        return self.o_proj(o), None, past_key_values

    def init_state(self, batch_size: int) -> Tuple[torch.Tensor]:
        """Zero states of one layer: the recurrent state [B, num_heads, head_dim] in fp32, behind the convolution
        caches [B, channels, conv_size] (activation dtype) when use_short_conv."""
        device = self.g_norm.weight.device       # the projections' latent weights may be absent (packed checkpoints)
        state = tuple()
        if self.use_short_conv:
            dt = self.g_norm.weight.dtype
            if self.share_conv_kernel:
                state += (torch.zeros(batch_size, self.hidden_size, self.conv_size, dtype=dt, device=device),)
            else:
                state += (torch.zeros(batch_size, self.input_dim, self.conv_size, dtype=dt, device=device),
                          torch.zeros(batch_size, self.input_dim, self.conv_size, dtype=dt, device=device))
        return state + (torch.zeros(batch_size, self.num_heads, self.head_dim, dtype=torch.float32, device=device),)

    def state_size(self, **kwargs) -> int:
        state_size = self.hidden_size
        for module in self.children():
            if hasattr(module, "state_size") and isinstance(module, nn.Conv1d):
                state_size += module.state_size
        return state_size
