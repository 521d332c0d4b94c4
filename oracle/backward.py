"""Differentiable CPU restatement of the training side: what torch.autograd derives for the reference's PyTorch
formulation is the expected gradient of every backward kernel.

Test infrastructure only (tests/ and the smoke check may import it; the product never does).

  bitlinear_ste        BitLinear.forward with its straight-through estimators, mmfreelm/ops/fusedbitnet.py:558-581
                       (LayerNormLinearQuantFn.backward :470-510 is the hand-written derivative of the same expression)
  cross_entropy_ref    the loss of mmfreelm/modules/fused_cross_entropy.py:26-98 written with torch ops
  model_loss           next-token loss of the assembled model (oracle.model, mode "literal_ste")
The other ops (oracle.norms.rms_norm_literal, rms_norm_swish_gate_literal, swiglu_literal, oracle.hgrn.hgrn_gate_literal,
naive_recurrent_hgrn_literal) are plain torch expressions already: autograd differentiates them as they are.
The hand-written backward formulas of the reference's kernels are restated separately in tests/test_oracle_backward.py and
checked against this autograd, which pins both against each other.
"""
import torch
import torch.nn.functional as F

from .norms import rms_norm_literal
from .quant import activation_quant_literal, weight_quant_literal


def bitlinear_ste(x, weight, norm_weight, bias=None, eps=1e-8, weight_dtype=None):
    """weight_dtype: the dtype the latent weight is stored in when this function is evaluated in a wider one
    (weight_quant runs in the weight's own dtype, fusedbitnet.py:43-45: a bf16 weight rounds w * scale to bf16 before
    it is rounded to a code, so its codes differ from the fp32 evaluation's near the +-0.5 boundaries)."""
    x_norm = rms_norm_literal(x, norm_weight, eps=eps, upcast=True)
    x_q = x_norm + (activation_quant_literal(x_norm) - x_norm).detach()
    wd = weight.detach() if weight_dtype is None else weight.detach().to(weight_dtype)
    w_q = weight + (weight_quant_literal(wd).to(weight.dtype) - weight).detach()
    return F.linear(x_q, w_q.to(x_q.dtype), bias)


def cross_entropy_ref(logits, labels, smoothing=0.0, logit_scale=1.0, lse_square_scale=0.0, ignore_index=-100):
    """Per-row (loss, z_loss) in fp32: lse - smoothing mean(l) - (1 - smoothing) l[label] + z, z = lse_square_scale lse^2;
    zeros on ignored rows (fused_cross_entropy.py:55-87)."""
    l = logits.float() * logit_scale
    lse = torch.logsumexp(l, dim=-1)
    keep = labels != ignore_index
    safe = labels.clamp(min=0)
    picked = l.gather(1, safe[:, None])[:, 0]
    loss = lse - smoothing * l.mean(dim=-1) - (1.0 - smoothing) * picked
    z = lse_square_scale * lse * lse
    zero = torch.zeros_like(loss)
    return torch.where(keep, loss + z, zero), torch.where(keep, z, zero)


def model_loss(params, input_ids, labels, num_layers, **kw):
    """Mean next-token loss as HGRNBitForCausalLM.forward computes it (modeling_hgrn_bit.py:388-397)."""
    from . import model as om
    logits, _ = om.forward(params, input_ids, num_layers, mode="literal_ste", **kw)
    targets = torch.cat((labels[..., 1:], torch.full_like(labels[:, :1], -100)), 1).reshape(-1)
    loss, _ = cross_entropy_ref(logits.reshape(-1, logits.shape[-1]), targets)
    return loss.sum() / (targets != -100).sum()
