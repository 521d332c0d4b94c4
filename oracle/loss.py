"""Next-token loss: CPU restatement used by the tests only (test infrastructure, never the product path).

The reference computes the loss in HGRNBitForCausalLM.forward
(mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:388-397): labels are shifted left by one, the last position gets
ignore_index, and FusedCrossEntropyLoss (mmfreelm/modules/fused_cross_entropy.py, default smoothing 0 and z-loss 0)
or nn.CrossEntropyLoss takes the mean over the positions that count.  Restated here in float64.
"""
import torch

IGNORE_INDEX = -100


def shift_labels(labels, ignore_index=IGNORE_INDEX):
    """labels [B, T] -> targets [B, T]: position t is scored against token t + 1; the last position is ignored."""
    return torch.cat((labels[..., 1:], torch.full_like(labels[:, :1], ignore_index)), 1)


def cross_entropy_rows(logits, targets, ignore_index=IGNORE_INDEX):
    """float64 [rows]: logsumexp(l) - l[target], 0 where the target is ignored."""
    l = logits.reshape(-1, logits.shape[-1]).double()
    t = targets.reshape(-1)
    counted = t != ignore_index
    mx = l.max(dim=-1, keepdim=True).values
    lse = (l - mx).exp().sum(-1).log() + mx[:, 0]
    picked = l.gather(1, t.clamp_min(0)[:, None])[:, 0]
    return torch.where(counted, lse - picked, torch.zeros_like(lse)), counted


def causal_lm_loss(logits, labels, ignore_index=IGNORE_INDEX):
    """The scalar the reference's forward returns for (logits [B, T, V], labels [B, T])."""
    rows, counted = cross_entropy_rows(logits, shift_labels(labels, ignore_index), ignore_index)
    return rows.sum() / counted.sum()
