"""GPU parity of the loss head (floating point: hardware exp / log, fp32 accumulation; tolerance 1e-5 relative on the
fp32 result against the float64 oracle evaluated on the same logits)."""
import pytest
import torch

from oracle import loss as ol
from oracle import model as om

pytestmark = pytest.mark.gpu
TOL = 1e-5


def F():
    import matmulfreellm_amd.functional as F_
    return F_


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,v", [(64, 32000), (7, 1000), (3, 33), (5, 1), (2, 50257), (2, 70001)])
def test_rows_and_mean_against_the_oracle(dev, dtype, rows, v):
    g = torch.Generator().manual_seed(70 + v)
    wide = (torch.randn(rows, v + 3, generator=g) * 3).to(dtype)
    logits = wide[:, :v] if v % 2 else wide[:, :v].contiguous()      # odd widths: strided rows, unaligned path
    targets = torch.randint(0, v, (rows,), generator=g)
    targets[rows // 2] = -100
    want_rows, counted = ol.cross_entropy_rows(logits, targets)
    got = F().cross_entropy(logits.to(dev), targets.to(dev)).cpu().double()
    want = want_rows.sum() / counted.sum()
    assert abs(got - want) <= TOL * max(1.0, abs(want)), (got.item(), want.item())


def test_extreme_logits_and_all_ignored(dev):
    logits = torch.zeros(4, 256)
    logits[0, 3] = 3.0e4
    logits[1] = -3.0e4
    logits[2, :] = float("-inf")
    logits[2, 7] = 0.0
    targets = torch.tensor([3, 10, 7, 0])
    want_rows, counted = ol.cross_entropy_rows(logits, targets)
    got = F().cross_entropy(logits.to(dev), targets.to(dev)).cpu().double()
    assert abs(got - want_rows.sum() / counted.sum()) < 1e-5
    nothing = F().cross_entropy(logits.to(dev), torch.full((4,), -100).to(dev))
    assert torch.isnan(nothing)                                       # as torch: the mean of no rows


def test_model_forward_with_labels(dev):
    """model(input_ids, labels=...) as the reference's forward: the loss of the oracle's logits (bit-identical to the
    model's) under the oracle's float64 cross entropy."""
    import matmulfreellm_amd as mm
    V, H, L = 1000, 256, 2
    params = om.init_params(V, H, L, seed=3, dtype=torch.bfloat16)
    model = mm.HGRNBitForCausalLM(mm.HGRNBitConfig(vocab_size=V, hidden_size=H, num_hidden_layers=L))
    model.load_state_dict(params, strict=True)
    model = model.to(device=dev, dtype=torch.bfloat16).eval()
    torch.manual_seed(4)
    ids = torch.randint(0, V, (3, 40))
    labels = ids.clone()
    labels[0, :5] = -100
    ref_logits, _ = om.forward(params, ids, L, mode="spec")
    out = model(input_ids=ids.to(dev), labels=labels.to(dev), logits_to_keep=1)
    assert out.logits.shape == (3, 40, V) and torch.equal(out.logits.cpu(), ref_logits)
    want = ol.causal_lm_loss(ref_logits, labels)
    assert out.loss.dtype == torch.float32 and abs(out.loss.item() - want.item()) <= TOL * want.item()
    tup = model(input_ids=ids.to(dev), labels=labels.to(dev), return_dict=False)
    assert torch.equal(tup[0], out.loss) and torch.equal(tup[1], out.logits)
