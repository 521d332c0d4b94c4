"""The loss oracle, pinned by closed forms and by torch's own cross entropy (what the reference's non-fused branch calls)."""
import math

import torch

from oracle import loss as ol


def test_closed_forms():
    v = 50
    flat = torch.zeros(1, 3, v)
    labels = torch.tensor([[4, 9, 2]])
    assert abs(ol.causal_lm_loss(flat, labels).item() - math.log(v)) < 1e-12       # uniform prediction: log V per position
    sure = torch.full((1, 3, v), -1e4)
    sure[0, 0, 9] = sure[0, 1, 2] = 0.0                                            # position t predicts token t + 1 with certainty
    assert ol.causal_lm_loss(sure, labels).item() < 1e-9
    wrong = sure.clone()
    wrong[0, 1, 2], wrong[0, 1, 3] = -1e4, 0.0                                     # one of the two scored positions is wrong by 1e4
    assert abs(ol.causal_lm_loss(wrong, labels).item() - 5e3) < 1e-6
    two = torch.tensor([[[0.0, math.log(3.0)], [0.0, 0.0]]], dtype=torch.float64)                     # p = (1/4, 3/4): -log(1/4) for target 0
    assert abs(ol.causal_lm_loss(two, torch.tensor([[1, 0]])).item() - math.log(4.0)) < 1e-12


def test_shift_and_ignore():
    labels = torch.tensor([[5, 6, 7], [8, -100, 9]])
    assert ol.shift_labels(labels).tolist() == [[6, 7, -100], [-100, 9, -100]]
    torch.manual_seed(0)
    logits = torch.randn(2, 3, 12)
    rows, counted = ol.cross_entropy_rows(logits, ol.shift_labels(labels))
    assert counted.tolist() == [True, True, False, False, True, False] and rows[2] == 0 and rows[3] == 0


def test_equals_torch_cross_entropy():
    torch.manual_seed(1)
    logits = torch.randn(3, 17, 101, dtype=torch.float64) * 4
    labels = torch.randint(0, 101, (3, 17))
    labels[1, 5] = -100
    want = torch.nn.CrossEntropyLoss()(logits.view(-1, 101), ol.shift_labels(labels).view(-1))
    assert abs(ol.causal_lm_loss(logits, labels).item() - want.item()) < 1e-12
