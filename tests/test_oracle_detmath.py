"""The deterministic exp used by the spec arithmetic: accuracy against float64 and edge cases."""
import torch

from oracle.detmath import det_exp, det_sigmoid


def test_det_exp_accuracy():
    x = torch.linspace(-87.0, 88.0, 1000001)
    y = det_exp(x)
    ref = torch.exp(x.double())
    rel = ((y.double() - ref).abs() / ref).max().item()
    assert rel < 2 ** -22, rel           # < 2 ulp
    assert torch.all(y[1:] >= y[:-1])    # monotone on the grid


def test_det_exp_edges():
    v = det_exp(torch.tensor([0.0, -200.0, 200.0, float("inf"), -float("inf")]))
    assert v[0].item() == 1.0 and v[1].item() == 0.0 and torch.isinf(v[2]) and torch.isinf(v[3]) and v[4].item() == 0.0
    assert torch.isnan(det_exp(torch.tensor([float("nan")]))).all()


def test_det_sigmoid():
    x = torch.randn(100000) * 6
    assert (det_sigmoid(x) - torch.sigmoid(x.double()).float()).abs().max().item() < 2e-7
    s = det_sigmoid(torch.tensor([-200.0, 0.0, 200.0]))
    assert s.tolist() == [0.0, 0.5, 1.0]
