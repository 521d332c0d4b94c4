"""The backward oracle (torch.autograd through oracle/*_literal and oracle/backward.py) against the reference's
hand-written backward formulas, restated here in float64 numpy from the kernels' text:
  norm backward          mmfreelm/ops/fusedbitnet.py:272-300 (same in modules/layernorm.py:300-325)
  gated norm backward    mmfreelm/modules/fused_norm_gate.py:275-292
  swiglu backward        mmfreelm/modules/activations.py:121-126
  scan backward          mmfreelm/ops/hgrn/recurrent_fuse.py:112-132
  cross-entropy backward mmfreelm/modules/fused_cross_entropy.py:140-151
  BitLinear backward     mmfreelm/ops/fusedbitnet.py:470-510
A wrong sign, a dropped term or a transposed operand in either restatement fails here.
"""
import numpy as np
import torch

from oracle import backward as obw
from oracle import hgrn as oh
from oracle import norms as on

torch.manual_seed(0)


def _np(t):
    return t.detach().double().numpy()


def test_rmsnorm_backward_formula():
    m, n, eps = 5, 24, 1e-6
    x = torch.randn(m, n, dtype=torch.float64, requires_grad=True)
    w = torch.randn(n, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(m, n, dtype=torch.float64)
    on.rms_norm_literal(x, w, eps=eps).backward(dy)
    X, W, DY = _np(x), _np(w), _np(dy)
    rstd = 1.0 / np.sqrt((X * X).mean(-1, keepdims=True) + eps)
    xhat = X * rstd
    wdy = DY * W
    c1 = (xhat * wdy).sum(-1, keepdims=True) / n
    assert np.allclose(_np(x.grad), (wdy - xhat * c1) * rstd, rtol=1e-10, atol=1e-12)
    assert np.allclose(_np(w.grad), (DY * xhat).sum(0), rtol=1e-10, atol=1e-12)


def test_prenorm_residual_backward_adds_the_residual_gradient():
    m, n, eps = 4, 16, 1e-6
    x = torch.randn(m, n, dtype=torch.float64, requires_grad=True)
    r = torch.randn(m, n, dtype=torch.float64, requires_grad=True)
    w = torch.randn(n, dtype=torch.float64)
    dy, dres = torch.randn(m, n, dtype=torch.float64), torch.randn(m, n, dtype=torch.float64)
    y, s = on.rms_norm_literal(x, w, residual=r, eps=eps, prenorm=True)
    (y * dy).sum().add((s * dres).sum()).backward()
    S = _np(x) + _np(r)
    rstd = 1.0 / np.sqrt((S * S).mean(-1, keepdims=True) + eps)
    xhat, wdy = S * rstd, _np(dy) * _np(w)
    want = (wdy - xhat * (xhat * wdy).sum(-1, keepdims=True) / n) * rstd + _np(dres)
    assert np.allclose(_np(x.grad), want, rtol=1e-10) and np.allclose(_np(r.grad), want, rtol=1e-10)


def test_gated_norm_backward_formula():
    m, n, eps = 5, 24, 1e-6
    x = torch.randn(m, n, dtype=torch.float64, requires_grad=True)
    o = torch.randn(m, n, dtype=torch.float64, requires_grad=True)
    w = torch.randn(n, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(m, n, dtype=torch.float64)
    on.rms_norm_swish_gate_literal(x, o, w, eps=eps).backward(dy)
    X, O, W, DY = _np(x), _np(o), _np(w), _np(dy)
    rstd = 1.0 / np.sqrt((X * X).mean(-1, keepdims=True) + eps)
    xhat = X * rstd
    y = xhat * W
    sg = 1.0 / (1.0 + np.exp(-O))
    do = DY * y * (sg + O * sg * (1 - sg))
    dy2 = DY * O * sg
    wdy = W * dy2
    c1 = (xhat * wdy).sum(-1, keepdims=True) / n
    # the literal function computes in fp32 whatever it is given
    assert np.allclose(_np(o.grad), do, rtol=1e-4, atol=1e-6)
    assert np.allclose(_np(x.grad), (wdy - xhat * c1) * rstd, rtol=1e-4, atol=1e-6)
    assert np.allclose(_np(w.grad), (dy2 * xhat).sum(0), rtol=1e-4, atol=1e-6)


def test_swiglu_backward_formula():
    x = torch.randn(7, 9, dtype=torch.float64, requires_grad=True)
    y = torch.randn(7, 9, dtype=torch.float64, requires_grad=True)
    g = torch.randn(7, 9, dtype=torch.float64)
    (x * torch.sigmoid(x) * y).backward(g)                      # swiglu_literal computes in fp32; the expression is this one
    X, Y, G = _np(x), _np(y), _np(g)
    s = 1.0 / (1.0 + np.exp(-X))
    assert np.allclose(_np(x.grad), s * (1 + X * (1 - s)) * G * Y, rtol=1e-10)
    assert np.allclose(_np(y.grad), X * s * G, rtol=1e-10)
    x32, y32 = x.detach().float().requires_grad_(), y.detach().float().requires_grad_()
    on.swiglu_literal(x32, y32).backward(g.float())
    assert np.allclose(_np(x32.grad), _np(x.grad), rtol=1e-4, atol=1e-6)


def test_scan_backward_formula():
    b, h, t, d = 2, 1, 9, 5
    x = torch.randn(b, h, t, d, requires_grad=True)
    g = torch.sigmoid(torch.randn(b, h, t, d)).requires_grad_()
    h0 = torch.randn(b, h, d)
    do = torch.randn(b, h, t, d)
    o, _ = oh.naive_recurrent_hgrn_literal(x, g, h0, True)
    o.backward(do)
    G, O, DO, H0 = _np(g), _np(o), _np(do), _np(h0)
    dh = np.zeros((b, h, d))
    dx, dg = np.zeros_like(G), np.zeros_like(G)
    for i in range(t - 1, -1, -1):                              # recurrent_fuse.py:112-132
        prev = O[:, :, i - 1] if i > 0 else H0
        dh = dh + DO[:, :, i]
        dx[:, :, i] = dh
        dg[:, :, i] = dh * prev
        dh = dh * G[:, :, i]
    assert np.allclose(_np(x.grad), dx, rtol=1e-4, atol=1e-5) and np.allclose(_np(g.grad), dg, rtol=1e-4, atol=1e-5)


def test_cross_entropy_backward_formula_and_torch_equivalence():
    rows, v = 6, 11
    logits = torch.randn(rows, v, dtype=torch.float64, requires_grad=True)
    labels = torch.tensor([3, 0, -100, 10, 5, 5])
    s, scale, zs = 0.1, 0.7, 1e-2
    loss, z = obw.cross_entropy_ref(logits, labels, s, scale, zs)
    dl = torch.randn(rows)
    (loss.double() * dl.double()).sum().backward()
    L = _np(logits) * scale
    lse = np.log(np.exp(L).sum(-1))
    probs = np.exp(L - lse[:, None])
    probs = probs + 2.0 * zs * lse[:, None] * probs             # fused_cross_entropy.py:140-141
    onehot = np.zeros_like(probs)
    for r, lab in enumerate(labels.tolist()):
        if lab >= 0:
            onehot[r, lab] = 1.0
    want = (probs - onehot * (1 - s) - s / v) * (np.where(labels.numpy() == -100, 0.0, dl.numpy()) * scale)[:, None]
    assert np.allclose(_np(logits.grad), want, rtol=1e-5, atol=1e-7)
    # without z-loss the value is torch's own label-smoothed cross entropy
    plain, _ = obw.cross_entropy_ref(logits.detach(), labels, s, scale, 0.0)
    ref = torch.nn.functional.cross_entropy(logits.detach() * scale, labels, label_smoothing=s, reduction="none")
    assert torch.allclose(plain.double(), ref, rtol=1e-5, atol=1e-6)


def test_bitlinear_backward_is_the_reference_hand_written_one():
    """LayerNormLinearQuantFn.backward (fusedbitnet.py:470-510): dy = dout W_q; norm backward of dy with the quantised
    output y recomputed; dW = dout^T y; the gradient ignores both rounding steps (straight-through)."""
    from oracle.quant import activation_quant_literal, weight_quant_literal
    m, k, n, eps = 6, 32, 10, 1e-8
    x = torch.randn(m, k, requires_grad=True)
    w = (torch.randn(n, k) * 0.02).requires_grad_()
    nw = (torch.rand(k) + 0.5).requires_grad_()
    dout = torch.randn(m, n)
    obw.bitlinear_ste(x, w, nw, eps=eps).backward(dout)
    X, NW, DO = _np(x), _np(nw), _np(dout)
    wq = _np(weight_quant_literal(w.detach()))
    rstd = 1.0 / np.sqrt((X * X).mean(-1, keepdims=True) + eps)
    xhat = X * rstd
    y = _np(activation_quant_literal((x.detach() * torch.from_numpy(rstd).float() * nw.detach())))
    dy = DO @ wq
    wdy = dy * NW
    c1 = (xhat * wdy).sum(-1, keepdims=True) / k
    assert np.allclose(_np(x.grad), (wdy - xhat * c1) * rstd, rtol=2e-3, atol=1e-5)
    assert np.allclose(_np(nw.grad), (dy * xhat).sum(0), rtol=2e-3, atol=1e-5)
    assert np.allclose(_np(w.grad), DO.T @ y, rtol=2e-3, atol=1e-5)
