"""Pins the oracle's norms, swiglu, BitLinear and HGRN scans against textbook forms (fp64, closed forms,
torch's own rms_norm / silu) and checks that the spec arithmetic stays within the floating-point tolerance
of the literal reference formulation."""
import pytest
import torch
import torch.nn.functional as F

from oracle import bitlinear as ob
from oracle import hgrn as oh
from oracle import norms as on
from oracle import quant as oq


def rel(a, b):
    a, b = a.double(), b.double()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


# ---------------------------------------------------------------- norms
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 8e-3)])
def test_rmsnorm_against_textbook(dtype, tol):
    torch.manual_seed(0)
    x = torch.randn(7, 300).to(dtype)
    w = (1 + 0.1 * torch.randn(300)).to(dtype)
    xd = x.double()
    ref = xd / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert rel(on.rms_norm_spec(x, w, eps=1e-6), ref) < tol
    assert rel(on.rms_norm_literal(x, w, eps=1e-6, upcast=True), ref) < tol
    assert rel(on.rms_norm_spec(x, w, eps=1e-6), F.rms_norm(x.float(), (300,), w.float(), 1e-6)) < tol


def test_rmsnorm_residual_and_prenorm_dtypes():
    torch.manual_seed(1)
    x = torch.randn(3, 64).bfloat16()
    r = torch.randn(3, 64).bfloat16()
    w = torch.ones(64).bfloat16()
    y, ro = on.rms_norm_spec(x, w, residual=r, prenorm=True)
    assert ro.dtype == torch.bfloat16 and torch.equal(ro, (x.float() + r.float()).bfloat16())
    y2, ro2 = on.rms_norm_spec(x, w, prenorm=True, residual_in_fp32=True)
    assert ro2.dtype == torch.float32 and torch.equal(ro2, x.float())
    # the norm sees the un-rounded fp32 sum
    s = x.float() + r.float()
    assert torch.equal(y, on.rms_norm_spec(s, w.float()).bfloat16())


def test_gated_norm_and_swiglu_against_textbook():
    torch.manual_seed(2)
    x, o = torch.randn(5, 128), 3 * torch.randn(5, 128)
    w = 1 + 0.1 * torch.randn(128)
    xd, od = x.double(), o.double()
    ref = xd / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double() * od * torch.sigmoid(od)
    assert rel(on.rms_norm_swish_gate_spec(x, o, w, 1e-6), ref) < 1e-6
    assert rel(on.rms_norm_swish_gate_literal(x, o, w, 1e-6), ref) < 1e-6
    assert rel(on.swiglu_spec(x, o), F.silu(x.double()) * od) < 1e-6
    assert rel(on.swiglu_literal(x, o), F.silu(x.double()) * od) < 1e-6


# ---------------------------------------------------------------- BitLinear
def test_bitlinear_known_answers():
    # K = 4, weight rows chosen so mean|w| = 1 and the codes are the weights themselves
    w = torch.tensor([[1.0, -1.0, 1.0, -1.0], [1.0, 1.0, 1.0, 1.0], [1.0, -1.0, -1.0, 1.0]])
    x = torch.tensor([[2.0, 2.0, 2.0, 2.0], [1.0, -1.0, 1.0, -1.0]])
    nw = torch.ones(4)
    out = ob.bitlinear_spec(x, w, nw, eps=0.0)
    # RMSNorm makes both rows +-1; codes +-127; deq = 1/127: out = sum_k sign * t
    assert torch.allclose(out, torch.tensor([[0.0, 4.0, 0.0], [4.0, 0.0, 0.0]]), atol=1e-6)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 1e-2)])
def test_bitlinear_spec_vs_literal(dtype, tol):
    torch.manual_seed(3)
    x = torch.randn(33, 512).to(dtype)
    w = (torch.randn(192, 512) * 0.02).to(dtype)
    nw = (1 + 0.1 * torch.randn(512)).to(dtype)
    b = (0.1 * torch.randn(192)).to(dtype)
    spec = ob.bitlinear_spec(x, w, nw, bias=b, eps=1e-8)
    assert rel(spec, ob.bitlinear_literal(x, w, nw, bias=b, eps=1e-8)) < tol
    assert rel(spec, ob.bitlinear_fused_literal(x, w, nw, bias=b, eps=1e-8)) < tol


def test_bitlinear_integer_identity():
    """F.linear(q/s_a, t/s_w) == (q . t) / (s_a s_w): the contraction is exact in integers."""
    torch.manual_seed(4)
    x = torch.randn(9, 256)
    w = torch.randn(40, 256) * 0.02
    q, deq, qsum, _ = on.rms_norm_quant_spec(x, None, eps=1e-8)
    t, wdeq = oq.ternary_codes(w)
    out, acc = ob.contract_exact(q, deq, t, wdeq, torch.float32)
    acc64 = q.to(torch.int64) @ t.to(torch.int64).t()
    assert torch.equal(acc.to(torch.int64), acc64)
    assert torch.equal(qsum, q.sum(-1, dtype=torch.int32))
    dense = F.linear(q.double() * deq.double().reshape(-1, 1), t.double() * wdeq.double())
    assert rel(out, dense) < 1e-6


def test_contraction_on_fp32_codes_is_the_exact_accumulator():
    """The model oracle keeps the ternary codes as fp32 for a BLAS contraction: at the widest row of the
    benchmarked shapes (K = 6912, worst-case codes +-128 / +-1) every partial sum stays below 2**24, so the fp32
    result is the int64 one."""
    torch.manual_seed(8)
    k = 6912
    q = torch.randint(-128, 128, (5, k), dtype=torch.int8)
    q[0] = -128
    q[1] = 127
    t = torch.randint(-1, 2, (33, k), dtype=torch.int8)
    t[0] = 1
    t[1] = -1
    deq = torch.rand(5) + 0.5
    wdeq = torch.tensor(0.0123)
    out32, acc32 = ob.contract_exact(q, deq, t.float(), wdeq, torch.bfloat16)
    out64, acc64 = ob.contract_exact(q, deq, t, wdeq, torch.bfloat16)
    assert torch.equal(acc32.to(torch.int64), q.to(torch.int64) @ t.to(torch.int64).t())
    assert torch.equal(acc32, acc64) and torch.equal(out32, out64)


# ---------------------------------------------------------------- scans
def test_layernorm_form_of_the_quantiser_against_the_library_layer_norm():
    """mmfreelm/ops/fusedbitnet.py:102-121 (IS_RMS_NORM false): the normalised row is torch's own layer_norm (a library
    routine that shares no code with the oracle), the codes are round(y * 127 / max|y|); rows of zero mean without a
    bias reduce to the RMSNorm form bit for bit; the device-arithmetic form gives the same codes up to rounding ties."""
    torch.manual_seed(21)
    m, k = 9, 300
    x = torch.randn(m, k) * 3 + 1.5                      # a mean far from zero: dropping the centring cannot pass
    w, b = 1 + 0.2 * torch.randn(k), 0.3 * torch.randn(k)
    res = torch.randn(m, k)
    for bias, residual in ((None, None), (b, None), (b, res)):
        xs = x if residual is None else x + residual
        y = F.layer_norm(xs.double(), (k,), w.double(), None if bias is None else bias.double(), 1e-8)
        scale = 127.0 / y.abs().amax(dim=-1, keepdim=True)
        want_codes = (y * scale).round().clamp(-128, 127)
        got = on.layer_norm_quant_literal(x, w, bias, residual=residual, eps=1e-8)
        lit_codes = (got.double() * scale).round()
        assert (lit_codes - want_codes).abs().max().item() <= 1 and (lit_codes != want_codes).float().mean().item() < 0.01
        q, deq, qsum, xsum = on.layer_norm_quant_spec(x, w, bias, residual=residual, eps=1e-8)
        assert (q.double() - want_codes).abs().max().item() <= 1 and (q.double() != want_codes).float().mean().item() < 0.01
        assert torch.equal(qsum, q.to(torch.int32).sum(dim=-1)) and torch.equal(xsum, xs)
        assert rel(deq.reshape(-1, 1), 1.0 / scale.float()) < 1e-6
    # zero-mean rows (every value beside its negative), no bias: centring changes nothing
    half = torch.randn(m, k // 2)
    z = torch.cat([half, -half], dim=-1)
    qa, da, sa, _ = on.layer_norm_quant_spec(z, w, None, eps=1e-8)
    qb, db, sb, _ = on.rms_norm_quant_spec(z, w, eps=1e-8)
    assert torch.equal(qa, qb) and torch.equal(da, db) and torch.equal(sa, sb)
    # and the contraction behind it
    wt = torch.randn(24, k) * 0.02
    out = ob.bitlinear_spec(x, wt, w, eps=1e-8, norm_bias=b, is_rms_norm=False)
    want = (want_codes_for(x, w, b, k) @ oq.weight_quant_literal(wt).double().t()).float()
    assert rel(out, want) < 5e-3


def want_codes_for(x, w, b, k):
    y = F.layer_norm(x.double(), (k,), w.double(), b.double(), 1e-8)
    scale = 127.0 / y.abs().amax(dim=-1, keepdim=True)
    return (y * scale).round().clamp(-128, 127) / scale


def test_scan_closed_forms():
    B, H, T, D = 2, 1, 50, 8
    x = torch.full((B, H, T, D), 0.5)
    g = torch.full((B, H, T, D), 0.9)
    o, ht = oh.recurrent_hgrn_spec(x, g, None, True)
    t = torch.arange(1, T + 1, dtype=torch.float64)
    geo = 0.5 * (1 - 0.9 ** t) / (1 - 0.9)                              # geometric series
    assert rel(o[0, 0, :, 0], geo) < 1e-6 and rel(ht[0, 0, 0], geo[-1]) < 1e-6
    xr = torch.randn(B, H, T, D)
    o1, _ = oh.recurrent_hgrn_spec(xr, torch.ones_like(xr))             # g = 1 -> cumulative sum
    assert rel(o1, xr.double().cumsum(2)) < 1e-6
    o0, _ = oh.recurrent_hgrn_spec(xr, torch.zeros_like(xr))            # g = 0 -> identity
    assert torch.equal(o0, xr)


def test_scan_fp64_brute_force_and_state_split():
    torch.manual_seed(5)
    B, H, T, D = 2, 2, 70, 16
    g = torch.sigmoid(torch.randn(B, H, T, D) + 2)
    x = torch.randn(B, H, T, D)
    h0 = torch.randn(B, H, D)
    o, ht = oh.recurrent_hgrn_spec(x, g, h0, True)
    h = h0.double()
    for t in range(T):
        h = g[:, :, t].double() * h + x[:, :, t].double()
        assert rel(o[:, :, t], h) < 1e-5
    # split-sequence property: scan(x[:t]) -> state -> scan(x[t:], state) == full scan, bit for bit
    o_a, h_a = oh.recurrent_hgrn_spec(x[:, :, :30], g[:, :, :30], h0, True)
    o_b, h_b = oh.recurrent_hgrn_spec(x[:, :, 30:], g[:, :, 30:], h_a, True)
    assert torch.equal(torch.cat([o_a, o_b], 2), o) and torch.equal(h_b, ht)


@pytest.mark.parametrize("chunk", [128, 64, 16, 7])
def test_chunk_equals_recurrent(chunk):
    torch.manual_seed(6)
    B, H, T, D = 2, 1, 150, 8
    glog = F.logsigmoid(torch.randn(B, H, T, D) + 2)
    x = torch.randn(B, H, T, D)
    h0 = torch.randn(B, H, D)
    oc, hc = oh.chunk_hgrn_spec(x, glog, h0, True, chunk=chunk)
    orr, hr = oh.recurrent_hgrn_spec(x, glog.exp(), h0, True)
    assert rel(oc, orr) < 1e-5 and rel(hc, hr) < 1e-5
    on_, _ = oh.naive_recurrent_hgrn_literal(x, glog.exp(), h0, True)
    assert torch.equal(on_, orr)


def test_gate_spec_vs_literal_and_lower_bound():
    torch.manual_seed(7)
    i, f = 2 * torch.randn(3, 5, 64), 2 * torch.randn(3, 5, 64)
    lb = torch.rand(64) * 0.5
    xs, gs = oh.hgrn_gate_spec(i, f, lb, layer_idx=2)
    xl, gl = oh.hgrn_gate_literal(i, f, lb, 2)
    assert rel(xs, xl) < 1e-6 and rel(gs, gl) < 1e-6
    assert (gs >= lb - 1e-7).all() and (gs <= 1).all()                  # the decay never falls below its bound
    x0, g0 = oh.hgrn_gate_spec(i, f, lb, layer_idx=0)                   # layer 0 ignores the bound
    assert rel(g0, torch.sigmoid(f.double())) < 1e-6
    mask = torch.ones(3, 5)
    mask[1, :2] = 0
    xm, _ = oh.hgrn_gate_spec(i, f, lb, 2, mask)
    assert xm[1, :2].abs().sum() == 0 and torch.equal(xm[0], xs[0])
