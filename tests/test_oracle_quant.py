"""Pins the oracle's quantisers (reference: mmfreelm/ops/fusedbitnet.py:15-46) without importing the reference:
hand-computed rows with exact .5 ties, invariants, and agreement of the code-returning and the literal forms."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle import pack as op
from oracle import quant as oq


def test_activation_known_answer_with_ties():
    # amax = 127 -> scale = 1: codes are the round-half-to-even integers of the row itself
    row = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, 3.51, -126.5]])
    q, deq, qsum = oq.activation_codes(row)
    assert q.tolist() == [[127, 0, 2, 2, 0, -2, -2, 3, 4, -126]]
    assert deq.item() == 1.0 and qsum.item() == 127 + 2 + 2 - 2 - 2 + 3 + 4 - 126
    # the literal fake-quantised output is codes / scale
    assert torch.equal(oq.activation_quant_literal(row), q.float())


def test_activation_scale_and_clamp():
    row = torch.tensor([[2.0, -4.0, 1.0, 0.0]])
    q, deq, _ = oq.activation_codes(row)
    # scale = 127/4 = 31.75: 2*31.75 = 63.5 -> 64 (even), 1*31.75 = 31.75 -> 32
    assert q.tolist() == [[64, -127, 32, 0]]
    assert deq.item() == np.float32(1.0) / (np.float32(127.0) / np.float32(4.0))
    zero = torch.zeros(1, 8)
    q0, deq0, _ = oq.activation_codes(zero)
    assert q0.abs().sum() == 0 and deq0.item() == np.float32(1.0) / (np.float32(127.0) / np.float32(1e-5))


@settings(max_examples=50, deadline=None)
@given(st.integers(0, 2**31 - 1), st.integers(1, 6), st.sampled_from([1, 7, 64, 300]))
def test_activation_invariants(seed, m, k):
    g = torch.Generator().manual_seed(seed)
    y = torch.randn(m, k, generator=g) * (10 ** torch.empty(m, 1).uniform_(-3, 3, generator=g))
    q, deq, qsum = oq.activation_codes(y)
    assert q.min() >= -127 and q.max() <= 127
    assert (q.abs().max(dim=-1).values == 127).all()                    # the absmax element always hits +-127
    qn, _, qsn = oq.activation_codes(-y)
    assert torch.equal(qn, -q) and torch.equal(qsn, -qsum)             # half-even rounding is odd-symmetric
    q2, deq2, _ = oq.activation_codes(y * 4.0)                         # power-of-two rescaling changes nothing
    assert torch.equal(q2, q) and torch.equal(deq2, deq * 4.0)
    # literal form rounds to the same integers
    lit = oq.activation_quant_literal(y)
    scale = 127.0 / y.abs().max(dim=-1, keepdim=True).values.clamp(min=1e-5)
    assert torch.equal(torch.round(lit * scale).to(torch.int8), q)
    # idempotence: quantising the de-quantised row gives the same codes
    q3, _, _ = oq.activation_codes(q.float() * deq.reshape(-1, 1))
    assert torch.equal(q3, q)


def test_ternary_known_answer():
    # mean|w| = 1 -> scale 1: codes = clamp(round_half_even(w), -1, 1)
    w = torch.tensor([[0.5, 1.5, -0.5, -1.5], [2.0, -2.0, 0.49, 0.0]])
    w = w * (8.0 / w.abs().sum())          # make mean|w| exactly 1
    t, deq = oq.ternary_codes(w)
    s = 8.0 / 8.99
    expect = torch.tensor([[0.5 * s, 1.5 * s, -0.5 * s, -1.5 * s], [2 * s, -2 * s, 0.49 * s, 0.0]]).round().clamp(-1, 1)
    assert torch.equal(t.float(), expect)
    assert abs(deq.item() - 1.0) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_ternary_matches_literal_and_invariants(dtype):
    torch.manual_seed(0)
    w = (torch.randn(96, 200) * 0.02).to(dtype)
    t, deq = oq.ternary_codes(w)
    assert set(t.unique().tolist()) <= {-1, 0, 1}
    frac0 = (t == 0).float().mean().item()
    assert 0.25 < frac0 < 0.37                                          # P(|z| < 0.5*sqrt(2/pi)) ~ 0.31 for Gaussian w
    lit = oq.weight_quant_literal(w).float()                            # fake-quantised: t * (1/scale) in w.dtype
    assert torch.equal(torch.sign(lit).to(torch.int8), t)               # same ternary codes
    # same step up to the summation order of mean|w| (torch sums in fp32, the spec in fp64)
    assert abs(lit.abs().max().item() - deq.item()) <= deq.item() * (2 ** -7 if dtype != torch.float32 else 2 ** -21)
    t2, deq2 = oq.ternary_codes((w.float() * 8.0).to(dtype))           # codes invariant under power-of-two scaling
    assert torch.equal(t2, t) and deq2.item() == deq.item() * 8.0
    tn, _ = oq.ternary_codes(-w)
    assert torch.equal(tn, -t)
    tz, dz = oq.ternary_codes(torch.zeros(4, 4, dtype=dtype))
    assert tz.abs().sum() == 0


@settings(max_examples=30, deadline=None)
@given(st.integers(1, 100), st.integers(1, 400), st.integers(0, 2**31 - 1))
def test_pack_roundtrip(n, k, seed):
    rng = np.random.default_rng(seed)
    t = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    p = op.pack_ternary(t)
    npad, kpad, nd = op.packed_shape(n, k)
    assert p.size == nd and npad % 32 == 0 and kpad % 128 == 0
    assert np.array_equal(op.unpack_ternary(p, n, k), t)


def test_pack_layout_known_positions():
    # one +1 at (row 33, input 150): block nb=1, kb=1, s=0 (150-128=22 -> s=0, half=1, i=6), lane = 32 + 1
    t = np.zeros((64, 256), dtype=np.int8)
    t[33, 150] = 1
    p = op.pack_ternary(t).reshape(2, 2, 64, 4)
    base = 0x55555555
    assert p[1, 1, 33, 0] == base + (1 << (8 * (6 % 4) + 2 * (6 // 4)))
    others = p.copy()
    others[1, 1, 33, 0] = base
    assert (others == base).all()
