"""The sampling oracle, pinned: closed forms on tiny rows, the installed transformers' own TopPLogitsWarper (the
third-party code the reference's generate.py samples through), and the distribution the draw realises."""
import numpy as np
import pytest
import torch

from oracle import sampling as S


def test_three_token_closed_form():
    lg = np.log(np.array([0.5, 0.3, 0.2], dtype=np.float32))
    # top_p 0.7: 0.5 kept (nothing heavier), 0.3 kept (0.5 < 0.7), 0.2 dropped (0.8 >= 0.7); renormalised 0.625 / 0.375
    for u, want in ((0.0, 0), (0.6, 0), (0.62, 0), (0.63, 1), (0.999, 1)):
        tok, keep, _ = S.sample_top_p_spec(lg, 1.0, 0.7, u)
        assert tok == want and keep.tolist() == [True, True, False]
    assert S.sample_top_p_spec(lg, 1.0, 0.0, 0.9)[1].tolist() == [True, False, False]      # at least one token stays
    assert S.sample_top_p_spec(lg, 1.0, 1.0, 0.95)[:1] == (2,)
    assert S.sample_top_p_spec(lg, 1.0, 7.0, 0.95)[1].all()                                 # top_p is clamped to 1
    # the index order of the draw, not the probability order: token 2 is the heaviest here
    lg2 = np.log(np.array([0.2, 0.3, 0.5], dtype=np.float32))
    assert [S.sample_top_p_spec(lg2, 1.0, 0.7, u)[0] for u in (0.0, 0.37, 0.38, 0.9)] == [1, 1, 2, 2]


def test_equal_masses_stay_together_and_temperature_scales():
    flat = np.zeros(10, dtype=np.float32)
    tok, keep, m = S.sample_top_p_spec(flat, 0.6, 0.05, 0.55)
    assert keep.all() and (m == 2 ** 31).all() and tok == 5
    lg = np.array([0.0, -1.0], dtype=np.float32)
    m1 = S.masses(lg, 1.0)
    m2 = S.masses(lg, 0.5)
    assert m1[0] == 2 ** 31 and abs(int(m1[1]) / 2 ** 31 - np.exp(-1.0)) < 1e-6
    assert abs(int(m2[1]) / 2 ** 31 - np.exp(-2.0)) < 1e-6
    nan_row = np.array([np.nan, 1.0, -np.inf, 1.0], dtype=np.float32)
    tok, keep, m = S.sample_top_p_spec(nan_row, 1.0, 1.0, 0.75)
    assert m.tolist() == [0, 2 ** 31, 0, 2 ** 31] and keep.tolist() == [False, True, False, True] and tok == 3


@pytest.mark.parametrize("top_p", [0.05, 0.4, 0.9, 0.999])
def test_nucleus_is_the_one_transformers_keeps(top_p):
    from transformers.generation.logits_process import TemperatureLogitsWarper, TopPLogitsWarper
    rng = np.random.default_rng(11)
    for case in range(6):
        sharp = (0.5, 1.0, 3.0)[case % 3]
        lg = (rng.standard_normal(4000) * sharp).astype(np.float32)
        t = 0.6
        scores = TopPLogitsWarper(top_p=top_p)(None, TemperatureLogitsWarper(t)(None, torch.from_numpy(lg)[None]))[0]
        hf_keep = torch.isfinite(scores).numpy()
        lit = S.nucleus_literal(lg, t, top_p)
        spec = S.nucleus_spec(S.masses(lg, t), top_p)
        assert (lit == hf_keep).all()
        assert (spec == hf_keep).all()


@pytest.mark.parametrize("top_k,top_p", [(50, 0.4), (50, 0.999), (5, 0.9), (1, 1.0), (300, 0.95)])
def test_top_k_then_nucleus_is_what_transformers_keeps(top_k, top_p):
    """The reference's generate.py passes no top_k, so transformers applies its default of 50 before the nucleus:
    TemperatureLogitsWarper -> TopKLogitsWarper -> TopPLogitsWarper.  On flat rows (where the nucleus alone would hold
    more than top_k tokens) the limit changes the kept set: both restatements must keep what the installed warpers keep."""
    from transformers.generation.logits_process import TemperatureLogitsWarper, TopKLogitsWarper, TopPLogitsWarper
    rng = np.random.default_rng(12)
    limited = 0
    for case in range(6):
        sharp = (0.3, 1.0, 3.0)[case % 3]
        lg = (rng.standard_normal(4000) * sharp).astype(np.float32)
        t = 0.6
        scores = TemperatureLogitsWarper(t)(None, torch.from_numpy(lg)[None])
        scores = TopPLogitsWarper(top_p=top_p)(None, TopKLogitsWarper(top_k=top_k)(None, scores))[0]
        hf_keep = torch.isfinite(scores).numpy()
        lit = S.nucleus_literal(lg, t, top_p, top_k)
        m = S.masses(lg, t, top_k)
        spec = S.nucleus_spec(m, top_p)
        assert (lit == hf_keep).all()
        assert (spec == hf_keep).all()
        assert int((m > 0).sum()) <= top_k          # a kept token far below the maximum may still round to mass 0
        limited += int(hf_keep.sum() < S.nucleus_literal(lg, t, top_p).sum())
    assert limited > 0 or top_k >= 300, "no case where the top-k limit bites: the test would not see it dropped"


def test_top_k_closed_forms():
    lg = np.log(np.array([0.1, 0.4, 0.2, 0.3], dtype=np.float32))
    # top_k 2 keeps tokens 1 and 3 (0.4, 0.3), renormalised 4/7 and 3/7; top_p 1.0 then keeps both
    tok = [S.sample_top_p_spec(lg, 1.0, 1.0, u, top_k=2)[0] for u in (0.0, 0.57, 0.58, 0.99)]
    assert tok == [1, 1, 3, 3]
    assert S.sample_top_p_spec(lg, 1.0, 1.0, 0.0, top_k=2)[1].tolist() == [False, True, False, True]
    # the nucleus is taken of the limited set: 0.4 / 0.7 = 0.571 >= 0.5, so top_p 0.5 keeps token 1 only
    assert S.sample_top_p_spec(lg, 1.0, 0.5, 0.9, top_k=2)[1].tolist() == [False, True, False, False]
    # without the limit 0.4 < 0.5 and the second token stays
    assert S.sample_top_p_spec(lg, 1.0, 0.5, 0.9, top_k=0)[1].tolist() == [False, True, False, True]
    # equal masses at the limit stay together; a limit of V or more is no limit
    flat = np.zeros(6, dtype=np.float32)
    assert S.sample_top_p_spec(flat, 1.0, 1.0, 0.0, top_k=2)[1].all()
    assert S.sample_top_p_spec(lg, 1.0, 1.0, 0.0, top_k=4)[1].all() and S.sample_top_p_spec(lg, 1.0, 1.0, 0.0, top_k=9)[1].all()


def test_a_row_without_a_finite_logit_is_uniform_with_and_without_the_limit():
    """All -inf (or NaN, which counts as -inf): every mass is 2^31, the nucleus is the whole row, the draw is floor(u * V)."""
    for row in (np.full(40, -np.inf, dtype=np.float32), np.full(40, np.nan, dtype=np.float32)):
        for top_k in (0, 1, 7, 39, 40):
            for u in (0.0, 0.26, 0.5, 0.999):
                tok, keep, m = S.sample_top_p_spec(row, 0.6, 0.4, u, top_k=top_k)
                assert keep.all() and (m == 2 ** 31).all() and tok == int(np.float32(u) * 40)


def test_the_draw_realises_the_renormalised_distribution():
    rng = np.random.default_rng(3)
    lg = (rng.standard_normal(50) * 2).astype(np.float32)
    t, top_p = 0.8, 0.9
    _, keep, m = S.sample_top_p_spec(lg, t, top_p, 0.0)
    want = np.where(keep, m.astype(np.float64), 0.0)
    want /= want.sum()
    n = 20000
    counts = np.zeros(50)
    for u in (np.arange(n, dtype=np.float64) + 0.5) / n:
        counts[S.sample_top_p_spec(lg, t, top_p, np.float32(u))[0]] += 1
    assert np.abs(counts / n - want).max() < 2e-4
    assert (counts[~keep] == 0).all()
