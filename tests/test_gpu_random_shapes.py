"""GPU parity on seeded random shapes: the shapes the hand-picked cases of test_gpu_ops.py do not name (odd row counts,
K and N that are not multiples of anything, both contraction paths, every dtype).  Each case is checked against the
CPU oracle exactly as its hand-picked sibling is."""
import random

import numpy as np
import pytest
import torch

from oracle import hgrn as oh
from oracle import norms as on
from oracle import sampling as osamp
from test_gpu_ops import DTYPES, F, _bitlinear_case, assert_same, tol_of

pytestmark = pytest.mark.gpu


def _cases(seed, n, gen):
    rnd = random.Random(seed)
    return [gen(rnd) for _ in range(n)]


def _pick_dim(rnd, hi):
    """Mostly ragged sizes, sometimes a multiple of 128 or a power of two, sometimes tiny."""
    kind = rnd.random()
    if kind < 0.15:
        return rnd.choice([1, 2, 3, 7, 8, 9, 31, 32, 33])
    if kind < 0.35:
        return min(hi, 128 * rnd.randint(1, max(1, hi // 128)))
    return rnd.randint(1, hi)


BITLINEAR = _cases(101, 36, lambda r: (r.choice(DTYPES), _pick_dim(r, 260), _pick_dim(r, 3000), _pick_dim(r, 1500),
                                       r.random() < 0.3))


@pytest.mark.parametrize("case", BITLINEAR, ids=lambda c: f"{str(c[0]).split('.')[-1]}-{c[1]}x{c[2]}x{c[3]}{'-bias' if c[4] else ''}")
def test_bitlinear_random_shapes(dev, case):
    dtype, m, k, n, bias = case
    _bitlinear_case(dev, dtype, m, k, n, path=None, bias=bias, seed=1000 + m + k + n)
    if m <= 8:                                                 # the small-M problem through the matrix cores too
        _bitlinear_case(dev, dtype, m, k, n, path="mfma", bias=bias, seed=2000 + m + k + n)


QUANT = _cases(102, 24, lambda r: (r.choice(DTYPES), _pick_dim(r, 400), _pick_dim(r, 9000), r.random() < 0.5, r.random() < 0.4))


@pytest.mark.parametrize("case", QUANT, ids=lambda c: f"{str(c[0]).split('.')[-1]}-{c[1]}x{c[2]}-{'tiled' if c[3] else 'rows'}{'-res' if c[4] else ''}")
def test_rmsnorm_quant_random_shapes(dev, case):
    dtype, m, k, tiled, with_res = case
    torch.manual_seed(3000 + m + k)
    x = (torch.randn(m, k) * (0.2 + 3 * torch.rand(m, 1))).to(dtype)
    w = (1 + 0.2 * torch.randn(k)).to(dtype)
    res = torch.randn(m, k).to(dtype) if with_res else None
    q_ref, deq_ref, qsum_ref, _ = on.rms_norm_quant_spec(x, w, residual=res, eps=1e-8)
    out = F().rmsnorm_quant(x.to(dev), w.to(dev), residual=res.to(dev) if with_res else None, eps=1e-8, tiled=tiled)
    q, deq, qsum = out[:3]
    if tiled:
        q = F().codes_tiled_to_rowmajor(q, m, k)
    q = q.reshape(m, -1)[:, :k].cpu()
    assert torch.equal(q, q_ref), f"{(q != q_ref).sum().item()} codes differ"
    assert torch.equal(deq.cpu(), deq_ref) and torch.equal(qsum.cpu(), qsum_ref)


SCAN = _cases(103, 16, lambda r: (r.choice(DTYPES), r.randint(1, 5), r.randint(1, 3), _pick_dim(r, 700), _pick_dim(r, 300),
                                  r.random() < 0.5))


@pytest.mark.parametrize("case", SCAN, ids=lambda c: f"{str(c[0]).split('.')[-1]}-{c[1]}x{c[2]}x{c[3]}x{c[4]}{'-h0' if c[5] else ''}")
def test_hgrn_recurrent_random_shapes(dev, case):
    dtype, b, h, t, d, with_h0 = case
    torch.manual_seed(4000 + t + d)
    g = torch.sigmoid(torch.randn(b, h, t, d) + 2).to(dtype)
    x = ((1 - g.float()) * torch.randn(b, h, t, d)).to(dtype)
    h0 = torch.randn(b, h, d) if with_h0 else None
    o_ref, ht_ref = oh.recurrent_hgrn_spec(x, g, h0, True)
    o, ht = F().hgrn_recurrent(x.to(dev), g.to(dev), h0.to(dev) if with_h0 else None, True)
    assert assert_same(o, o_ref, tol_of(dtype), f"recurrent {case}") == 0
    assert torch.equal(ht.cpu(), ht_ref)


SAMPLE = _cases(104, 16, lambda r: (r.choice(DTYPES), r.randint(1, 5), _pick_dim(r, 65536), r.choice([0.05, 0.4, 0.9, 1.0]),
                                    r.choice([0.3, 0.6, 1.0, 2.0]), r.choice([0.5, 2.0, 8.0])))


@pytest.mark.parametrize("case", SAMPLE, ids=lambda c: f"{str(c[0]).split('.')[-1]}-{c[1]}x{c[2]}-p{c[3]}-T{c[4]}-s{c[5]}")
def test_sample_top_p_random_shapes(dev, case):
    dtype, rows, v, top_p, temperature, sharp = case
    g = torch.Generator().manual_seed(5000 + v)
    logits = (torch.randn(rows, v, generator=g) * sharp).to(dtype)
    u = torch.rand(rows, generator=g)
    got = F().sample_top_p(logits.to(dev), top_p, temperature, u.to(dev)).cpu().tolist()
    want = [osamp.sample_top_p_spec(logits[r].float().numpy(), temperature, top_p, float(u[r]))[0] for r in range(rows)]
    assert got == want


MODELS = _cases(105, 24, lambda r: (r.choice([torch.bfloat16, torch.float32, torch.float16]), r.choice([128, 256, 384, 640]), r.randint(1, 3),
                                    r.choice([517, 1000, 4099, 32]), r.choice([1, 1, 2, 5, 9, 20]), r.randint(1, 40)))


@pytest.mark.parametrize("case", MODELS, ids=lambda c: f"{str(c[0]).split('.')[-1]}-H{c[1]}-L{c[2]}-V{c[3]}-B{c[4]}-T{c[5]}")
def test_model_greedy_random_configurations(dev, case):
    """Small random model configurations (ragged vocabularies, 1-3 layers, batches on every decode path): prefill +
    greedy tokens equal the oracle's on the module path and through the decode engine's graph."""
    import matmulfreellm_amd as mm
    from oracle import model as om
    dtype, hidden, layers, vocab, batch, t = case
    params = om.init_params(vocab, hidden, layers, seed=7, dtype=dtype)
    cfg = mm.HGRNBitConfig(vocab_size=vocab, hidden_size=hidden, num_hidden_layers=layers)
    model = mm.HGRNBitForCausalLM(cfg)
    model.load_state_dict(params, strict=True)
    model = model.to(device=dev, dtype=dtype).eval()
    model.generation_config.eos_token_id = None                # tiny vocabularies hit the default end-of-sequence id (2)
    torch.manual_seed(6000 + hidden + t)
    ids = torch.randint(0, vocab, (batch, t))
    n_new = 5
    ref_toks, _ = om.greedy(params, ids, layers, n_new, mode="spec")
    for use_graph in (False, True):
        got = model.generate(ids.to(dev), max_new_tokens=n_new, use_graph=use_graph).cpu()
        assert torch.equal(got[:, t:], ref_toks), (use_graph, got[:, t:].tolist(), ref_toks.tolist())
