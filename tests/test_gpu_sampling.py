"""GPU parity of the top-p sampler: the drawn token must be the integer restatement's, exactly, on the same logits
and the same uniform numbers (the arithmetic is integer, so there is no tolerance)."""
import numpy as np
import pytest
import torch

from oracle import sampling as S

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _inference_mode():
    """These are inference tests: gradients off, as generate() and every serving loop run (with gradients on, a model whose
    parameters require them takes the differentiable path, in eval mode too -- tests/test_gpu_backward.py covers that)."""
    with torch.no_grad():
        yield



def F():
    import matmulfreellm_amd.functional as F_
    return F_


def _check_rows(dev, logits, temperature, top_p, u, what, top_k=0):
    got = F().sample_top_p(logits.to(dev), top_p, temperature, u.to(dev), top_k=top_k).cpu()
    want = [S.sample_top_p_spec(logits[r].float().numpy(), temperature, top_p, float(u[r]), top_k=top_k)[0]
            for r in range(logits.shape[0])]
    bad = [(r, int(got[r]), want[r]) for r in range(len(want)) if int(got[r]) != want[r]]
    print(f"{what}: {len(want)} rows, {len(bad)} differ", flush=True)
    assert not bad, (what, bad[:5])
    return got


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_tokens_equal_the_integer_restatement_at_vocabulary_32000(dev, dtype):
    g = torch.Generator().manual_seed(21)
    rows = 48
    sharp = torch.tensor([0.3, 1.0, 2.5, 6.0]).repeat(rows // 4)[:, None]
    logits = (torch.randn(rows, 32000, generator=g) * sharp).to(dtype)
    u = torch.rand(rows, generator=g)
    for temperature, top_p in ((0.6, 0.4), (1.0, 0.9), (0.25, 0.05), (1.3, 1.0)):
        _check_rows(dev, logits, temperature, top_p, u, f"{dtype} T={temperature} top_p={top_p}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_top_k_limit_before_the_nucleus(dev, dtype):
    """transformers' default top_k = 50 (what the reference's generate.py samples with) and other limits, on flat rows
    (where the nucleus alone would hold hundreds of tokens, so the limit decides), peaked rows, rows of equal logits
    (ties at the limit stay together), ragged and two-pass vocabularies, and limits of V or more (no limit)."""
    g = torch.Generator().manual_seed(31)
    rows = 32
    sharp = torch.tensor([0.05, 0.3, 1.0, 4.0]).repeat(rows // 4)[:, None]
    logits = (torch.randn(rows, 32000, generator=g) * sharp).to(dtype)
    logits[5] = 0.25                                              # every token ties
    logits[6, 100:] = -3.0                                        # 100 random heads, then one big tie
    u = torch.rand(rows, generator=g)
    for top_k, temperature, top_p in ((50, 0.6, 0.4), (50, 1.0, 1.0), (1, 0.7, 0.9), (7, 1.0, 0.95), (1000, 0.6, 0.999),
                                      (32000, 0.6, 0.4), (40000, 0.6, 0.4)):
        _check_rows(dev, logits, temperature, top_p, u, f"{dtype} top_k={top_k} T={temperature} top_p={top_p}", top_k=top_k)
    # the limit bites on the flat rows: fewer tokens can be drawn than without it
    flat = logits[0].float().numpy()
    assert S.sample_top_p_spec(flat, 0.6, 0.4, 0.0, top_k=50)[1].sum() < S.sample_top_p_spec(flat, 0.6, 0.4, 0.0)[1].sum()
    for v in (3, 33, 4097, 50257):
        lg = (torch.randn(6, v, generator=g) * 0.5).to(dtype)
        _check_rows(dev, lg, 0.8, 0.9, u[:6], f"{dtype} V={v} top_k=50", top_k=50)
    with pytest.raises(Exception):
        F().sample_top_p(logits.to(dev), 0.5, 1.0, u.to(dev), top_k=-1)


def test_ragged_vocabularies_strided_rows_and_two_passes_per_thread(dev):
    g = torch.Generator().manual_seed(22)
    for v in (1, 7, 33, 1000, 4097, 32768, 50257, 65536):
        rows = 6
        wide = torch.randn(rows, v + 5, generator=g) * 2.0
        logits = wide[:, :v]                                    # row stride v + 5: the unaligned path
        u = torch.rand(rows, generator=g)
        got = F().sample_top_p(logits.to(dev), 0.8, 0.7, u.to(dev)).cpu()
        want = [S.sample_top_p_spec(logits[r].numpy(), 0.7, 0.8, float(u[r]))[0] for r in range(rows)]
        assert got.tolist() == want, (v, got.tolist(), want)
        lb = logits.contiguous().bfloat16()
        _check_rows(dev, lb, 0.7, 0.8, u, f"V={v} bf16")


def test_edge_values_of_top_p_u_and_the_logits(dev):
    g = torch.Generator().manual_seed(23)
    logits = (torch.randn(8, 2048, generator=g) * 3).bfloat16()
    logits[1, 5] = float("nan")
    logits[2, 9] = float("inf")
    logits[3] = float("-inf")
    logits[3, 100] = 0.0
    logits[4] = 1.5                                             # every token ties: all are kept whatever top_p says
    logits[5, :] = float("nan")                                 # nothing to prefer: uniform over the row
    u = torch.tensor([0.0, 0.5, 0.99, 0.3, 0.7, 0.25, 0.99999994, 0.5])
    for top_p in (0.0, 1e-9, 0.4, 1.0, 3.0, -1.0):
        got = _check_rows(dev, logits, 0.6, top_p, u, f"edges top_p={top_p}")
        assert int(got[2]) == 9 and int(got[3]) == 100
        if top_p <= 1e-9:                                       # only the most probable tokens stay
            assert got[0] == logits[0].float().argmax()
    assert int(got[4]) == int(0.7 * 2048) and int(got[5]) == 512
    # out-of-range uniform numbers are clamped, never read past the row
    bad_u = torch.tensor([1.0, 7.0, -3.0, float("nan"), 0.5, 0.5, 0.5, 0.5])
    _check_rows(dev, logits, 0.6, 0.9, bad_u, "clamped u")
    # a row without a finite logit (all NaN, all -inf) is drawn uniformly with the top-k limit too, and always written:
    # the output buffer starts from a value no draw can produce
    logits[6] = float("-inf")
    for top_k in (1, 50, 2047):
        out = torch.full((8,), -7, dtype=torch.int64, device=dev)
        F().sample_top_p(logits.to(dev), 0.4, 0.6, u.to(dev), top_k=top_k, out=out)
        got = _check_rows(dev, logits, 0.6, 0.4, u, f"no finite logit, top_k={top_k}", top_k=top_k)
        assert torch.equal(out.cpu(), got) and int(got[5]) == 512 and int(got[6]) == int(np.float32(0.99999994) * 2048)


def test_draws_follow_the_renormalised_nucleus(dev):
    """20000 draws from one row (stratified uniforms): only kept tokens appear, with the kept masses' frequencies."""
    g = torch.Generator().manual_seed(24)
    row = (torch.randn(512, generator=g) * 2).bfloat16()
    n = 20000
    u = ((torch.arange(n, dtype=torch.float64) + 0.5) / n).float()
    got = F().sample_top_p(row[None].expand(n, -1).contiguous().to(dev), 0.9, 0.8, u.to(dev)).cpu().numpy()
    _, keep, m = S.sample_top_p_spec(row.float().numpy(), 0.8, 0.9, 0.0)
    want = np.where(keep, m.astype(np.float64), 0.0)
    want /= want.sum()
    freq = np.bincount(got, minlength=512) / n
    assert (freq[~keep] == 0).all() and np.abs(freq - want).max() < 2e-4


def test_rejected_arguments(dev):
    from matmulfreellm_amd._lib import MMFError
    logits = torch.zeros(2, 64, device=dev)
    u = torch.rand(2, device=dev)
    for bad_t in (0.0, -1.0, float("nan")):
        with pytest.raises(MMFError):
            F().sample_top_p(logits, 0.5, bad_t, u)
    with pytest.raises(MMFError):
        F().sample_top_p(logits, float("nan"), 1.0, u)
    with pytest.raises(MMFError):
        F().sample_top_p(torch.zeros(1, 70000, device=dev), 0.5, 1.0, u[:1])      # wider than the kernel's registers hold
    with pytest.raises(MMFError):
        F().sample_top_p(logits, 0.5, 1.0, u.double())
    with pytest.raises(MMFError):
        F().sample_top_p(logits.cpu(), 0.5, 1.0, u)
