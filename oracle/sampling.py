"""Top-p (nucleus) sampling: CPU restatement used by the tests only (test infrastructure, never the product path).

The reference samples through transformers (generate.py:11: ``model.generate(..., do_sample=True, top_p=0.4,
temperature=0.6)``): TemperatureLogitsWarper (scores / temperature), TopKLogitsWarper (the call passes no top_k, so
the default generation parameters' 50 applies: scores below the 50th largest become -inf), TopPLogitsWarper (sort
ascending, softmax, cumulative sum, drop the tokens whose cumulative probability is <= 1 - top_p, keep at least one)
and a multinomial draw from the softmax of what is left.  transformers is a third-party dependency of the reference (not vendored);
``nucleus_literal`` restates that published algorithm in float64, and tests compare it with the installed
transformers' own TopPLogitsWarper.

``sample_top_p_spec`` is the integer restatement the HIP kernel must reproduce exactly: probabilities become integer
masses (2^31 for the most probable token), the nucleus is decided on exact integer sums, and the draw is the inverse
CDF, over the kept masses in index order, of a uniform number supplied by the caller.  The random stream of
``torch.multinomial`` is not reproduced (parity of drawn tokens with the reference's stream is unpinned; the nucleus
and the distribution drawn from are pinned).
"""
import numpy as np
import torch

from .detmath import det_exp

MASS_ONE = 2147483648.0          # 2^31


def masses(logits, temperature, top_k=0):
    """uint64 array [V]: trunc(p_i * 2^31), p_i = exp(l_i - max l) with the deterministic fp32 exp, l = logits / T;
    top_k > 0: every l_i below the top_k-th largest becomes -inf first (equal values stay together)."""
    l = torch.as_tensor(logits).float() / torch.tensor(temperature, dtype=torch.float32)
    l = torch.where(torch.isnan(l), torch.full_like(l, float("-inf")), l)
    if 0 < top_k < l.shape[0]:
        kth = torch.sort(l).values[-top_k]
        l = torch.where(l >= kth, l, torch.full_like(l, float("-inf")))
    mx = l.max()
    p = torch.where(l == mx, torch.ones_like(l), det_exp(l - mx))
    m = (p * torch.tensor(MASS_ONE, dtype=torch.float32)).to(torch.float64).floor()
    return m.numpy().astype(np.uint64)


def nucleus_spec(m, top_p):
    """bool [V]: kept iff m_i > 0 and the mass of all strictly heavier tokens is below P = max(1, trunc(top_p * Z))."""
    top_p = np.float32(min(max(float(top_p), 0.0), 1.0))
    mi = m.astype(np.int64)                                    # a row's masses sum to less than 2^47
    big_p = max(1, int(np.float64(top_p) * np.float64(int(mi.sum()))))
    order = np.argsort(-mi, kind="stable")
    ms = mi[order]                                             # heaviest first
    before = np.cumsum(ms) - ms                                # mass in front of each position
    first = np.searchsorted(-ms, -ms, side="left")             # where each run of equal masses starts
    keep = np.zeros(mi.shape[0], dtype=bool)
    keep[order] = (ms > 0) & (before[first] < big_p)
    return keep


def sample_top_p_spec(logits, temperature, top_p, u, top_k=0):
    """One row: (token, keep mask, masses after the top-k limit).  u is the caller's uniform number in [0, 1) (fp32)."""
    m = masses(logits, temperature, top_k)
    keep = nucleus_spec(m, top_p)
    cum = np.cumsum(np.where(keep, m.astype(np.int64), 0))
    s = int(cum[-1])
    u = np.float32(u)
    u = u if u >= 0 else np.float32(0.0)                       # NaN and negatives draw the first kept token
    target = min(int(np.float64(u) * np.float64(s)), s - 1)
    return int(np.searchsorted(cum, target, side="right")), keep, m


def nucleus_literal(logits, temperature, top_p, top_k=0):
    """bool [V]: what TemperatureLogitsWarper + TopKLogitsWarper(top_k) + TopPLogitsWarper(top_p, min_tokens_to_keep=1)
    leave, in float64 (top_k = 0: no TopKLogitsWarper)."""
    s = np.asarray(logits, dtype=np.float64) / float(temperature)
    if 0 < top_k < s.shape[0]:
        s = np.where(s < np.sort(s)[-top_k], -np.inf, s)
    order = np.argsort(s, kind="stable")                       # ascending
    e = np.exp(s[order] - s.max())
    cum = np.cumsum(e / e.sum())
    remove = cum <= (1.0 - float(top_p))
    remove[-1:] = False
    keep = np.zeros(s.shape[0], dtype=bool)
    keep[order[~remove]] = True
    return keep
