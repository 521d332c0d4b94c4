"""ShortConvolution oracle (oracle/conv.py), pinned without the oracle's own arithmetic: torch's conv1d + silu (library
routines), shift / identity kernels with known answers, causality, and a step on the cache against one more position of the
whole-sequence form."""
import pytest
import torch
import torch.nn.functional as F

from oracle import conv as oc


def rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp(min=1e-30)).item()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("w,bias,act", [(4, False, True), (4, True, True), (2, True, False), (8, False, True)])
def test_spec_against_torch_conv1d(dtype, tol, w, bias, act):
    """mmfreelm/modules/convolution.py:116-131 (the branch without causal_conv1d): nn.Conv1d with padding W - 1, cut to the
    sequence, then SiLU.  The expected values come from torch's conv1d / silu in float64."""
    torch.manual_seed(1)
    b, t, d = 2, 11, 6
    x = torch.randn(b, t, d).to(dtype)
    wt = (torch.randn(d, 1, w) * 0.5).to(dtype)
    bs = torch.randn(d).to(dtype) if bias else None
    want = F.conv1d(x.double().transpose(1, 2), wt.double(), bs.double() if bias else None, padding=w - 1, groups=d)[..., :t]
    want = (F.silu(want) if act else want).transpose(1, 2)
    got, cache = oc.short_conv_spec(x, wt, bs, act)
    assert got.dtype == dtype and rel(got, want) < tol
    assert rel(oc.short_conv_literal(x.float(), wt.float(), bs.float() if bias else None, act), want) < 1e-6
    # the cache is the last W inputs, oldest first
    assert torch.equal(cache[:, :, -1], x[:, -1]) and torch.equal(cache[:, :, -w:], x[:, -w:].transpose(1, 2)[:, :, -w:])


def test_known_answers_and_causality():
    torch.manual_seed(2)
    b, t, d, w = 1, 7, 3, 4
    x = torch.randn(b, t, d)
    ident = torch.zeros(d, 1, w); ident[:, 0, -1] = 1.0          # the last tap multiplies the current input
    y, _ = oc.short_conv_spec(x, ident, None, False)
    assert torch.equal(y, x)
    shift = torch.zeros(d, 1, w); shift[:, 0, -2] = 1.0          # the tap before it: the previous input
    y, _ = oc.short_conv_spec(x, shift, None, False)
    assert torch.equal(y[:, 1:], x[:, :-1]) and y[:, 0].abs().sum().item() == 0
    oldest = torch.zeros(d, 1, w); oldest[:, 0, 0] = 2.0         # tap 0 reaches W - 1 positions back
    y, _ = oc.short_conv_spec(x, oldest, None, False)
    assert torch.equal(y[:, w - 1:], 2.0 * x[:, :t - (w - 1)]) and y[:, :w - 1].abs().sum().item() == 0
    # a channel only sees its own filter
    wt = torch.randn(d, 1, w)
    y0, _ = oc.short_conv_spec(x, wt, None, True)
    wt2 = wt.clone(); wt2[1] += 1.0
    y1, _ = oc.short_conv_spec(x, wt2, None, True)
    assert torch.equal(y0[..., 0], y1[..., 0]) and torch.equal(y0[..., 2], y1[..., 2]) and not torch.equal(y0[..., 1], y1[..., 1])
    # causality: a later input does not move an earlier output
    x2 = x.clone(); x2[:, 4] += 1.0
    y2, _ = oc.short_conv_spec(x2, wt, None, True)
    assert torch.equal(y2[:, :4], y0[:, :4]) and not torch.equal(y2[:, 4], y0[:, 4])
    # silu(0) = 0 with a zero bias: a zero input row stays zero
    assert oc.short_conv_spec(torch.zeros(1, 3, d), wt, None, True)[0].abs().sum().item() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t", [1, 2, 9])
def test_step_on_the_cache_is_one_more_position(dtype, t):
    torch.manual_seed(3)
    b, d, w = 2, 5, 4
    x = torch.randn(b, t + 1, d).to(dtype)
    wt, bs = (torch.randn(d, 1, w) * 0.5).to(dtype), torch.randn(d).to(dtype)
    full, cache_full = oc.short_conv_spec(x, wt, bs, True)
    part, cache = oc.short_conv_spec(x[:, :t], wt, bs, True)
    y, cache2 = oc.short_conv_step_spec(x[:, t], wt, bs, cache, True)
    assert torch.equal(part, full[:, :t]) and torch.equal(y, full[:, t]) and torch.equal(cache2, cache_full)
