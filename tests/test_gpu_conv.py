"""GPU parity of ShortConvolution (csrc/conv.hip) and of HGRNBitAttention / HGRNBitForCausalLM with use_short_conv=True:
forward, cache and step bit for bit against oracle/conv.py; backward against torch.autograd through the reference's
conv1d + silu formulation; the layer against a composition of the oracle's ops in the order of
mmfreelm/layers/hgrn_bit.py:97-139; cached decoding against the whole-sequence forward."""
import pytest
import torch

from oracle import bitlinear as ob
from oracle import conv as oc
from oracle import hgrn as oh
from oracle import norms as on

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def F():
    import matmulfreellm_amd.functional as F_
    return F_


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("btd", [(2, 11, 6), (1, 1, 64), (3, 2, 100), (2, 300, 256), (1, 3, 2048)])
@pytest.mark.parametrize("w,bias,act", [(4, False, True), (4, True, True), (2, True, False), (8, False, True)])
def test_forward_cache_and_step_are_the_oracles(dev, dtype, btd, w, bias, act):
    torch.manual_seed(5)
    b, t, d = btd
    x = torch.randn(b, t + 2, d).to(dtype)
    wt = (torch.randn(d, 1, w) * 0.5).to(dtype)
    bs = torch.randn(d).to(dtype) if bias else None
    y_ref, cache_ref = oc.short_conv_spec(x[:, :t], wt, bs, act)
    cache = torch.full((b, d, w), 7.0, dtype=dtype, device=dev)
    y = F().short_conv(x[:, :t].to(dev), wt.to(dev), bs.to(dev) if bias else None, act, cache=cache)
    assert torch.equal(y.cpu(), y_ref), (y.cpu().float() - y_ref.float()).abs().max()
    assert torch.equal(cache.cpu(), cache_ref)
    assert torch.equal(F().short_conv(x[:, :t].to(dev), wt.to(dev), bs.to(dev) if bias else None, act).cpu(), y_ref)
    full, _ = oc.short_conv_spec(x, wt, bs, act)
    for s in range(2):                                           # two steps on the cache = two more positions
        ys_ref, cache_ref = oc.short_conv_step_spec(x[:, t + s], wt, bs, cache_ref, act)
        ys = F().short_conv_step(x[:, t + s].to(dev), wt.to(dev), bs.to(dev) if bias else None, cache, act)
        assert torch.equal(ys.cpu(), ys_ref) and torch.equal(ys.cpu(), full[:, t + s]) and torch.equal(cache.cpu(), cache_ref)


def test_module_interface_and_rejections(dev):
    import matmulfreellm_amd as mm
    conv = mm.ShortConvolution(64, 4, activation="silu").to(dev, torch.bfloat16)
    assert tuple(conv.weight.shape) == (64, 1, 4) and conv.bias is None and conv.state_size == 256
    x = torch.randn(2, 5, 64, device=dev, dtype=torch.bfloat16)
    cache = torch.zeros(2, 64, 4, device=dev, dtype=torch.bfloat16)
    y = conv(x, cache)
    ref, cache_ref = oc.short_conv_spec(x.cpu(), conv.weight.detach().cpu(), None, True)
    assert torch.equal(y.cpu(), ref) and torch.equal(cache.cpu(), cache_ref)
    y1 = conv(x[:, :1], cache)                                   # one token with a cache: the step
    assert torch.equal(y1.cpu()[:, 0], oc.short_conv_step_spec(x.cpu()[:, 0], conv.weight.detach().cpu(), None, cache_ref, True)[0])
    with pytest.raises(Exception):
        F().short_conv(x, torch.randn(64, 1, 9, device=dev, dtype=torch.bfloat16))          # kernel wider than 8
    with pytest.raises(Exception):
        F().short_conv(x.cpu(), conv.weight.cpu())
    with pytest.raises(Exception):
        conv(x, cache.float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("btd", [(2, 9, 6), (3, 130, 300), (1, 2, 64)])
@pytest.mark.parametrize("w,bias,act", [(4, True, True), (3, False, False)])
def test_backward(dev, dtype, btd, w, bias, act):
    import matmulfreellm_amd as mm
    torch.manual_seed(6)
    b, t, d = btd
    x = torch.randn(b, t, d).to(dtype)
    conv = mm.ShortConvolution(d, w, bias=bias, activation="silu" if act else None)
    with torch.no_grad():
        conv.weight.copy_(torch.randn(d, 1, w) * 0.5)
    conv = conv.to(dtype)
    dy = torch.randn(b, t, d).to(dtype)
    xc = x.float().detach().clone().requires_grad_()
    wc = conv.weight.detach().float().requires_grad_()
    bc = conv.bias.detach().float().requires_grad_() if bias else None
    (oc.short_conv_literal(xc, wc, bc, act) * dy.float()).sum().backward()
    conv = conv.to(dev)
    xg = x.to(dev).detach().clone().requires_grad_()
    (conv(xg).float() * dy.to(dev).float()).sum().backward()
    tol = 1e-4 if dtype == torch.float32 else 2e-2

    def close(got, want, what):
        err = ((got.detach().double().cpu() - want.double()).abs().max() / want.double().abs().max().clamp_min(1e-30)).item()
        assert err <= tol, (what, err)
    close(xg.grad, xc.grad, "dx")
    close(conv.weight.grad, wc.grad, "dweight")
    if bias:
        close(conv.bias.grad, bc.grad, "dbias")


@pytest.mark.parametrize("share", [True, False])
def test_attention_layer_with_short_convolutions(dev, share):
    """HGRNBitAttention(use_short_conv=True) against the oracle's ops composed as mmfreelm/layers/hgrn_bit.py:97-139 reads
    (with conv(x, cache) for the call the reference gets wrong): shared kernel - the convolved hidden states feed i, f AND g;
    separate kernels - the convolutions sit behind i_proj and f_proj, g sees the plain input.  Then a cached decode step."""
    import matmulfreellm_amd as mm
    torch.manual_seed(8)
    H, B, T = 128, 2, 7
    dtype = torch.bfloat16
    attn = mm.HGRNBitAttention(hidden_size=H, num_heads=1, use_short_conv=True, conv_size=4, share_conv_kernel=share,
                               layernorm_eps=1e-6, layer_idx=1).to(dtype).eval()
    with torch.no_grad():
        attn.g_norm.weight.copy_(1 + 0.1 * torch.randn(H))
    p = {k: v.detach().clone() for k, v in attn.state_dict().items()}
    x = torch.randn(B, T + 1, H).to(dtype)
    lb = torch.rand(H) * 0.3

    def bl(v, name):
        return ob.bitlinear_spec(v, p[name + ".weight"], p[name + ".norm.weight"], eps=1e-6)

    def layer(xs):
        if share:
            hc, _ = oc.short_conv_spec(xs, p["h_conv1d.weight"], None, True)
            i, f, g_in = bl(hc, "i_proj"), bl(hc, "f_proj"), hc
        else:
            i, _ = oc.short_conv_spec(bl(xs, "i_proj"), p["i_conv1d.weight"], None, True)
            f, _ = oc.short_conv_spec(bl(xs, "f_proj"), p["f_conv1d.weight"], None, True)
            g_in = xs
        x_in, gate = oh.hgrn_gate_spec(i, f, lb, 1, None)
        t = xs.shape[1]
        o, _ = oh.recurrent_hgrn_spec(x_in.reshape(B, 1, t, H), gate.reshape(B, 1, t, H), None, True)
        o2 = on.rms_norm_swish_gate_spec(bl(g_in, "g_proj"), o.reshape(B, t, H), p["g_norm.weight"], 1e-6)
        return bl(o2, "o_proj")

    want = layer(x)
    attn = attn.to(dev)
    with torch.no_grad():
        got, _, _ = attn(x.to(dev), lower_bound=lb.to(dev))
        assert torch.equal(got.cpu(), want)
        cache = mm.RecurrentCache.from_legacy_cache([attn.init_state(B), attn.init_state(B)])    # layer_idx 1
        pre, _, cache = attn(x[:, :T].to(dev), past_key_values=cache, use_cache=True, lower_bound=lb.to(dev))
        step, _, cache = attn(x[:, T:].to(dev), past_key_values=cache, use_cache=True, lower_bound=lb.to(dev))
    assert torch.equal(pre.cpu(), want[:, :T]) and torch.equal(step.cpu(), want[:, T:])
    assert len(cache[1]) == (2 if share else 3) and cache[1][-1].dtype == torch.float32


@pytest.mark.parametrize("share", [True, False])
def test_model_with_short_convolutions_decodes_and_trains(dev, share):
    import matmulfreellm_amd as mm
    torch.manual_seed(9)
    cfg = mm.HGRNBitConfig(vocab_size=96, hidden_size=128, num_hidden_layers=2, use_short_conv=True, share_conv_kernel=share)
    model = mm.HGRNBitForCausalLM(cfg).to(torch.bfloat16).to(dev).eval()
    ids = torch.randint(0, 96, (2, 10), device=dev)
    with torch.no_grad():
        full = model(input_ids=ids, use_cache=False).logits
        out = model(input_ids=ids[:, :6], use_cache=True)
        logits = [out.logits]
        cache = out.past_key_values
        for t in range(6, 10):
            out = model(input_ids=ids[:, t:t + 1], past_key_values=cache, use_cache=True)
            cache = out.past_key_values
            logits.append(out.logits)
    assert torch.equal(torch.cat(logits, dim=1), full)           # cached decoding = the whole sequence, bit for bit
    gen = model.generate(ids[:, :6], max_new_tokens=5)
    assert gen.shape == (2, 11) and torch.equal(gen[:, 6], full[:, 5].float().argmax(-1))
    with pytest.raises(NotImplementedError):
        mm.DecodeEngine(model, 1)
    model.train()
    loss = model(input_ids=ids, labels=ids).loss
    loss.backward()
    conv = model.model.layers[0].attn.h_conv1d if share else model.model.layers[0].attn.i_conv1d
    assert torch.isfinite(loss).item() and conv.weight.grad is not None and conv.weight.grad.abs().sum().item() > 0
