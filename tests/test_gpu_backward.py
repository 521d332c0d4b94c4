"""GPU parity of the training side: every backward kernel, through the autograd Functions of matmulfreellm_amd.autograd and
the reference-named modules, against torch.autograd through the CPU restatement (oracle/*_literal, oracle/backward.py).
Tolerances: 1e-3 relative to the largest expected gradient for fp32 tensors, 1e-2 for bf16 (gradients have no bit-level
contract: nothing re-quantises them)."""
import pytest
import torch

from oracle import backward as obw
from oracle import hgrn as oh
from oracle import model as om
from oracle import norms as on

pytestmark = pytest.mark.gpu


def close(got, want, tol, what):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()
    print(f"{what}: max err / max |want| = {err:.3e}", flush=True)
    assert err <= tol, f"{what}: {err} > {tol}"


def tol_of(dtype):
    return 1e-3 if dtype == torch.float32 else 2e-2


def leaf(t, dev=None):
    t = t.detach().clone()
    if dev is not None:
        t = t.to(dev)
    return t.requires_grad_()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mk", [(7, 64), (33, 300), (16, 2048), (5, 5632), (9, 301)])   # 301: the element-wise access path
@pytest.mark.parametrize("residual", [False, True])
def test_rmsnorm_backward(dev, dtype, mk, residual):
    import matmulfreellm_amd as mm
    torch.manual_seed(1)
    m, k = mk
    x, r = torch.randn(m, k).to(dtype), torch.randn(m, k).to(dtype)
    w = (torch.rand(k) + 0.5).to(dtype)
    dy, dres = torch.randn(m, k).to(dtype), torch.randn(m, k).to(dtype)
    xc, rc, wc = leaf(x.float()), leaf(r.float()), leaf(w.float())
    if residual:
        y, s = on.rms_norm_literal(xc, wc, residual=rc, eps=1e-6, prenorm=True)
        ((y * dy.float()).sum() + (s * dres.float()).sum()).backward()
    else:
        (on.rms_norm_literal(xc, wc, eps=1e-6) * dy.float()).sum().backward()
    norm = mm.RMSNorm(k, eps=1e-6).to(dev, dtype)
    with torch.no_grad():
        norm.weight.copy_(w)
    xg, rg = leaf(x, dev), leaf(r, dev)
    if residual:
        y, s = norm(xg, rg, True)
        ((y.float() * dy.to(dev).float()).sum() + (s.float() * dres.to(dev).float()).sum()).backward()
        close(rg.grad, rc.grad, tol_of(dtype), "dresidual")
    else:
        (norm(xg).float() * dy.to(dev).float()).sum().backward()
    close(xg.grad, xc.grad, tol_of(dtype), "dx")
    close(norm.weight.grad, wc.grad, tol_of(dtype), "dweight")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mk", [(9, 128), (16, 2048)])
def test_gated_norm_backward(dev, dtype, mk):
    import matmulfreellm_amd as mm
    torch.manual_seed(2)
    m, k = mk
    x, o = torch.randn(m, k).to(dtype), torch.randn(m, k).to(dtype)
    w = (torch.rand(k) + 0.5).to(dtype)
    dy = torch.randn(m, k).to(dtype)
    xc, oc, wc = leaf(x.float()), leaf(o.float()), leaf(w.float())
    (on.rms_norm_swish_gate_literal(xc, oc, wc, 1e-6) * dy.float()).sum().backward()
    mod = mm.FusedRMSNormSwishGate(k, eps=1e-6).to(dev, dtype)
    with torch.no_grad():
        mod.weight.copy_(w)
    xg, og = leaf(x, dev), leaf(o, dev)
    (mod(xg, og).float() * dy.to(dev).float()).sum().backward()
    for name, got, want in (("dx", xg.grad, xc.grad), ("do", og.grad, oc.grad), ("dweight", mod.weight.grad, wc.grad)):
        close(got, want, tol_of(dtype), name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mkn", [(8, 256, 96), (40, 2048, 512), (3, 1536, 64)])
@pytest.mark.parametrize("bias", [False, True])
def test_bitlinear_backward(dev, dtype, mkn, bias):
    import matmulfreellm_amd as mm
    torch.manual_seed(3)
    m, k, n = mkn
    x = torch.randn(m, k).to(dtype)
    w = (torch.randn(n, k) * 0.02).to(dtype)
    nw = (torch.rand(k) + 0.5).to(dtype)
    b = torch.randn(n).to(dtype) if bias else None
    dout = torch.randn(m, n).to(dtype)
    xc, wc, nwc = leaf(x.float()), leaf(w.float()), leaf(nw.float())
    bc = leaf(b.float()) if bias else None
    (obw.bitlinear_ste(xc, wc, nwc, bc, eps=1e-6, weight_dtype=dtype) * dout.float()).sum().backward()
    lin = mm.FusedBitLinear(k, n, bias=bias).to(dev, dtype)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.norm.weight.copy_(nw)
        if bias:
            lin.bias.copy_(b)
    xg = leaf(x, dev)
    (lin(xg).float() * dout.to(dev).float()).sum().backward()
    # a code that sits on a rounding tie may differ between the fp32 CPU expression and the device's: a few units of
    # 1/127 in single elements of the recomputed activations, hence the wider bound on the weight gradient
    close(xg.grad, xc.grad, 2 * tol_of(dtype), "dx")
    close(lin.norm.weight.grad, nwc.grad, 2 * tol_of(dtype), "dnorm_weight")
    close(lin.weight.grad, wc.grad, 2 * tol_of(dtype), "dweight")
    if bias:
        close(lin.bias.grad, bc.grad, tol_of(dtype), "dbias")


def test_bitlinear_weight_update_is_seen_by_the_next_forward(dev):
    """The packed codes follow the latent weight: an optimiser step changes the next forward."""
    import matmulfreellm_amd as mm
    torch.manual_seed(4)
    lin = mm.FusedBitLinear(256, 64).to(dev)
    x = torch.randn(4, 256, device=dev)
    y0 = lin(x).detach().clone()
    with torch.no_grad():
        lin.weight.mul_(-1.0)
    assert torch.equal(lin(x).detach(), -y0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_backward_on_column_slices(dev, dtype):
    import matmulfreellm_amd as mm
    torch.manual_seed(5)
    y = torch.randn(6, 2 * 352).to(dtype)
    g = torch.randn(6, 352).to(dtype)
    yc = leaf(y.float())
    (on.swiglu_literal(yc[:, :352], yc[:, 352:]) * g.float()).sum().backward()
    yg = leaf(y, dev)
    (mm.swiglu(yg[:, :352], yg[:, 352:]).float() * g.to(dev).float()).sum().backward()
    close(yg.grad, yc.grad, tol_of(dtype), "d(gate, up)")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_lb", [False, True])
@pytest.mark.parametrize("d", [192, 70])                                                 # 70: the element-wise access path
def test_gate_math_backward(dev, dtype, use_lb, d):
    from matmulfreellm_amd.autograd import HGRNGateFn
    torch.manual_seed(6)
    b, t = 3, 5
    i, f = (2 * torch.randn(b, t, d)).to(dtype), (2 * torch.randn(b, t, d)).to(dtype)
    lb = torch.rand(d) * 0.5 if use_lb else None
    mask = torch.ones(b, t)
    mask[1, :2] = 0
    gx, gg = torch.randn(b, t, d).to(dtype), torch.randn(b, t, d).to(dtype)
    ic, fc = leaf(i.float()), leaf(f.float())
    lbc = leaf(lb) if use_lb else None
    xo, go = oh.hgrn_gate_literal(ic, fc, lbc, layer_idx=1, attention_mask=mask)
    ((xo * gx.float()).sum() + (go * gg.float()).sum()).backward()
    ig, fg = leaf(i, dev), leaf(f, dev)
    lbg = leaf(lb, dev) if use_lb else None
    xo2, go2 = HGRNGateFn.apply(ig, fg, lbg, mask.to(dev))
    ((xo2.float() * gx.to(dev).float()).sum() + (go2.float() * gg.to(dev).float()).sum()).backward()
    close(ig.grad, ic.grad, tol_of(dtype), "di")
    close(fg.grad, fc.grad, tol_of(dtype), "df")
    if use_lb:
        close(lbg.grad, lbc.grad, tol_of(dtype), "dlower_bound")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bhtd", [(2, 1, 70, 128), (1, 2, 33, 100), (2, 1, 1, 64), (1, 2, 130, 100), (1, 1, 301, 64),
                                  (2, 1, 1000, 192)])   # one wave; 2, 4 and 8 waves along time with ragged last segments
@pytest.mark.parametrize("with_h0", [False, True])
def test_recurrent_scan_backward(dev, dtype, bhtd, with_h0):
    import matmulfreellm_amd as mm
    torch.manual_seed(7)
    b, h, t, d = bhtd
    g = torch.sigmoid(torch.randn(b, h, t, d) + 1).to(dtype)
    x = torch.randn(b, h, t, d).to(dtype)
    h0 = torch.randn(b, h, d) if with_h0 else None
    do = torch.randn(b, h, t, d).to(dtype)
    xc, gc = leaf(x.float()), leaf(g.float())
    o, _ = oh.naive_recurrent_hgrn_literal(xc, gc, h0, False)
    (o * do.float()).sum().backward()
    xg, gg = leaf(x, dev), leaf(g, dev)
    o2, _ = mm.fused_recurrent_hgrn(xg, gg, h0.to(dev) if with_h0 else None)
    (o2.float() * do.to(dev).float()).sum().backward()
    close(xg.grad, xc.grad, tol_of(dtype), "dx")
    close(gg.grad, gc.grad, tol_of(dtype), "dg")


def test_chunk_scan_backward_log_gates(dev):
    import matmulfreellm_amd as mm
    torch.manual_seed(8)
    b, h, t, d = 2, 1, 330, 64
    g = torch.nn.functional.logsigmoid(torch.randn(b, h, t, d) + 1)
    x, do, h0 = torch.randn(b, h, t, d), torch.randn(b, h, t, d), torch.randn(b, h, d)
    xc, gc = leaf(x), leaf(g)
    o, _ = oh.naive_recurrent_hgrn_literal(xc, gc.exp(), h0, False)
    (o * do).sum().backward()
    xg, gg = leaf(x, dev), leaf(g, dev)
    o2, _ = mm.chunk_hgrn(xg, gg, h0.to(dev))
    (o2 * do.to(dev)).sum().backward()
    close(xg.grad, xc.grad, 1e-3, "dx")
    close(gg.grad, gc.grad, 1e-3, "dg (log gates)")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("smoothing,scale,zs", [(0.0, 1.0, 0.0), (0.1, 0.7, 1e-3)])
@pytest.mark.parametrize("inplace", [False, True])
def test_fused_cross_entropy_forward_and_backward(dev, dtype, smoothing, scale, zs, inplace):
    from matmulfreellm_amd.autograd import FusedCrossEntropyLoss
    torch.manual_seed(9)
    rows, v = 37, 3000
    logits = (3 * torch.randn(rows, v)).to(dtype)
    labels = torch.randint(0, v, (rows,))
    labels[5] = -100
    lc = leaf(logits.float())
    loss_c, z_c = obw.cross_entropy_ref(lc, labels, smoothing, scale, zs)
    n = (labels != -100).sum()
    (loss_c.sum() / n).backward()
    lg = leaf(logits, dev)
    crit = FusedCrossEntropyLoss(label_smoothing=smoothing, logit_scale=scale, lse_square_scale=zs, inplace_backward=inplace,
                                 return_z_loss=True)
    loss_g, z_g = crit(lg, labels.to(dev))
    close(loss_g, loss_c.sum() / n, 1e-4 if dtype == torch.float32 else 1e-2, "loss")
    if zs:
        close(z_g, z_c.sum() / n, 1e-4 if dtype == torch.float32 else 1e-2, "z loss")
    loss_g.backward()
    close(lg.grad, lc.grad, tol_of(dtype), "dlogits")
    none = FusedCrossEntropyLoss(reduction="none", label_smoothing=smoothing, logit_scale=scale, lse_square_scale=zs)(
        logits.to(dev), labels.to(dev))
    close(none, loss_c, 1e-4 if dtype == torch.float32 else 1e-2, "per-row losses")


# ------------------------------------------------------------------ the model
V, H, L = 512, 128, 2


def _model(dev, dtype, seed=0):
    import matmulfreellm_amd as mm
    params = om.init_params(V, H, L, seed=seed, dtype=dtype)
    torch.manual_seed(seed + 1)
    params["model.lower_bounds"] = (torch.randn(L, H) * 0.5).to(dtype)        # a live lower-bound schedule
    for k in list(params):
        if k.endswith("norm.weight") or ".g_norm." in k:
            params[k] = (torch.rand_like(params[k].float()) * 0.5 + 0.75).to(dtype)
    model = mm.HGRNBitForCausalLM(mm.HGRNBitConfig(vocab_size=V, hidden_size=H, num_hidden_layers=L))
    model.load_state_dict(params, strict=True)
    return model.to(device=dev, dtype=dtype), params


def test_model_training_step_matches_the_oracle(dev):
    """loss and parameter gradients of one training step (fp32) against autograd through the CPU restatement.  The
    quantisers make the two forward passes differ in a few codes, so gradients are compared by direction and size."""
    model, params = _model(dev, torch.float32)
    model.train()
    torch.manual_seed(11)
    ids = torch.randint(0, V, (2, 24))
    cparams = {k: leaf(v) for k, v in params.items()}
    loss_c = obw.model_loss(cparams, ids, ids, L)
    loss_c.backward()
    out = model(input_ids=ids.to(dev), labels=ids.to(dev))
    assert out.loss.requires_grad
    out.loss.backward()
    assert abs(out.loss.item() - loss_c.item()) <= 2e-3 * abs(loss_c.item())
    names = dict(model.named_parameters())
    checked = 0
    for k, pc in cparams.items():
        g = names[k].grad
        assert g is not None and torch.isfinite(g).all(), k
        gc = pc.grad
        if gc is None or gc.abs().max() == 0:
            continue
        cos = torch.nn.functional.cosine_similarity(g.flatten().double().cpu(), gc.flatten().double(), dim=0).item()
        ratio = (g.double().norm().cpu() / gc.double().norm()).item()
        assert cos > 0.97 and 0.9 < ratio < 1.1, (k, cos, ratio)
        checked += 1
    assert checked >= 10 * L + 3


def test_training_reduces_the_loss_and_eval_path_is_unchanged(dev):
    """A few SGD steps on one batch in bf16 lower the loss; the inference path of the trained weights still equals the
    spec oracle bit for bit (the packed codes follow the updated latent weights)."""
    model, _ = _model(dev, torch.bfloat16, seed=3)
    model.train()
    torch.manual_seed(12)
    ids = torch.randint(0, V, (4, 32), device=dev)
    opt = torch.optim.SGD(model.parameters(), lr=0.5)
    losses = []
    for _ in range(8):
        opt.zero_grad()
        loss = model(input_ids=ids, labels=ids).loss
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0] - 0.05, losses
    model.eval()
    with torch.no_grad():
        got = model(input_ids=ids[:1, :8], use_cache=False).logits.cpu()
    sd = {k: v.detach().cpu() for k, v in model.state_dict().items()}
    ref, _ = om.forward(sd, ids[:1, :8].cpu(), L, mode="spec")
    assert torch.equal(got, ref)


def test_eval_mode_gradients_equal_train_mode_gradients(dev):
    """The differentiable path is chosen by what requires a gradient, not by model.training: the reference differentiates in
    eval mode too.  Loss and every parameter gradient of an eval-mode step equal the train-mode step's bit for bit (the
    model has no dropout; the backward kernels sum in a fixed order), and with frozen parameters a gradient still reaches
    inputs_embeds (attribution)."""
    model, _ = _model(dev, torch.float32, seed=5)
    torch.manual_seed(13)
    ids = torch.randint(0, V, (2, 16), device=dev)
    grads = []
    for mode in (model.train, model.eval):
        mode()
        model.zero_grad(set_to_none=True)
        out = model(input_ids=ids, labels=ids)
        assert out.loss.requires_grad, "no graph in " + mode.__name__
        out.loss.backward()
        grads.append((out.loss.detach().clone(), {k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(grads[0][0], grads[1][0])
    assert grads[0][1].keys() == grads[1][1].keys() and len(grads[0][1]) > 10
    for k in grads[0][1]:
        assert torch.equal(grads[0][1][k], grads[1][1][k]), k
    # under no_grad the same eval-mode call builds no graph and returns the recurrent-state cache
    with torch.no_grad():
        out = model(input_ids=ids, use_cache=True)
    assert not out.logits.requires_grad and out.past_key_values is not None
    # frozen parameters, gradient with respect to the input embeddings
    for p in model.parameters():
        p.requires_grad_(False)
    emb = model.get_input_embeddings()(ids).detach().requires_grad_()
    model(inputs_embeds=emb).logits.float().square().mean().backward()
    assert emb.grad is not None and torch.isfinite(emb.grad).all() and emb.grad.abs().max() > 0
