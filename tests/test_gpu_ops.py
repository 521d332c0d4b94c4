"""GPU parity: every HIP entry point against the CPU oracle on the same seeded inputs.

Integer codes must match bit for bit.  Float outputs of kernels that follow the spec
arithmetic are compared for exact equality too (a mismatch count is reported), with the
stated tolerance (1e-2 relative in bf16, 1e-3 with fp32 tensors) as the hard bound.
"""
import numpy as np
import pytest
import torch

from oracle import bitlinear as ob
from oracle import hgrn as oh
from oracle import norms as on
from oracle import pack as op
from oracle import quant as oq

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float32, torch.float16]


def F():
    import matmulfreellm_amd.functional as F_
    return F_


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def assert_same(got, want, tol, what):
    got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape and got.dtype == want.dtype, (what, got.shape, want.shape, got.dtype, want.dtype)
    neq = (got.float() != want.float()).sum().item()
    err = rel_err(got, want)
    print(f"{what}: mismatching elements {neq}/{got.numel()}, max rel err {err:.3e}", flush=True)
    assert err <= tol, f"{what}: rel err {err} > {tol}"
    return neq


def tol_of(dtype):
    return 1e-3 if dtype == torch.float32 else 1e-2


# ------------------------------------------------------------------ weights
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(64, 256), (2048, 2048), (70, 300), (32, 128), (1, 1), (33, 129)])
def test_ternarize_pack(dev, dtype, shape):
    torch.manual_seed(1)
    w = (torch.randn(*shape) * 0.02).to(dtype)
    t_ref, deq_ref = oq.ternary_codes(w)
    pw = F().ternarize_pack(w.to(dev))
    codes = F().unpack_ternary(pw).cpu()
    assert torch.equal(codes, t_ref), f"ternary codes differ in {(codes != t_ref).sum().item()} places"
    assert pw.wdeq.cpu().item() == deq_ref.item()
    packed_ref = op.pack_ternary(t_ref.numpy())
    got = pw.packed.cpu().numpy().view(np.uint32)
    assert np.array_equal(got, packed_ref), "packed layout differs from the host restatement"


def test_ternarize_degenerate(dev):
    w = torch.zeros(32, 128, dtype=torch.bfloat16)
    pw = F().ternarize_pack(w.to(dev))
    assert F().unpack_ternary(pw).abs().sum().item() == 0
    t_ref, deq_ref = oq.ternary_codes(w)
    assert pw.wdeq.cpu().item() == deq_ref.item()


# ------------------------------------------------------------------ norms
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mk", [(1, 512), (5, 2048), (37, 5632), (3, 100), (2, 6912), (4, 16384)])
def test_rmsnorm(dev, dtype, mk):
    torch.manual_seed(2)
    m, k = mk
    x = torch.randn(m, k).to(dtype)
    w = (1 + 0.1 * torch.randn(k)).to(dtype)
    y = F().rmsnorm(x.to(dev), w.to(dev), eps=1e-6)
    assert_same(y, on.rms_norm_spec(x, w, eps=1e-6), tol_of(dtype), f"rmsnorm {dtype} {mk}")
    lit = on.rms_norm_literal(x, w, eps=1e-6, upcast=True)
    assert rel_err(y, lit) <= tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("res_fp32", [False, True])
def test_rmsnorm_residual_prenorm(dev, dtype, res_fp32):
    torch.manual_seed(3)
    x = torch.randn(2, 7, 1024).to(dtype)
    r = torch.randn(2, 7, 1024).to(torch.float32 if res_fp32 else dtype)
    w = (1 + 0.1 * torch.randn(1024)).to(dtype)
    y, ro = F().rmsnorm(x.to(dev), w.to(dev), residual=r.to(dev), eps=1e-6, prenorm=True)
    y_ref, ro_ref = on.rms_norm_spec(x, w, residual=r, eps=1e-6, prenorm=True)
    assert_same(y, y_ref, tol_of(dtype), "rmsnorm+res y")
    assert_same(ro, ro_ref, tol_of(dtype), "rmsnorm+res residual_out")
    # residual_in_fp32 without a residual
    y2, ro2 = F().rmsnorm(x.to(dev), w.to(dev), eps=1e-6, prenorm=True, residual_in_fp32=True)
    y2_ref, ro2_ref = on.rms_norm_spec(x, w, eps=1e-6, prenorm=True, residual_in_fp32=True)
    assert_same(y2, y2_ref, tol_of(dtype), "rmsnorm res_in_fp32 y")
    assert ro2.dtype == ro2_ref.dtype and torch.equal(ro2.cpu(), ro2_ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_swishgate(dev, dtype):
    torch.manual_seed(4)
    x = torch.randn(3, 11, 2048).to(dtype)
    o = (2 * torch.randn(3, 11, 2048)).to(dtype)
    w = (1 + 0.1 * torch.randn(2048)).to(dtype)
    y = F().rmsnorm_swishgate(x.to(dev), o.to(dev), w.to(dev), eps=1e-6)
    assert_same(y, on.rms_norm_swish_gate_spec(x, o, w, eps=1e-6), tol_of(dtype), f"gated norm {dtype}")
    assert rel_err(y, on.rms_norm_swish_gate_literal(x, o, w, eps=1e-6)) <= tol_of(dtype)
    # x as a column slice of a wider matrix
    wide = torch.randn(33, 3 * 2048).to(dtype)
    xs = wide[:, 2048 * 2:]
    og = torch.randn(33, 2048).to(dtype)
    wd = wide.to(dev)
    y2 = F().rmsnorm_swishgate(wd[:, 2048 * 2:], og.to(dev), w.to(dev), eps=1e-6)
    assert_same(y2, on.rms_norm_swish_gate_spec(xs.contiguous(), og, w, eps=1e-6), tol_of(dtype), "gated norm strided")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gated_norm_with_extreme_gate_values(dev, dtype):
    """A vector of sigmoids runs branch-free code after one range test of all its arguments (x >= -69); one argument below
    that, or a NaN, sends the whole vector through the general form.  Gates at and around the limit, far below it and far
    above, in rows with and without such values: every output equals the oracle's bit for bit."""
    torch.manual_seed(41)
    x = torch.randn(6, 2048).to(dtype)
    o = (2 * torch.randn(6, 2048)).to(dtype)
    o[1, 5] = -69.0
    o[1, 6] = -69.5
    o[2, 0::8] = -100.0
    o[3, 3::64] = 90.0
    o[3, 7] = -88.0
    o[4, 11] = -1e30 if dtype == torch.float32 else -3e38
    o[5, :] = torch.linspace(-120, 120, 2048).to(dtype)
    w = (1 + 0.1 * torch.randn(2048)).to(dtype)
    want = on.rms_norm_swish_gate_spec(x, o, w, eps=1e-6)
    got = F().rmsnorm_swishgate(x.to(dev), o.to(dev), w.to(dev), eps=1e-6).cpu()
    bad = ((got != want) & ~(got.isnan() & want.isnan())).sum().item()
    print(f"gated norm, extreme gates, {dtype}: {bad} of {got.numel()} outputs differ", flush=True)
    assert bad == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(dev, dtype):
    torch.manual_seed(5)
    y = (3 * torch.randn(4, 9, 2 * 1536)).to(dtype)
    g, u = y.chunk(2, -1)
    yd = y.to(dev)
    gd, ud = yd.chunk(2, -1)
    out = F().swiglu(gd, ud)
    assert_same(out, on.swiglu_spec(g, u), tol_of(dtype), f"swiglu {dtype}")
    assert rel_err(out, on.swiglu_literal(g, u)) <= tol_of(dtype)
    a, b = torch.randn(7, 13).to(dtype), torch.randn(7, 13).to(dtype)      # ragged -> scalar kernel
    assert_same(F().swiglu(a.to(dev), b.to(dev)), on.swiglu_spec(a, b), tol_of(dtype), "swiglu ragged")


# ------------------------------------------------------------------ activation codes
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mk", [(1, 2048), (64, 2048), (33, 5632), (5, 300), (4096, 2048), (130, 1536), (300, 5632), (257, 300),
                                (700, 8192)])   # more than 256 rows, tiled: several rows per workgroup
@pytest.mark.parametrize("tiled", [False, True])
def test_rmsnorm_quant_codes(dev, dtype, mk, tiled):
    torch.manual_seed(6)
    m, k = mk
    x = torch.randn(m, k).to(dtype)
    w = (1 + 0.1 * torch.randn(k)).to(dtype)
    q_ref, deq_ref, qsum_ref, _ = on.rms_norm_quant_spec(x, w, eps=1e-8)
    q, deq, qsum = F().rmsnorm_quant(x.to(dev), w.to(dev), eps=1e-8, tiled=tiled)
    if tiled:
        q = F().codes_tiled_to_rowmajor(q, m, k)
    else:
        assert q[:, k:].abs().sum().item() == 0, "padding columns must be zero"
        q = q[:, :k]
    nbad = (q.cpu() != q_ref).sum().item()
    assert nbad == 0, f"{nbad} of {q_ref.numel()} int8 codes differ"
    assert torch.equal(deq.cpu(), deq_ref)
    assert torch.equal(qsum.cpu(), qsum_ref)


def test_rmsnorm_quant_ties_and_zero_rows(dev):
    """Rows whose mean square is exactly 1 (so rstd = 1, scale = 127/127 = 1) put y*scale on exact .5 ties:
    the codes must be the round-half-to-even integers, sign-symmetric; an all-zero row gives all-zero codes."""
    k = 16384
    row = torch.zeros(k)
    vals = torch.tensor([127.0, 0.5, 1.5, 2.5, 15.0, 4.0, 2.0, 1.0, 0.5])     # sum of squares = 16384 = k
    row[:9] = vals
    x = torch.stack([row, -row, torch.zeros(k)]).float()
    q_ref, deq_ref, qsum_ref, _ = on.rms_norm_quant_spec(x, None, eps=1e-8)
    assert q_ref[0, :9].tolist() == [127, 0, 2, 2, 15, 4, 2, 1, 0]             # hand-computed known answer
    assert q_ref[1, :9].tolist() == [-127, 0, -2, -2, -15, -4, -2, -1, 0]
    for dtype in (torch.float32, torch.bfloat16):
        q, deq, qsum = F().rmsnorm_quant(x.to(dtype).to(dev), None, eps=1e-8)
        assert torch.equal(q[:, :k].cpu(), q_ref)
        assert torch.equal(deq.cpu(), deq_ref) and torch.equal(qsum.cpu(), qsum_ref)
        assert q[2].abs().sum().item() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mk", [(3, 100), (64, 2048), (33, 5632), (130, 1536)])
@pytest.mark.parametrize("bias,residual", [(False, False), (True, False), (True, True)])
def test_layernorm_quant_codes(dev, dtype, mk, bias, residual):
    """The IS_RMS_NORM = False branch (fusedbitnet.py:102-121): codes, scales and code sums bit for bit."""
    torch.manual_seed(16)
    m, k = mk
    x = (torch.randn(m, k) * 2 + 0.7).to(dtype)
    w = (1 + 0.1 * torch.randn(k)).to(dtype)
    b = (0.2 * torch.randn(k)).to(dtype) if bias else None
    r = torch.randn(m, k).to(dtype) if residual else None
    q_ref, deq_ref, qsum_ref, xs_ref = on.layer_norm_quant_spec(x, w, b, residual=r, eps=1e-8)
    got = F().rmsnorm_quant(x.to(dev), w.to(dev), residual=r.to(dev) if residual else None, eps=1e-8, prenorm=residual,
                            norm_bias=b.to(dev) if bias else None, is_rms_norm=False)
    q, deq, qsum = got[:3]
    assert q[:, k:].abs().sum().item() == 0, "padding columns must be zero"
    nbad = (q[:, :k].cpu() != q_ref).sum().item()
    assert nbad == 0, f"{nbad} of {q_ref.numel()} int8 codes differ"
    assert torch.equal(deq.cpu(), deq_ref) and torch.equal(qsum.cpu(), qsum_ref)
    if residual:
        assert torch.equal(got[3].cpu(), xs_ref.to(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [2, 200])
def test_layer_norm_linear_quant_fn_layernorm_form(dev, dtype, m):
    """layer_norm_linear_quant_fn(..., is_rms_norm=False) with a norm bias (fusedbitnet.py:513-536) against the oracle,
    bit for bit; it has no backward here and says so; a norm bias on the RMSNorm form is refused."""
    import matmulfreellm_amd as mm
    from matmulfreellm_amd.bitlinear import layer_norm_linear_quant_fn
    torch.manual_seed(17)
    k, n = 512, 192
    x = (torch.randn(m, k) + 0.5).to(dtype)
    w = (torch.randn(n, k) * 0.02).to(dtype)
    nw, nb = (1 + 0.1 * torch.randn(k)).to(dtype), (0.1 * torch.randn(k)).to(dtype)
    lb = (0.1 * torch.randn(n)).to(dtype)
    ref = ob.bitlinear_spec(x, w, nw, bias=lb, eps=1e-6, norm_bias=nb, is_rms_norm=False)
    out = layer_norm_linear_quant_fn(x.to(dev), nw.to(dev), nb.to(dev), w.to(dev), lb.to(dev), eps=1e-6, is_rms_norm=False)
    assert assert_same(out, ref, tol_of(dtype), f"LayerNorm-form BitLinear {dtype} M={m}") == 0
    with pytest.raises(NotImplementedError):
        layer_norm_linear_quant_fn(x.to(dev).requires_grad_(), nw.to(dev), nb.to(dev), w.to(dev), None, is_rms_norm=False)
    with pytest.raises(NotImplementedError):
        layer_norm_linear_quant_fn(x.to(dev), nw.to(dev), nb.to(dev), w.to(dev), None, is_rms_norm=True)


# ------------------------------------------------------------------ BitLinear
def _bitlinear_case(dev, dtype, m, k, n, path, bias=False, seed=7):
    torch.manual_seed(seed)
    x = torch.randn(m, k).to(dtype)
    w = (torch.randn(n, k) * 0.02).to(dtype)
    nw = (1 + 0.1 * torch.randn(k)).to(dtype)
    b = (0.1 * torch.randn(n)).to(dtype) if bias else None
    ref = ob.bitlinear_spec(x, w, nw, bias=b, eps=1e-8)
    pw = F().ternarize_pack(w.to(dev))
    out = F().bitlinear(x.to(dev), nw.to(dev), pw, bias=b.to(dev) if bias else None, eps=1e-8, path=path)
    neq = assert_same(out, ref, tol_of(dtype), f"bitlinear[{path}] {dtype} M={m} K={k} N={n}")
    assert neq == 0, "integer-exact contraction must reproduce the spec bit for bit"
    lit = ob.bitlinear_fused_literal(x, w, nw, bias=b, eps=1e-8)
    assert rel_err(out, lit) <= tol_of(dtype), "float-dequant reference formulation"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mkn", [(1, 2048, 2048), (1, 512, 3072), (3, 5632, 2048), (1, 300, 70), (2, 6912, 2560),
                                 (1, 5632, 2048), (1, 1024, 3200), (1, 8192, 96), (2, 384, 1504), (1, 301, 70), (2, 6913, 64)])
def test_bitlinear_gemv(dev, dtype, mkn):
    _bitlinear_case(dev, dtype, *mkn, path="gemv")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mkn", [(1, 2048, 2048), (16, 2048, 6144), (64, 5632, 2048), (33, 300, 70), (128, 2560, 512),
                                 (200, 1536, 512), (300, 512, 3072), (1000, 2048, 1024)])
def test_bitlinear_mfma(dev, dtype, mkn):
    _bitlinear_case(dev, dtype, *mkn, path="mfma")


def test_bitlinear_bias_and_known_answers(dev):
    _bitlinear_case(dev, torch.bfloat16, 1, 2048, 512, "gemv", bias=True)
    _bitlinear_case(dev, torch.bfloat16, 40, 2048, 512, "mfma", bias=True)


@pytest.mark.parametrize("config,m,k,n", [(0, 300, 1024, 640), (1, 300, 1024, 640), (0, 20, 2048, 512), (1, 64, 2048, 512),
                                          (5, 32, 2048, 640), (5, 7, 5632, 2048), (5, 1, 300, 70), (5, 64, 2048, 6144),
                                          (5, 40, 5632, 2048), (5, 64, 8192, 96), (5, 33, 6912, 2560), (5, 300, 1024, 648),
                                          (15, 520, 2048, 1032), (15, 300, 128, 640), (15, 300, 256, 648), (16, 300, 1152, 640),
                                          (15, 4096, 2048, 1024), (16, 70, 384, 100), (15, 300, 1024, 644), (16, 300, 1024, 648),
                                          (16, 200, 128, 520), (-1, 4096, 512, 2048), (-1, 100, 512, 256), (-1, 40, 8320, 96),
                                          (17, 300, 1152, 640), (17, 520, 2048, 1032), (17, 4096, 2048, 1024), (17, 512, 256, 648),
                                          (17, 70, 384, 100), (16, 1024, 256, 520), (15, 2048, 256, 300), (17, 1000, 128, 1600)])
def test_bitlinear_mfma_all_tile_configs(dev, config, m, k, n):
    """Every tile shape of the matrix-core contraction (0/1 register-staged, 5 the weight-stream kernel,
    15/16/17 DMA-staged; ragged M, K, N; one and two k-blocks; tile-row counts that do and do not divide by the
    8 XCDs, which selects the tile order)."""
    torch.manual_seed(8)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) * 0.02).bfloat16()
    nw = torch.ones(k).bfloat16()
    ref = ob.bitlinear_spec(x, w, nw, eps=1e-8)
    pw = F().ternarize_pack(w.to(dev))
    q, deq, qsum = F().rmsnorm_quant(x.to(dev), nw.to(dev), eps=1e-8, tiled=True)
    out = F().bitlinear_mfma(q, deq, qsum, pw, m, torch.bfloat16, config=config)
    assert assert_same(out, ref, 1e-2, f"mfma config {config} M={m} K={k} N={n}") == 0


def test_bitlinear_full_size_gate_proj(dev):
    """The 1.3B gate projection at prefill size, M=4096, K=2048, N=11264 against the exact integer accumulator on the device
    (int64 matmul of the oracle's codes is too slow on CPU at this size, so the check is
    torch's own integer matmul in fp64 on the GPU: exact for |acc| < 2**53)."""
    torch.manual_seed(9)
    m, k, n = 4096, 2048, 11264
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) * 0.02).bfloat16()
    nw = torch.ones(k).bfloat16()
    q_ref, deq_ref, _, _ = on.rms_norm_quant_spec(x, nw, eps=1e-8)
    t_ref, wdeq_ref = oq.ternary_codes(w)
    pw = F().ternarize_pack(w.to(dev))
    out = F().bitlinear(x.to(dev), nw.to(dev), pw, eps=1e-8, path="mfma")
    acc = (q_ref.to(dev).double() @ t_ref.to(dev).double().t())
    ref = ((acc.float() * deq_ref.to(dev).reshape(-1, 1)) * wdeq_ref.to(dev)).bfloat16()
    assert torch.equal(out, ref), f"{(out != ref).sum().item()} outputs differ"


# ------------------------------------------------------------------ HGRN
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bhtd", [(2, 1, 64, 128), (1, 2, 200, 100), (2, 1, 1, 64), (1, 1, 1030, 256), (3, 1, 65, 70)])
@pytest.mark.parametrize("with_h0", [False, True])
def test_hgrn_recurrent(dev, dtype, bhtd, with_h0):
    torch.manual_seed(10)
    b, h, t, d = bhtd
    g = torch.sigmoid(torch.randn(b, h, t, d) + 2).to(dtype)
    x = ((1 - g.float()) * torch.randn(b, h, t, d)).to(dtype)
    h0 = torch.randn(b, h, d) if with_h0 else None
    o_ref, ht_ref = oh.recurrent_hgrn_spec(x, g, h0, True)
    o, ht = F().hgrn_recurrent(x.to(dev), g.to(dev), h0.to(dev) if with_h0 else None, True)
    assert assert_same(o, o_ref, tol_of(dtype), f"recurrent {dtype} {bhtd}") == 0
    assert torch.equal(ht.cpu(), ht_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bhtd", [(2, 1, 64, 128), (1, 2, 200, 100), (2, 1, 1, 64), (1, 1, 1030, 256), (1, 1, 4100, 192),
                                  (2, 2, 777, 64), (1, 1, 16384, 128)])
@pytest.mark.parametrize("chunk", [64, 16, 7, 48, 1])
def test_hgrn_chunk(dev, dtype, bhtd, chunk):
    torch.manual_seed(11)
    b, h, t, d = bhtd
    z = torch.randn(b, h, t, d) + 2
    g = torch.nn.functional.logsigmoid(z).to(dtype)
    x = torch.randn(b, h, t, d).to(dtype)
    h0 = torch.randn(b, h, d)
    o_ref, ht_ref = oh.chunk_hgrn_spec(x, g, h0, True, chunk=chunk)
    o, ht = F().hgrn_chunk(x.to(dev), g.to(dev), h0.to(dev), True, chunk_size=chunk)
    assert_same(o, o_ref, tol_of(dtype), f"chunk {dtype} {bhtd} c{chunk}")
    assert rel_err(ht, ht_ref) <= 1e-3
    # the time axis is cut into parallel segments exactly when batch * channel blocks leave CUs idle
    lib = F().L.load()
    nws = lib.mmf_hgrn_chunk_workspace_bytes(b * h, t, d, chunk)
    assert (nws > 0) == (b * h * -(-d // 64) < 256 and t // (4 * min(64 // chunk, 8) * chunk) >= 2)
    # without an initial state, and without asking for the final one
    o2, none = F().hgrn_chunk(x.to(dev), g.to(dev), None, False, chunk_size=chunk)
    o2_ref, _ = oh.chunk_hgrn_spec(x, g, None, False, chunk=chunk)
    assert none is None
    assert_same(o2, o2_ref, tol_of(dtype), f"chunk without state {dtype} {bhtd} c{chunk}")
    # the chunked and the sequential form agree (g_lin = exp(g_log))
    o_seq, _ = oh.recurrent_hgrn_spec(x, g.float().exp().to(dtype) if dtype == torch.float32 else g.float().exp(), h0, True) \
        if dtype == torch.float32 else (None, None)
    if o_seq is not None:
        assert rel_err(o, o_seq) <= 1e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_lb", [False, True])
def test_hgrn_gate_and_step(dev, dtype, use_lb):
    torch.manual_seed(12)
    b, t, d = 3, 5, 512
    wide = (2 * torch.randn(b, t, 3 * d)).to(dtype)
    i, f = wide[..., :d], wide[..., d:2 * d]
    lb = torch.rand(d) * 0.5 if use_lb else None
    mask = torch.ones(b, t)
    mask[0, :2] = 0
    x_ref, g_ref = oh.hgrn_gate_spec(i, f, lb, layer_idx=1, attention_mask=mask)
    wd = wide.to(dev)
    xg, gg = F().hgrn_gate(wd[..., :d], wd[..., d:2 * d], lb.to(dev) if use_lb else None, mask.to(dev))
    assert assert_same(xg, x_ref, tol_of(dtype), "gate x") == 0
    assert assert_same(gg, g_ref, tol_of(dtype), "gate g") == 0
    x_lit, g_lit = oh.hgrn_gate_literal(i, f, lb.to(dtype) if use_lb else None, 1, mask.to(dtype))
    assert rel_err(xg, x_lit) <= 2e-2 and rel_err(gg, g_lit) <= 2e-2
    # one decode step == gate + one recurrence step
    state = torch.randn(b, d)
    i1, f1 = wide[:, 0, :d], wide[:, 0, d:2 * d]
    x1, g1 = oh.hgrn_gate_spec(i1, f1, lb, layer_idx=1)
    h_ref = g1.float() * state + x1.float()
    st = state.clone().to(dev)
    o = F().hgrn_step(wd[:, 0, :d], wd[:, 0, d:2 * d], st, lb.to(dev) if use_lb else None)
    assert torch.equal(st.cpu(), h_ref)
    assert torch.equal(o.cpu(), h_ref.to(dtype))


def test_embedding_and_argmax(dev):
    torch.manual_seed(13)
    table = torch.randn(1000, 512).bfloat16()
    ids = torch.randint(0, 1000, (3, 7))
    out = F().embedding(table.to(dev), ids.to(dev))
    assert torch.equal(out.cpu(), table[ids])
    logits = torch.randn(5, 32000).bfloat16()
    logits[0, 100] = logits[0, 31000] = 50.0       # exact tie -> lowest index
    logits[1, :] = 0.0
    am = F().argmax(logits.to(dev)).cpu()
    assert am[0].item() == 100 and am[1].item() == 0
    for r in range(2, 5):
        row = logits[r].float()
        assert am[r].item() == int((row == row.max()).nonzero()[0])
    # ragged and wide rows (element path, more than one 32768-element sweep), fp32 / fp16 tables, NaNs never win
    for dtype, v, h in ((torch.float32, 70001, 36), (torch.float16, 32768 + 8, 72), (torch.bfloat16, 301, 7)):
        table = torch.randn(50, h).to(dtype)
        ids = torch.randint(0, 50, (2, 3))
        assert torch.equal(F().embedding(table.to(dev), ids.to(dev)).cpu(), table[ids])
        logits = torch.randn(3, v).to(dtype)
        logits[0, v - 1] = 60.0                     # the last element of the row wins
        logits[1, 5] = float("nan")
        logits[2, :] = float("nan")                 # nothing comparable: index 0
        am = F().argmax(logits.to(dev)).cpu()
        row1 = logits[1].float().nan_to_num(nan=-float("inf"))
        assert am.tolist() == [v - 1, int(row1.argmax()), 0], (dtype, v, am.tolist())


@pytest.mark.parametrize("m", [5, 300])
@pytest.mark.parametrize("k", [2048, 301, 5632, 9000, 3072])
@pytest.mark.parametrize("pro", [1, 2, 4, 5])
def test_fused_quantiser_equals_the_separate_ops(dev, m, k, pro):
    """mmf_rmsnorm_quant_fused through the C ABI (vector and ragged-row builds; one row per workgroup for
    decode-sized M, 2 / 4 / 8 rows per workgroup above 256 rows) against the chain of separately validated
    ops it replaces: identical codes, scales, code sums."""
    import matmulfreellm_amd._lib as L_
    lib = L_.load()
    torch.manual_seed(20 + pro)
    dt = torch.bfloat16
    x = torch.randn(m, k).to(dt).to(dev)
    aux = torch.randn(m, k).to(dt).to(dev)
    w1 = (1 + 0.1 * torch.randn(k)).to(dt).to(dev)
    nw = (1 + 0.1 * torch.randn(k)).to(dt).to(dev)
    if pro == 1:
        v = F().rmsnorm(x, w1, eps=1e-6)
    elif pro == 2:
        v, res = F().rmsnorm(x, w1, residual=aux, eps=1e-6, prenorm=True)
    elif pro == 4:
        v = F().swiglu(x, aux)
    else:
        v = F().rmsnorm_swishgate(x, aux, w1, eps=1e-6)
    q_ref, deq_ref, qsum_ref = F().rmsnorm_quant(v, nw, eps=1e-8, tiled=True)
    q = torch.empty_like(q_ref)
    deq, qsum = torch.empty_like(deq_ref), torch.empty_like(qsum_ref)
    res_out = torch.empty_like(x)
    rc = lib.mmf_rmsnorm_quant_fused(pro, x.data_ptr(), k, aux.data_ptr(), k, None, 0, res_out.data_ptr() if pro == 2 else None,
                                     w1.data_ptr() if pro != 4 else None, 1e-6, nw.data_ptr(), 1e-8, None, None, q.data_ptr(),
                                     deq.data_ptr(), qsum.data_ptr(), m, k, L_.dtype_id(dt), L_.dtype_id(dt), L_.stream())
    assert rc == 0
    assert torch.equal(F().codes_tiled_to_rowmajor(q, m, k), F().codes_tiled_to_rowmajor(q_ref, m, k))
    assert torch.equal(deq, deq_ref) and torch.equal(qsum, qsum_ref)
    if pro == 2:
        assert torch.equal(res_out, res)


@pytest.mark.parametrize("m", [3, 40])
@pytest.mark.parametrize("k", [512, 300])
@pytest.mark.parametrize("kind", ["norm", "resnorm", "gatednorm", "swiglu"])
def test_bitlinear_prologue_equals_the_separate_ops(dev, m, k, kind):
    """functional.bitlinear(..., prologue=...) — fused GEMV launch for M <= 8, fused quantiser + matrix cores
    above — against the separately validated op followed by a plain BitLinear; operands are column slices of
    wider tensors as in the model (stacked projections), with and without a fused residual add."""
    torch.manual_seed(31)
    dt, n = torch.bfloat16, 96
    wide = torch.randn(m, 2 * k + 8).to(dt).to(dev)
    x, aux = wide[:, :k], wide[:, k + 8:2 * k + 8]              # row stride 2k+8, second operand offset by 8 elements
    w1 = (1 + 0.1 * torch.randn(k)).to(dt).to(dev)
    nw = (1 + 0.1 * torch.randn(k)).to(dt).to(dev)
    pw = F().ternarize_pack((torch.randn(n, k) * 0.02).to(dt).to(dev))
    addend = torch.randn(m, n).to(dt).to(dev)
    if kind == "norm":
        v, pro = F().rmsnorm(x.contiguous(), w1, eps=1e-6), ("norm", w1, 1e-6)
    elif kind == "resnorm":
        v, res = F().rmsnorm(x.contiguous(), w1, residual=aux.contiguous(), eps=1e-6, prenorm=True)
        pro = ("resnorm", aux, w1, 1e-6)
    elif kind == "gatednorm":
        v, pro = F().rmsnorm_swishgate(x.contiguous(), aux.contiguous(), w1, eps=1e-6), ("gatednorm", aux, w1, 1e-6)
    else:
        v, pro = F().swiglu(x, aux), ("swiglu", aux)
    for add in (None, addend):
        want = F().bitlinear(v, nw, pw, eps=1e-8, addend=add)
        got = F().bitlinear(x, nw, pw, eps=1e-8, addend=add, prologue=pro)
        if kind == "resnorm":
            got, res_got = got
            assert torch.equal(res_got, res)
        assert torch.equal(got, want), f"{kind} M={m} K={k} addend={'yes' if add is not None else 'no'}"


def test_fp16_outputs_are_rounded_fp32_results(dev):
    """fp16 outputs at scale (2 M elements per op): every output is the fp32 result of the last operation rounded
    once more to fp16, as the separately rounded operations of the reference give it -- not the exact product
    rounded once (what a fused multiply-convert instruction returns; the two differ on about 1 output in 10^5,
    exactly where the fp32 product lands on an fp16 tie)."""
    torch.manual_seed(40)
    x = torch.randn(1024, 2048).half()
    o = (2 * torch.randn(1024, 2048)).half()
    w = (1 + 0.1 * torch.randn(2048)).half()
    y = F().rmsnorm_swishgate(x.to(dev), o.to(dev), w.to(dev), eps=1e-6).cpu()
    assert torch.equal(y, on.rms_norm_swish_gate_spec(x, o, w, eps=1e-6))
    y = F().rmsnorm(x.to(dev), w.to(dev), eps=1e-6).cpu()
    assert torch.equal(y, on.rms_norm_spec(x, w, eps=1e-6))
    z = F().swiglu(x.to(dev), o.to(dev)).cpu()
    assert torch.equal(z, on.swiglu_spec(x, o))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k,i", [(4096, 2048, 5632), (513, 512, 96), (70, 640, 32), (1000, 2560, 6912), (64, 128, 8000)])
def test_mfma_swiglu_epilogue_equals_contraction_then_swiglu(dev, dtype, m, k, i):
    """mmf_bitlinear_mfma_swiglu against the two ops it folds together (each checked against the oracle above): the
    contraction on the stacked [gate; up] weight, then swiglu on the two halves."""
    g = torch.Generator(device=dev).manual_seed(63)
    x = torch.randn(m, k, generator=g, device=dev).to(dtype)
    nw = (1 + 0.1 * torch.randn(k, generator=g, device=dev)).to(dtype)
    pw = F().ternarize_pack((torch.randn(2 * i, k, generator=g, device=dev) * 0.02).to(dtype))
    q, deq, qsum = F().rmsnorm_quant(x, nw, eps=1e-8, tiled=True)[:3]
    full = F().bitlinear_mfma(q, deq, qsum, pw, m, dtype)
    want = F().swiglu(full[:, :i], full[:, i:])
    got = F().bitlinear_mfma_swiglu(q, deq, qsum, pw, m, dtype)
    assert got.shape == (m, i) and torch.equal(got, want)


def test_mfma_swiglu_rejects_what_it_cannot_run(dev):
    from matmulfreellm_amd._lib import load
    lib = load()
    z = torch.zeros(1 << 16, device=dev)
    p = z.data_ptr()
    call = lambda n, ldo, out=p, seg=32: lib.mmf_bitlinear_mfma_swiglu(p, p, p, p, p, seg, out, ldo, 8, 128, n, 1, None)
    assert call(96, 48) == -1           # the two halves are not whole 32-row blocks
    assert call(128, 32) == -1          # rows of the result overlap
    assert call(128, 68) == -3          # rows of the result are not 16-byte aligned
    assert call(128, 64, out=p + 2) == -3
    assert call(128, 64, seg=48) == -1
    assert call(128, 64, out=None) == -1


def test_short_forms_equal_their_definitions_for_every_float(dev):
    """The kernels scale exp's result with one ldexp and take reciprocals, square roots and the quantiser's 127 / amax from
    the hardware approximations plus Newton steps; the CPU restatement follows the defining sequences (two scaling
    multiplications, correctly rounded division and square root).  All 2^32 arguments go through both on the device: not
    one may differ."""
    import matmulfreellm_amd._lib as L
    lib = L.load()
    counts = torch.zeros(7, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_diag_check_exact_forms(counts.data_ptr(), L.stream()), "mmf_diag_check_exact_forms")
    torch.cuda.synchronize()
    *bad, seen, bad_mid = counts.tolist()
    print(f"exact forms over {seen} arguments: differing results for exp / sigmoid / 1/x / sqrt / 127/x: {bad}; "
          f"branch-free sigmoid on x >= -69: {bad_mid}", flush=True)
    assert seen == 1 << 32 and bad == [0] * 5 and bad_mid == 0
