"""GPU parity at the benchmark configurations' own sizes, against the CPU oracle (spec arithmetic, bit for bit).

  config 2  single BitLinear, bf16: M = 4096 at 5632 -> 2048 (down_proj) and M = 1 / 64 at 2048 -> 11264 and 5632 -> 2048
  config 3  HGRN recurrence B = 8, T = 2048, D = 2048: recurrent (bit-exact), chunk 64 (tolerance), decode step B = 64
  config 4  1.3B-shape model: greedy decode at batch 1 (resident launch and launch chain), 16 and 64 -- tokens and
            every step's logits -- and the 8 x 2048 prefill (last-position logits and final states of two rows)
  config 5  2.7B-shape model, 512-token prompt, batch 128: two rows of the batch against the oracle

The oracle runs on the host cores (fp32 BLAS on integer codes: exact), so the model cases keep the token counts
the oracle sees to a few thousand: short prompts for the decode cases; two of the batch's rows where the batch is
large (rows are independent; the GPU still runs the whole batch).
"""
import pytest
import torch

from oracle import hgrn as oh
from oracle import model as om
from oracle import norms as on
from oracle import quant as oq

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


# ------------------------------------------------------------------ config 2
def _bitlinear_case(dev, m, k, n, seed, path=None):
    torch.manual_seed(seed)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) * 0.02).bfloat16()
    nw = torch.ones(k).bfloat16()
    q_ref, deq_ref, _, _ = on.rms_norm_quant_spec(x, nw, eps=1e-8)
    t_ref, wdeq_ref = oq.ternary_codes(w)
    pw = F().ternarize_pack(w.to(dev))
    assert torch.equal(F().unpack_ternary(pw).cpu(), t_ref), "ternary codes differ"
    q, deq, _ = F().rmsnorm_quant(x.to(dev), nw.to(dev), eps=1e-8, tiled=False)
    assert torch.equal(q.cpu()[:, :k], q_ref), "int8 activation codes differ"
    assert torch.equal(deq.cpu(), deq_ref)
    kw = {} if path is None else {"path": path}
    out = F().bitlinear(x.to(dev), nw.to(dev), pw, eps=1e-8, **kw)
    # exact integer accumulator on the device (fp64 matmul of the ORACLE's codes: |acc| < 2**53), oracle's scaling
    acc = q_ref.to(dev).double() @ t_ref.to(dev).double().t()
    ref = ((acc.float() * deq_ref.to(dev).reshape(-1, 1)) * wdeq_ref.to(dev)).bfloat16()
    assert torch.equal(out, ref), f"{(out != ref).sum().item()} of {out.numel()} outputs differ"


def test_config2_down_proj_at_4096_rows(dev):
    _bitlinear_case(dev, 4096, 5632, 2048, seed=21, path="mfma")


@pytest.mark.parametrize("m,k,n", [(1, 2048, 70001), (3, 5632, 40000), (2, 2048, 131072)])
def test_vocabulary_sized_gemv_walks_its_n_blocks(dev, m, k, n):
    """Far more n-blocks than resident workgroups: the batch-1 kernel then runs a grid of resident workgroups, each
    walking several n-blocks behind one prologue.  Same exact-contraction check as the other shapes (ragged N too)."""
    _bitlinear_case(dev, m, k, n, seed=23, path="gemv")


def test_vocabulary_sized_gemv_carries_bias_and_addend_along_its_walk(dev):
    """The n-block walk fetches the epilogue operands (bias, addend, the segment's scale) of the next block along with its
    weights.  A launch that walks (N = 100000, ragged) against the exact integer contraction of the same codes (fp64 matmul)
    put through the epilogue's own sequence of fp32 operations: T(T(acc * deq * wdeq + bias) + addend)."""
    g = torch.Generator(device=dev).manual_seed(29)
    m, k, n = 2, 2048, 100003
    w = torch.empty(n, k, device=dev, dtype=torch.bfloat16).normal_(0.0, 0.02, generator=g)
    x = torch.randn(m, k, generator=g, device=dev).bfloat16()
    nw = (1 + 0.1 * torch.randn(k, generator=g, device=dev)).bfloat16()
    bias = torch.randn(n, generator=g, device=dev).bfloat16()
    add = torch.randn(m, n, generator=g, device=dev).bfloat16()
    pw = F().ternarize_pack(w)
    out = F().bitlinear_gemv(x, nw, pw, 1e-6, bias=bias, addend=add)
    q, deq, _ = F().rmsnorm_quant(x, nw, eps=1e-6, tiled=False)
    acc = q[:, :k].double() @ F().unpack_ternary(pw).double().t()
    o = (acc.float() * deq.reshape(-1, 1)) * pw.wdeq
    o = o + bias.float()
    ref = (o.bfloat16().float() + add.float()).bfloat16()
    assert torch.equal(out, ref), f"{(out != ref).sum().item()} of {out.numel()} outputs differ"


@pytest.mark.parametrize("m,k,n", [(8192, 5632, 2048), (16384, 5632, 2048), (16384, 2048, 6144)])
def test_tiled_contraction_with_two_workgroups_per_cu_and_warm_weights(dev, m, k, n):
    """Prefill-sized problems (more tiles than CUs, so two workgroups share a CU) run several times in a row, so that the
    packed weights come from the cache while the activation panels still come from memory: a transfer into LDS and an
    ordinary load complete in no fixed order, and the k-loop's wait has to cover both.  Every run must equal the exact
    integer contraction of the same codes (fp64 matmul: |acc| < 2**53) under the kernel's scaling."""
    g = torch.Generator(device=dev).manual_seed(77)
    x = torch.randn(m, k, generator=g, device=dev).bfloat16()
    w = (torch.randn(n, k, generator=g, device=dev) * 0.02).bfloat16()
    nw = torch.ones(k, device=dev, dtype=torch.bfloat16)
    pw = F().ternarize_pack(w)
    q, deq, qsum = F().rmsnorm_quant(x, nw, eps=1e-8, tiled=True)
    q_rows, deq_rows, _ = F().rmsnorm_quant(x, nw, eps=1e-8, tiled=False)
    t = F().unpack_ternary(pw)
    ref = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
    for r0 in range(0, m, 4096):                                 # fp64 operands in slabs: bounded memory
        acc = q_rows[r0:r0 + 4096, :k].double() @ t.double().t()
        ref[r0:r0 + 4096] = ((acc.float() * deq_rows[r0:r0 + 4096].reshape(-1, 1)) * pw.wdeq).bfloat16()
    bad = []
    for _ in range(6):
        out = torch.zeros(m, n, device=dev, dtype=torch.bfloat16)
        F().bitlinear_mfma(q, deq, qsum, pw, m, torch.bfloat16, out=out, config=17)
        bad.append(int((out != ref).sum()))
    print(f"tiled contraction {m} x {k} -> {n}: outputs differing from the exact contraction over 6 runs: {bad}", flush=True)
    assert bad == [0] * 6


@pytest.mark.parametrize("m", [1, 64])
@pytest.mark.parametrize("kn", [(2048, 11264), (5632, 2048)])
def test_config2_decode_rows(dev, m, kn):
    _bitlinear_case(dev, m, kn[0], kn[1], seed=22 + m)


# ------------------------------------------------------------------ config 3
@pytest.fixture(scope="module")
def scan_case():
    torch.manual_seed(23)
    b, t, d = 8, 2048, 2048
    z = torch.randn(b, 1, t, d) + 2
    x = torch.randn(b, 1, t, d).bfloat16()
    return x, z


def test_config3_recurrent_full_size(dev, scan_case):
    x, z = scan_case
    g = torch.sigmoid(z).bfloat16()
    o_ref, ht_ref = oh.recurrent_hgrn_spec(x, g, None, True)
    o, ht = F().hgrn_recurrent(x.to(dev), g.to(dev), None, True)
    assert torch.equal(o.cpu(), o_ref), f"{(o.cpu() != o_ref).sum().item()} outputs differ"
    assert torch.equal(ht.cpu(), ht_ref)


def test_config3_chunk64_full_size(dev, scan_case):
    x, z = scan_case
    g = torch.nn.functional.logsigmoid(z).bfloat16()
    o_ref, ht_ref = oh.chunk_hgrn_spec(x, g, None, True, chunk=64)
    o, ht = F().hgrn_chunk(x.to(dev), g.to(dev), None, True, chunk_size=64)
    err = ((o.cpu().double() - o_ref.double()).abs().max() / o_ref.double().abs().max()).item()
    assert err <= 1e-2, err                                      # bf16 tolerance of the benchmark definition
    errh = ((ht.cpu().double() - ht_ref.double()).abs().max() / ht_ref.double().abs().max()).item()
    assert errh <= 1e-3, errh                                    # fp32 state


def test_config3_decode_step_batch_64(dev):
    """Single-step decode with carried fp32 state, B = 64, D = 2048: 4 steps == the 4-token recurrence."""
    torch.manual_seed(24)
    b, d, steps = 64, 2048, 4
    i = (2 * torch.randn(b, steps, d)).bfloat16()
    f = (2 * torch.randn(b, steps, d)).bfloat16()
    lb = torch.rand(d) * 0.5
    h0 = torch.randn(b, d)
    x_ref, g_ref = oh.hgrn_gate_spec(i, f, lb, layer_idx=1)
    o_ref, ht_ref = oh.recurrent_hgrn_spec(x_ref.reshape(b, 1, steps, d), g_ref.reshape(b, 1, steps, d), h0.reshape(b, 1, d), True)
    state = h0.to(dev).clone()
    for t in range(steps):
        o = F().hgrn_step(i[:, t].contiguous().to(dev), f[:, t].contiguous().to(dev), state, lb.to(dev))
        assert torch.equal(o.cpu(), o_ref[:, 0, t]), f"step {t}"
    assert torch.equal(state.cpu(), ht_ref.reshape(b, d))


# ------------------------------------------------------------------ configs 4 and 5: the models
class _Case:
    """A benchmark-shape model on the device, its weights on the host, and an oracle whose ternary codes are cached."""
    def __init__(self, shape, dev, seed):
        import bench
        self.model = bench.build_model(shape, torch.bfloat16, dev, seed=seed)
        self.params = {k: v.detach().cpu() for k, v in self.model.state_dict().items()}
        self.L = self.model.config.num_hidden_layers
        self.V = self.model.config.vocab_size
        self.ops = om._Ops("spec", 1e-6)
        self.dev = dev

    def oracle_greedy(self, ids, n_new):
        """(tokens [B, n_new], per-step logits, states after the prompt) with the cached oracle ops."""
        logits, states = om.forward(self.params, ids, self.L, mode="spec", last_only=True, ops=self.ops)
        prompt_states = [s.clone() for s in states]
        toks, all_logits = [], []
        for _ in range(n_new):
            lg = logits[:, -1, :]
            all_logits.append(lg)
            nxt = om.argmax_lowest(lg.float())
            toks.append(nxt)
            logits, states = om.forward(self.params, nxt.reshape(-1, 1), self.L, states=states, mode="spec", ops=self.ops)
        return torch.stack(toks, 1), all_logits, prompt_states


@pytest.fixture(scope="module")
def case_1p3b(dev):
    c = _Case("1.3B", dev, seed=3)
    yield c
    del c.model
    torch.cuda.empty_cache()


def _decode_against_oracle(c, ids, n_new, rows=None, **engine_kw):
    """Prefill + n_new self-feeding greedy steps on the GPU; rows (default all) compared with the oracle."""
    from matmulfreellm_amd.decode import DecodeEngine
    dev, B = c.dev, ids.shape[0]
    rows = list(range(B)) if rows is None else rows
    ref_toks, ref_logits, ref_states = c.oracle_greedy(ids[rows], n_new)
    out = c.model(input_ids=ids.to(dev), use_cache=True, logits_to_keep=1)
    assert torch.equal(out.logits[rows, -1].cpu(), ref_logits[0]), "prefill logits differ from the oracle"
    states = [s[-1] for s in out.past_key_values]
    for li, s in enumerate(states):
        assert torch.equal(s.reshape(B, -1)[rows].cpu(), ref_states[li]), f"state of layer {li} after the prompt"
    eng = DecodeEngine(c.model, B, use_graph=True, **engine_kw)
    eng.load_state(states)
    eng.tok.copy_(out.logits[:, -1].argmax(-1))
    assert torch.equal(eng.tok[rows].cpu(), ref_toks[:, 0])
    for t in range(1, n_new):
        eng.advance()
        assert torch.equal(eng.logits[rows].cpu(), ref_logits[t]), f"logits of decode step {t} differ from the oracle"
        assert torch.equal(eng.tok[rows].cpu(), ref_toks[:, t]), f"greedy token of step {t}"
    eng.check()
    return eng


@pytest.mark.parametrize("batch,resident", [(1, True), (1, False), (16, None), (64, None)])
def test_config4_greedy_decode_vs_oracle(dev, case_1p3b, batch, resident):
    c = case_1p3b
    g = torch.Generator().manual_seed(40 + batch)
    ids = torch.randint(0, c.V, (batch, 8), generator=g)
    kw = {} if resident is None else {"resident": resident}
    eng = _decode_against_oracle(c, ids, 9, **kw)
    if resident is not None:
        assert eng.resident == resident


@pytest.mark.parametrize("batch", [1, 16, 64])
def test_config4_128_greedy_tokens_are_the_same_on_every_decode_path(dev, case_1p3b, batch):
    """The configuration's stated length: a 128-token prompt and 128 greedy tokens, at batch 1, 16 and 64.  The CPU
    oracle covers the first steps (test above); here every decode path the engine has for that batch -- the resident
    launch, one launch per fused BitLinear, the matrix-core contraction, one launch per reference op -- runs the whole
    length from the same prompt state: tokens of all 128 steps, the last step's logits and every layer's final
    recurrent state must be equal bit for bit."""
    from matmulfreellm_amd.decode import DecodeEngine
    c = case_1p3b
    g = torch.Generator().manual_seed(140 + batch)
    ids = torch.randint(0, c.V, (batch, 128), generator=g).to(dev)
    out = c.model(input_ids=ids, use_cache=True, logits_to_keep=1)
    states = [s[-1] for s in out.past_key_values]
    first = out.logits[:, -1].argmax(-1)
    runs, names = [], []
    for kw in ({}, {"resident": False}, {"fuse": False}):
        eng = DecodeEngine(c.model, batch, use_graph=True, **kw)
        name = ("resident" if eng.resident else "fused launch chain" if eng.fused else "fused quantiser + matrix cores"
                if eng.fused_mfma else "one launch per reference op")
        if name in names:
            continue
        eng.load_state(states)
        eng.tok.copy_(first)
        toks = [eng.tok.clone()]
        for _ in range(127):
            eng.advance()
            toks.append(eng.tok.clone())
        eng.check()
        names.append(name)
        runs.append((torch.stack(toks, 1).cpu(), eng.logits.clone().cpu(), [e["state"].clone().cpu() for e in eng.layers]))
        del eng
    print(f"config 4, batch {batch}: 128 greedy tokens on {names}; "
          f"{len(set(runs[0][0].flatten().tolist()))} distinct tokens drawn", flush=True)
    assert len(names) >= 2
    for name, (toks, logits, st) in zip(names[1:], runs[1:]):
        assert torch.equal(toks, runs[0][0]), f"{name} vs {names[0]}: tokens differ first at step " \
            f"{int((toks != runs[0][0]).any(0).nonzero()[0])}"
        assert torch.equal(logits, runs[0][1]), f"{name}: logits of step 128"
        for li, (a, b) in enumerate(zip(st, runs[0][2])):
            assert torch.equal(a, b), f"{name}: state of layer {li} after step 128"


def test_config4_prefill_8x2048_vs_oracle(dev, case_1p3b):
    """The whole 8 x 2048 prompt batch on the GPU; rows 1 and 6 through the oracle: last-position logits and the
    final recurrent state of every layer."""
    c = case_1p3b
    g = torch.Generator().manual_seed(44)
    ids = torch.randint(0, c.V, (8, 2048), generator=g)
    rows = [1, 6]
    ref_logits, ref_states = om.forward(c.params, ids[rows], c.L, mode="spec", last_only=True, ops=c.ops)
    out = c.model(input_ids=ids.to(dev), use_cache=True, logits_to_keep=1)
    got = out.logits[rows, -1].cpu()
    assert torch.equal(got, ref_logits[:, -1]), f"{(got != ref_logits[:, -1]).sum().item()} logits differ"
    for li, s in enumerate(out.past_key_values):
        assert torch.equal(s[-1].reshape(8, -1)[rows].cpu(), ref_states[li]), f"final state of layer {li}"


def test_config5_batch_128_rows_vs_oracle(dev, case_1p3b):
    """2.7B shape, 512-token prompt, batch 128 (the large-batch matrix-core decode): rows 0 and 77 of the batch against
    the oracle for the prompt and 6 greedy steps."""
    del case_1p3b                                                # only ordering: the 1.3B fixture is torn down after this module
    c = _Case("2.7B", dev, seed=5)
    g = torch.Generator().manual_seed(45)
    ids = torch.randint(0, c.V, (128, 512), generator=g)
    _decode_against_oracle(c, ids, 7, rows=[0, 77])
    del c.model
    torch.cuda.empty_cache()
