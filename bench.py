#!/usr/bin/env python3
"""Headline benchmark: greedy decode tok/s of the 1.3B-shape HGRNBit model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--only LEG[,LEG...]]

One step = one decode step of the whole model (24 layers, ternary 2-bit packed weights,
bf16 activations, fp32 recurrent state) for the whole batch, replayed as one HIP graph with
inputs resident in HBM.  Prints ONE JSON line:
  value        decode tokens/s at --batch (default 1)
  roofline     the dominant kernel at batch 1: the resident launch that is the whole decode step
               (decode_layers_kernel: embedding row, the 4L fused BitLinears, lm_head, argmax) --
               its algorithmic bytes (every 2-bit weight once + each link's activations, norm
               weights and state) / its launch time, timed live with HIP events on the launch
               stream; with --launch-chain the fused BitLinear GEMV launches of one step instead.
               The model's own 325 MB of packed weights exceed the 256 MB last-level cache, so
               HBM, not a cache, is measured.
  cpu_baseline the reference's PyTorch formulation (oracle, literal mode, weights
               re-quantised per call as the reference does) timed on this host's cores on bounded
               samples: 1.3B-shape decode (2 of 24 layers + head, scaled), the tiny config end to
               end, single BitLinears and the scan
  extra        batch-64 decode, prompt prefill (8 x 512 and 8 x 2048 tokens, with the whole forward's
               int8 TOP/s against 5.0 POP/s), prefill-sized BitLinear on the int8 matrix cores,
               HGRN scan, norm and loss bandwidths (cache-cold: the legs rotate through buffer sets
               of more than 512 MB in total; counted HBM traffic from rocprofv3 beside each),
               and one training step (forward + loss + backward) of the same model at 8 x 1024 tokens.
--only runs the named legs only (decode, bs64, prefill, mfma, gemv_stream, scan, norms, sampling, loss, train, cpu, link_trace): the
profiles under profiles/ are made that way.
Synthetic data: random-init N(0, 0.02) weights, uniform random token ids.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0

SHAPES = {
    "1.3B": dict(vocab_size=32000, hidden_size=2048, num_hidden_layers=24),
    "2.7B": dict(vocab_size=32000, hidden_size=2560, num_hidden_layers=32),
    "tiny": dict(vocab_size=32000, hidden_size=512, num_hidden_layers=4),
}


def build_model(shape, dtype, dev, seed=0):
    """Random-init model built on the meta device and filled on the GPU (no 1.3B-element host init)."""
    import matmulfreellm_amd as mm
    cfg = mm.HGRNBitConfig(**SHAPES[shape])
    with torch.device("meta"):
        model = mm.HGRNBitForCausalLM(cfg)
    model = model.to_empty(device=dev).to(dtype)
    g = torch.Generator(device=dev).manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("lower_bounds"):
                p.zero_()
            elif name.endswith("norm.weight") or ".g_norm." in name:
                p.fill_(1.0)
            else:
                p.copy_((torch.randn(p.shape, generator=g, device=dev, dtype=torch.float32) * 0.02).to(dtype))
    return model.eval()


def timed(fn, iters, warmup=2):
    """Average milliseconds of fn() over `iters` calls, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


def decode_bench(model, batch, steps, warmup, dev, prompt_len=128, resident=None):
    from matmulfreellm_amd.decode import DecodeEngine
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(1)
    ids = torch.randint(0, model.config.vocab_size, (batch, prompt_len), generator=g, device=dev)
    with torch.no_grad():
        out = model(input_ids=ids, use_cache=True, logits_to_keep=1)
    first = F_.argmax(out.logits[:, -1])
    eng = DecodeEngine.for_model(model, batch, use_graph=True, resident=resident)
    eng.load_state([c[-1] for c in out.past_key_values])
    eng.tok.copy_(first)
    for _ in range(max(warmup, 1)):
        eng.advance()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    s.record()
    for _ in range(steps):
        eng.advance()
    e.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = max(s.elapsed_time(e), wall * 1e3) / steps      # never report less than the wall clock
    eng.check()                                          # a timed-out wait inside the resident launch voids the figure
    return ms, eng


# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a plain copy of known size);
# see profiles/ for the runs and the scale factors.
GEMV_TRAFFIC_BYTES_PER_LAUNCH = 3623641          # one fused BitLinear GEMV launch of the launch chain
LAYERS_TRAFFIC_BYTES_PER_LAUNCH = 356434265         # the resident layer-chain launch


def _replay_time(launch, iters):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    return timed(graph.replay, iters)


def gemv_roofline(eng, iters=20):
    """The dominant kernel of a batch-1 decode step, timed on its own inside a graph.

    Resident engine: the one persistent launch that is the whole step -- the 4L fused BitLinears of the layers, the
    lm_head and the argmax (algorithmic bytes: every packed weight once, plus each link's activations, norm weights
    and state).  Otherwise: a graph that holds
    exactly the fused BitLinear GEMV launches of one step (4 per layer + lm_head), averaged per launch."""
    assert eng.fused and eng.B == 1
    counted = (eng.H, eng.L, eng.I, eng.V) == (2048, 24, 5632, 32000)    # the shape the counter runs were made on
    if eng.resident:
        launch = lambda: eng._launch_layers(True)
        ms = _replay_time(launch, iters)
        assert eng.resident_ok(), "a wait inside the resident layer chain timed out"
        total_bytes = eng.fused_step_bytes()
        achieved = total_bytes / (ms * 1e-3) / 1e9
        return {"bound": "hbm", "kernel": "decode_layers_kernel", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": LAYERS_TRAFFIC_BYTES_PER_LAUNCH if counted else None,
                "launches_per_step": 1, "links_per_launch": 4 * eng.L + 2,
                "algorithmic_bytes_per_launch": total_bytes, "avg_launch_us": round(ms * 1e3, 3)}
    ms = _replay_time(lambda: eng._launch_step_fused(ends=False), iters)
    n = 4 * eng.L + 1
    total_bytes = eng.fused_step_bytes()
    us_per_launch = ms * 1e3 / n
    achieved = (total_bytes / n) / (us_per_launch * 1e-6) / 1e9
    return {"bound": "hbm", "kernel": "bitlinear_gemv_kernel", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH if counted else None,
            "launches_per_step": n, "algorithmic_bytes_per_launch": total_bytes // n,
            "avg_launch_us": round(us_per_launch, 3)}


def gemv_stream_bench(dev, n=600000, k=2048, iters=12):
    """The batch-1 fused BitLinear kernel with nothing but HBM in its way: one launch over n x k packed ternary
    weights (n * k / 4 bytes, past 300 MB), two such operands alternating so that no launch finds its weights in the
    256 MB last-level cache, every launch independent of the others (same input row, outputs never read).  This is
    the rate the kernel's load path and dot reach when no hand-off waits on it."""
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(12)
    pws = []
    for _ in range(2):
        w = torch.empty(n, k, device=dev, dtype=torch.bfloat16).normal_(0.0, 0.02, generator=g)
        pws.append(F_.ternarize_pack(w))
        del w
    x = torch.randn(1, k, generator=g, device=dev).bfloat16()
    nw = torch.ones(k, device=dev, dtype=torch.bfloat16)
    turn = [0]

    def launch():
        turn[0] ^= 1
        return F_.bitlinear_gemv(x, nw, pws[turn[0]], 1e-8)
    ms = timed(launch, iters, warmup=4)
    packed = pws[0].packed.numel()
    nbytes = packed + 2 * k * 2 + n * 2            # packed weights, input row and norm weight, output row
    gbs = nbytes / ms / 1e6
    return {"kernel": "bitlinear_gemv_kernel", "M": 1, "N": n, "K": k, "packed_weight_bytes": packed, "operands_alternating": 2,
            "algorithmic_bytes_per_launch": nbytes, "avg_launch_us": round(ms * 1e3, 2), "GBs": round(gbs, 1),
            "frac_of_hbm": round(gbs / HBM_PEAK_GBS, 4), "counted_fetch_bytes_per_launch": COUNTED_TRAFFIC.get("gemv_stream")}


def link_trace_bench(model, dev, delay=6):
    """Where a link of the resident batch-1 launch spends its cycles: the kernel's own cycle stamps (thread 0 of three
    workgroups, nine points per link; the traced build of the kernel), averaged per kind of link over the layers of one
    decode step."""
    import numpy as np
    from matmulfreellm_amd.decode import DecodeEngine
    eng = DecodeEngine.for_model(model, 1, use_graph=True)
    if not eng.resident:
        return None
    for _ in range(4):
        eng._launch_layers(True)
    t = eng.link_trace(delay=delay).numpy().astype(np.float64)
    assert eng.resident_ok()
    names = ["i/f/g", "o_proj", "gate/up", "down"]
    stages = ["row arrives", "block norm", "sum of squares", "absmax", "codes -> LDS", "dot", "partials meet", "epilogue"]
    out = {"unit": "shader clock cycles (s_memtime), mean over layers 2.. of one step", "stages": stages, "poll_delay": delay,
           "workgroups": {}}
    nl = 4 * eng.L
    for wg in (0, 37, 200):
        slot = wg
        per = {}
        for kind in range(4):
            rows = t[slot, kind:nl:4, :9][2:]
            nxt = t[slot, kind + 1:nl + 1:4, 0][2:]                     # entry of the following link
            n = min(len(rows), len(nxt))
            per[names[kind]] = {"stages": [round(float(v)) for v in np.diff(rows, axis=1).mean(axis=0)],
                                "link_total": round(float((rows[:, 8] - rows[:, 0]).mean())),
                                "entry_to_next_entry": round(float((nxt[:n] - rows[:n, 0]).mean()))}
        per["whole_chain_cycles"] = int(t[slot, nl - 1, 8] - t[slot, 0, 0])
        out["workgroups"][str(wg)] = per
    # all 256 workgroups on the 100 MHz clock the XCDs share (stamps 9 / 10 / 11 = link entered / row arrived / last store
    # issued, 10 ns units): how long after the LAST producer's store the LAST consumer has its row, how long a workgroup
    # then needs, and the period of a link
    ent, arr, fin = t[:, :nl, 9] * 10.0, t[:, :nl, 10] * 10.0, t[:, :nl, 11] * 10.0
    allw = {}
    for kind in range(4):
        ls = np.arange(8 + kind, nl, 4)
        allw[names[kind]] = {
            "last_store_to_last_arrival_ns": round(float(np.mean(arr[:, ls].max(axis=0) - fin[:, ls - 1].max(axis=0)))),
            "arrival_to_own_last_store_ns_median": round(float(np.median(fin[:, ls] - arr[:, ls]))),
            "arrival_to_own_last_store_ns_max": round(float(np.mean((fin[:, ls] - arr[:, ls]).max(axis=0)))),
            "link_period_ns": round(float(np.mean(fin[:, ls].max(axis=0) - fin[:, ls - 1].max(axis=0))))}
    out["all_256_workgroups_shared_clock"] = allw
    return out


def mfma_bench(dev, m=4096, k=2048, n=11264, iters=20):
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn(m, k, generator=g, device=dev).bfloat16()
    w = (torch.randn(n, k, generator=g, device=dev) * 0.02).bfloat16()
    nw = torch.ones(k, device=dev, dtype=torch.bfloat16)
    pw = F_.ternarize_pack(w)
    q, deq, qsum = F_.rmsnorm_quant(x, nw, eps=1e-8, tiled=True)
    out = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
    ms_mm = timed(lambda: F_.bitlinear_mfma(q, deq, qsum, pw, m, torch.bfloat16, out=out), iters)
    ms_q = timed(lambda: F_.rmsnorm_quant(x, nw, eps=1e-8, tiled=True), iters)
    tops = 2.0 * m * k * n / (ms_mm * 1e-3) / 1e12
    # the clock the part sustains under this kernel: shader-clock ticks over 100 MHz ticks, per workgroup, of one launch
    lib, wgs = F_.L.load(), (m // 64) * (n // 512)
    clocks = torch.zeros(wgs, 2, dtype=torch.int64, device=dev)
    F_.L.check(lib.mmf_bitlinear_mfma_clock_sink(clocks.data_ptr(), wgs), "mmf_bitlinear_mfma_clock_sink")
    try:
        F_.bitlinear_mfma(q, deq, qsum, pw, m, torch.bfloat16, out=out)
        torch.cuda.synchronize()
    finally:
        F_.L.check(lib.mmf_bitlinear_mfma_clock_sink(None, 0), "mmf_bitlinear_mfma_clock_sink")
    c = clocks.double().cpu()
    ghz = float((c[:, 0] / c[:, 1].clamp(min=1)).median()) * 0.1
    # a SIMD holds 2 waves of a workgroup, each issuing (k / 32) steps of 4 MFMAs of 32 pipe cycles per tile; two
    # workgroups share a CU when the launch has more than 256 of them
    busy = (k // 32) * 4 * 32 * 2 * (2 if wgs > 256 else 1) / float(c[:, 0].median())
    return {"shape": [m, k, n], "contract_ms": round(ms_mm, 4), "quant_prologue_ms": round(ms_q, 4),
            "int8_TOPs": round(tops, 1), "frac_of_5POPs": round(tops / INT8_PEAK_TOPS, 4),
            "shader_clock_GHz_in_kernel": round(ghz, 3), "workgroup_cycles_median": int(c[:, 0].median()),
            "matrix_pipe_busy_frac": round(busy, 3)}


def mfma_pipe_bench(dev, random_operands, steps=512, per_cu=2):
    """The matrix pipe alone: the tiled kernel's four independent MFMAs per step on register operands, nothing else.
    With constant operands the pipe switches little and draws little power; random int8 codes and ternary weights
    are what a contraction feeds it."""
    import matmulfreellm_amd.functional as F_
    lib, wgs = F_.L.load(), 256 * per_cu
    clocks = torch.zeros(2 * wgs + 1, dtype=torch.int64, device=dev)
    run = lambda: F_.L.check(lib.mmf_mfma_pipe_probe(steps, wgs, int(random_operands), clocks.data_ptr(), F_.L.stream()), "mmf_mfma_pipe_probe")
    ms = timed(run, 10)
    c = clocks[:2 * wgs].view(wgs, 2).double().cpu()
    ghz = float((c[:, 0] / c[:, 1].clamp(min=1)).median()) * 0.1
    tops = wgs * 8 * steps * 4 * 65536.0 / (ms * 1e-3) / 1e12
    # a SIMD holds per_cu * 2 waves, each with steps * 4 MFMAs of 32 pipe cycles, against the launch's cycles at that clock
    busy = steps * 4 * 32 * per_cu * 2 / (ms * 1e-3 * ghz * 1e9)
    return {"workgroups": wgs, "steps": steps, "ms": round(ms, 4), "int8_TOPs": round(tops, 1),
            "frac_of_5POPs": round(tops / INT8_PEAK_TOPS, 4), "shader_clock_GHz_in_kernel": round(ghz, 3),
            "matrix_pipe_busy_frac": round(busy, 3)}


def _rotating(make_set, set_bytes, min_total=512 << 20, min_sets=3):
    """Independent buffer sets whose total exceeds the 256 MB last-level cache twice over, and a counter to walk them:
    by the time a set comes round again the others have pushed it out, so every launch reads from HBM."""
    n = max(min_sets, -(-min_total // set_bytes) + 1)
    sets = [make_set() for _ in range(n)]
    state = {"i": 0}

    def nxt():
        state["i"] = (state["i"] + 1) % n
        return sets[state["i"]]
    return nxt, n


# HBM bytes per launch of the bandwidth-bound kernels at the shapes below, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (profiles/hbm_traffic_scan_norm_loss.txt, profiles/bitlinear_gemv_stream_300MB.txt; same calibration copy as the decode
# kernels).
COUNTED_TRAFFIC = {"gemv_stream": 307306444, "hgrn_recurrent": 201454106, "hgrn_chunk": 201465983, "rmsnorm": 134327968,
                   "rmsnorm_swishgate": 201471067, "cross_entropy": 263063850}


def scan_bench(dev, b=8, t=2048, d=2048, iters=12):
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(3)

    def make():
        z = torch.randn(b, 1, t, d, generator=g, device=dev) + 2
        x = torch.randn(b, 1, t, d, generator=g, device=dev).bfloat16()
        return x, torch.nn.functional.logsigmoid(z).bfloat16(), torch.sigmoid(z).bfloat16()
    nbytes = 3 * b * t * d * 2
    nxt, nsets = _rotating(make, 4 * b * t * d * 2)

    def rec():
        x, _, glin = nxt()
        F_.hgrn_recurrent(x, glin)

    def chk():
        x, glog, _ = nxt()
        F_.hgrn_chunk(x, glog, chunk_size=64)
    ms_r = timed(rec, iters, warmup=nsets)
    ms_c = timed(chk, iters, warmup=nsets)
    # one long sequence: the same bytes as [1, 8 * t, d]; batch * channels alone give 32 workgroups, so the chunked entry
    # point also splits the time axis over workgroups (the sequential recurrence cannot)
    ms_r1 = timed(lambda: F_.hgrn_recurrent(*[v.view(1, 1, b * t, d) for v in (lambda s: (s[0], s[2]))(nxt())]), iters, warmup=nsets)
    ms_c1 = timed(lambda: F_.hgrn_chunk(*[v.view(1, 1, b * t, d) for v in nxt()[:2]], chunk_size=64), iters, warmup=nsets)
    long_seq = {"shape": [1, b * t, d], "recurrent_ms": round(ms_r1, 4), "recurrent_GBs": round(nbytes / ms_r1 / 1e6, 1),
                "chunk64_ms": round(ms_c1, 4), "chunk64_GBs": round(nbytes / ms_c1 / 1e6, 1)}
    return {"shape": [b, t, d], "buffer_sets": nsets, "recurrent_ms": round(ms_r, 4), "recurrent_GBs": round(nbytes / ms_r / 1e6, 1),
            "one_long_sequence": long_seq,
            "recurrent_frac_of_hbm": round(nbytes / ms_r / 1e6 / HBM_PEAK_GBS, 4),
            "chunk64_ms": round(ms_c, 4), "chunk64_GBs": round(nbytes / ms_c / 1e6, 1),
            "algorithmic_bytes": nbytes, "counted_traffic_bytes": {"recurrent": COUNTED_TRAFFIC["hgrn_recurrent"],
                                                                   "chunk64": COUNTED_TRAFFIC["hgrn_chunk"]}}


def prefill_bench(model, dev, batch=8, seq=512, iters=5):
    """Module-path forward over a prompt batch (state cache kept, last-position logits only)."""
    g = torch.Generator(device=dev).manual_seed(5)
    ids = torch.randint(0, model.config.vocab_size, (batch, seq), generator=g, device=dev)
    with torch.no_grad():
        ms = timed(lambda: model(input_ids=ids, use_cache=True, logits_to_keep=1), iters)
    # int8 operations of the whole forward: every row through every layer's ternary weights, the last position of
    # every sequence through the head
    layer_w = sum(p.numel() for n, p in model.named_parameters() if n.endswith("proj.weight"))
    head_w = model.lm_head.weight.numel()
    ops = 2.0 * (batch * seq * layer_w + batch * head_w)
    tops = ops / (ms * 1e-3) / 1e12
    return {"batch": batch, "seq_len": seq, "ms": round(ms, 3), "tok_s": round(batch * seq / ms * 1e3),
            "int8_TOPs_whole_forward": round(tops, 1), "frac_of_5POPs": round(tops / INT8_PEAK_TOPS, 4)}


def norm_bench(dev, m=16384, k=2048, iters=24):
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(4)
    w = torch.ones(k, device=dev, dtype=torch.bfloat16)

    def make():
        return (torch.randn(m, k, generator=g, device=dev).bfloat16(), torch.randn(m, k, generator=g, device=dev).bfloat16())
    nxt, nsets = _rotating(make, 3 * m * k * 2)

    def plain():
        x, _ = nxt()
        F_.rmsnorm(x, w)

    def gated():
        x, o = nxt()
        F_.rmsnorm_swishgate(x, o, w)
    ms_n = timed(plain, iters, warmup=nsets)
    ms_g = timed(gated, iters, warmup=nsets)
    return {"shape": [m, k], "buffer_sets": nsets, "rmsnorm_GBs": round(2 * m * k * 2 / ms_n / 1e6, 1),
            "rmsnorm_swishgate_GBs": round(3 * m * k * 2 / ms_g / 1e6, 1),
            "algorithmic_bytes": {"rmsnorm": 2 * m * k * 2, "rmsnorm_swishgate": 3 * m * k * 2},
            "counted_traffic_bytes": {"rmsnorm": COUNTED_TRAFFIC["rmsnorm"], "rmsnorm_swishgate": COUNTED_TRAFFIC["rmsnorm_swishgate"]}}


def loss_bench(dev, m=4096, v=32000, iters=12):
    """Evaluation loss of m rows of v-wide bf16 logits (one read of the logits)."""
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(6)
    targets = torch.randint(0, v, (m,), generator=g, device=dev)
    lib, rows = F_.L.load(), torch.empty(m, dtype=torch.float32, device=dev)
    nxt, nsets = _rotating(lambda: torch.randn(m, v, generator=g, device=dev).bfloat16(), m * v * 2)

    def run():
        logits = nxt()
        F_.L.check(lib.mmf_cross_entropy_fwd(logits.data_ptr(), v, targets.data_ptr(), -100, rows.data_ptr(), m, v,
                                             F_.L.dtype_id(logits.dtype), F_.L.stream()), "mmf_cross_entropy_fwd")
    ms = timed(run, iters, warmup=nsets)
    return {"shape": [m, v], "buffer_sets": nsets, "ms": round(ms, 4), "GBs": round(m * v * 2 / ms / 1e6, 1),
            "algorithmic_bytes": m * v * 2, "counted_traffic_bytes": COUNTED_TRAFFIC["cross_entropy"]}


def sampler_bench(model, dev, n_new=256):
    """Top-p sampling as the reference's generate.py asks for it (top_p 0.4, temperature 0.6): the sampling kernel
    alone on one 32000-wide row, and generate() end to end (128-token prompt, prefill included) against greedy."""
    import matmulfreellm_amd.functional as F_
    g = torch.Generator(device=dev).manual_seed(5)
    lg = (torch.randn(1, 32000, generator=g, device=dev) * 3).bfloat16()
    u = torch.rand(1, generator=g, device=dev)
    out = torch.empty(1, dtype=torch.int64, device=dev)
    us = timed(lambda: F_.sample_top_p(lg, 0.4, 0.6, u, out=out), 50) * 1e3
    us_k = timed(lambda: F_.sample_top_p(lg, 0.4, 0.6, u, out=out, top_k=50), 50) * 1e3
    ids = torch.randint(0, model.config.vocab_size, (1, 128), generator=g, device=dev)
    res = {"sample_top_p_us_per_row_of_32000": round(us, 2), "with_top_k_50_us": round(us_k, 2)}
    for name, kw in (("greedy", {}), ("top_p", dict(do_sample=True, top_p=0.4, temperature=0.6, generator=g))):
        model.generate(ids, max_new_tokens=8, eos_token_id=None, **kw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.generate(ids, max_new_tokens=n_new, eos_token_id=None, **kw)
        torch.cuda.synchronize()
        res[f"generate_{name}_tok_s"] = round(n_new / (time.perf_counter() - t0), 1)
    return res


def train_bench(model, dev, batch=8, seq=1024, iters=3):
    """One training step of the module path: forward with the fused loss, backward to the gradient of every
    parameter (no optimiser step), plus the two backward kernels that carry the most bytes, timed alone."""
    import matmulfreellm_amd as mm
    g = torch.Generator(device=dev).manual_seed(9)
    ids = torch.randint(0, model.config.vocab_size, (batch, seq), generator=g, device=dev)
    model.train()

    def step():
        for p in model.parameters():
            p.grad = None
        model(input_ids=ids, labels=ids).loss.backward()
    try:
        ms = timed(step, iters, warmup=2)
    finally:
        model.eval()
        for p in model.parameters():
            p.grad = None
    res = {"batch": batch, "seq_len": seq, "ms_per_step": round(ms, 2), "tok_s": round(batch * seq / ms * 1e3),
           "what": "forward + loss + backward, bf16 parameters, no optimiser step"}
    b, t, d = 8, 2048, model.config.hidden_size
    x = torch.randn(b, 1, t, d, generator=g, device=dev).bfloat16().requires_grad_()
    gt = torch.sigmoid(torch.randn(b, 1, t, d, generator=g, device=dev)).bfloat16().requires_grad_()
    o, _ = mm.fused_recurrent_hgrn(x, gt)
    do = torch.randn_like(o)
    ms_s = timed(lambda: torch.autograd.grad(o, (x, gt), do, retain_graph=True), 10)
    res["scan_backward"] = {"shape": [b, t, d], "ms": round(ms_s, 4), "GBs": round(5 * b * t * d * 2 / ms_s / 1e6, 1),
                            "algorithmic_bytes": 5 * b * t * d * 2}
    m, k = 16384, d
    xn = torch.randn(m, k, generator=g, device=dev).bfloat16().requires_grad_()
    norm = mm.RMSNorm(k).to(dev, torch.bfloat16)
    y = norm(xn)
    dy = torch.randn_like(y)
    ms_n = timed(lambda: torch.autograd.grad(y, (xn, norm.weight), dy, retain_graph=True), 10)
    res["rmsnorm_backward"] = {"shape": [m, k], "ms": round(ms_n, 4), "GBs": round(3 * m * k * 2 / ms_n / 1e6, 1),
                               "algorithmic_bytes": 3 * m * k * 2}
    return res


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _median_s(fn, reps, warm=1):
    for _ in range(warm):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def cpu_baseline(shape="1.3B", budget_s=25.0):
    """The reference's PyTorch formulation (oracle, literal mode; weights re-quantised on every call, as the reference
    does) on the host cores.  Headline leg: batch-1 decode of a 1.3B-shape model, timed on 2 of its 24 layers plus the
    head and scaled to 24 layers.  Further legs: the tiny configuration end to end (batch 1, 128 tokens: one forward
    and greedy steps), single BitLinears at the benchmark's shapes, and the recurrence."""
    from oracle import bitlinear as ob
    from oracle import hgrn as oh
    from oracle import model as om
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    cfg = SHAPES[shape]
    H, V, Lfull = cfg["hidden_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    Ls = 2
    params = om.init_params(V, H, Ls, seed=0, dtype=torch.float32)
    ids = torch.randint(0, V, (1, 1))
    states = [torch.zeros(1, H) for _ in range(Ls)]
    x = torch.randn(1, 1, H)

    def run_model():
        om.forward(params, ids, Ls, states=states, mode="literal")

    def run_head():
        ob.bitlinear_literal(x, params["lm_head.weight"], params["lm_head.norm.weight"])

    run_model(); run_head()
    t_one = _median_s(run_model, 1, warm=0)
    reps = max(3, min(15, int(budget_s / 3 / max(t_one, 1e-3))))
    t_model = _median_s(run_model, reps, warm=0)
    t_head = _median_s(run_head, reps, warm=0)
    t_layer = max(t_model - t_head, 1e-9) / Ls
    t_tok = t_layer * Lfull + t_head
    del params

    legs = {}
    # tiny configuration, fp32, batch 1, 128-token prompt: forward over the prompt, then greedy steps with carried state
    tc = SHAPES["tiny"]
    tp = om.init_params(tc["vocab_size"], tc["hidden_size"], tc["num_hidden_layers"], seed=0, dtype=torch.float32)
    tids = torch.randint(0, tc["vocab_size"], (1, 128))
    nl = tc["num_hidden_layers"]
    t_fwd = _median_s(lambda: om.forward(tp, tids, nl, mode="literal"), 3)
    _, st = om.forward(tp, tids, nl, mode="literal", last_only=True)
    t_step = _median_s(lambda: om.forward(tp, tids[:, :1], nl, states=st, mode="literal"), 5)
    legs["tiny_config_fp32"] = {"prompt_128_forward_ms": round(t_fwd * 1e3, 1), "prompt_tok_s": round(128 / t_fwd, 1),
                                "greedy_decode_tok_s": round(1.0 / t_step, 2)}
    del tp
    # single BitLinear, bf16-valued inputs computed in fp32 (the reference's CPU-runnable path), weights re-quantised per call
    for name, (m, k, n) in (("bitlinear_4096x2048x11264", (4096, 2048, 11264)), ("bitlinear_4096x5632x2048", (4096, 5632, 2048)),
                            ("bitlinear_64x2048x11264", (64, 2048, 11264)), ("bitlinear_1x2048x11264", (1, 2048, 11264))):
        xx, ww, nw = torch.randn(m, k), torch.randn(n, k) * 0.02, torch.ones(k)
        legs[name + "_ms"] = round(_median_s(lambda: ob.bitlinear_literal(xx, ww, nw), 3) * 1e3, 2)
    # recurrence, naive loop as the reference's CPU oracle runs it: B = 8, D = 2048, T reduced from 2048 to 512
    b, t, d = 8, 512, 2048
    gg = torch.sigmoid(torch.randn(b, 1, t, d) + 2)
    xs = torch.randn(b, 1, t, d)
    legs["hgrn_naive_scan_8x512x2048_ms"] = round(_median_s(lambda: oh.naive_recurrent_hgrn_literal(xs, gg), 3) * 1e3, 2)
    legs["hgrn_scan_note"] = "T reduced from 2048 to 512 (time is linear in T)"
    return {"value": round(1.0 / t_tok, 3), "unit": "tok/s", "cores": cores, "kind": "port",
            "sample": f"batch-1 decode step of a {shape}-shape model in fp32, {Ls} of {Lfull} layers + lm_head timed "
                      f"(median of {reps}), scaled to {Lfull} layers; weights re-quantised on every call as the reference does",
            "ms_per_token": round(t_tok * 1e3, 2), "cpu_model": _cpu_model(), "torch": torch.__version__, "legs": legs}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--shape", default="1.3B", choices=list(SHAPES))
    ap.add_argument("--launch-chain", action="store_true",
                    help="batch 1: one launch per fused BitLinear instead of the resident layer chain")
    ap.add_argument("--no-extra", action="store_true", help="skip the batch-64 / matrix-core / scan / norm / CPU legs")
    ap.add_argument("--only", default="", help="comma-separated legs to run instead of everything: decode, bs64, prefill, mfma, gemv_stream, "
                                               "scan, norms, sampling, loss, train, cpu, link_trace (profiling runs)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    only = {t for t in args.only.split(",") if t}
    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    if only and not (only & {"decode", "bs64", "prefill", "sampling", "link_trace", "train"}):
        # legs that need no model: run them alone and print what they measured
        res = {}
        if "mfma" in only:
            res["bitlinear_mfma_gate_proj"] = mfma_bench(dev, 4096, 2048, 11264)
            res["bitlinear_mfma_down_proj"] = mfma_bench(dev, 4096, 5632, 2048)
            res["matrix_pipe_alone_random_operands"] = mfma_pipe_bench(dev, True)
            res["matrix_pipe_alone_constant_operands"] = mfma_pipe_bench(dev, False)
        if "gemv_stream" in only:
            res["gemv_stream"] = gemv_stream_bench(dev)
        if "scan" in only:
            res["hgrn_scan"] = scan_bench(dev)
        if "norms" in only:
            res["norms"] = norm_bench(dev)
        if "loss" in only:
            res["cross_entropy"] = loss_bench(dev)
        if "cpu" in only:
            res["cpu_baseline"] = cpu_baseline(args.shape)
        print(json.dumps({"only": sorted(only), "extra": res}))
        return
    model = build_model(args.shape, torch.bfloat16, dev)
    n_tern = sum(p.numel() for n, p in model.named_parameters() if n.endswith("proj.weight") or n == "lm_head.weight")

    ms, eng = decode_bench(model, args.batch, args.steps, args.warmup, dev, resident=False if args.launch_chain else None)
    tok_s = args.batch * 1e3 / ms
    result = {
        "metric": "decode tok/s 1.3B-shape bs=1/64; BitLinear HBM GB/s & int8 MFMA util",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"{args.shape}-shape HGRNBit greedy decode, batch {args.batch}, 128-token prompt, "
                               f"{args.steps} timed steps, whole step = one HIP graph",
                   "batch": args.batch, "ternary_weights": n_tern, "packed_weight_bytes": n_tern // 4,
                   "decode_path": ("one resident launch (embedding row, layers, lm_head, argmax)" if eng.resident
                                   else "one launch per fused BitLinear (4 per layer)" if eng.fused
                                   else "fused quantiser + matrix-core contraction per BitLinear (8 launches per layer)"
                                   if eng.fused_mfma else "one launch per reference op")},
    }
    hbm_step_us = (n_tern / 4) / (HBM_PEAK_GBS * 1e3)
    result["decode_frac_of_weight_stream_bound"] = round(hbm_step_us / (ms * 1e3), 4)

    eng1 = eng
    if args.batch != 1:
        from matmulfreellm_amd.decode import DecodeEngine
        eng1 = DecodeEngine.for_model(model, 1, use_graph=True, resident=False if args.launch_chain else None)
    result["roofline"] = gemv_roofline(eng1)

    def want(leg):
        return (leg in only) if only else not args.no_extra

    extra = {}
    other = 64 if args.batch == 1 else 1
    if want("bs64"):
        ms_o, _ = decode_bench(model, other, args.steps, args.warmup, dev)
        extra[f"decode_bs{other}_tok_s"] = round(other * 1e3 / ms_o, 1)
        extra[f"decode_bs{other}_ms_per_step"] = round(ms_o, 4)
    if want("prefill"):
        extra["prefill_8x512"] = prefill_bench(model, dev, 8, 512)
        extra["prefill_8x2048"] = prefill_bench(model, dev, 8, 2048, iters=3)
    if want("mfma"):
        extra["bitlinear_mfma_gate_proj"] = mfma_bench(dev, 4096, 2048, 11264)
        extra["bitlinear_mfma_down_proj"] = mfma_bench(dev, 4096, 5632, 2048)
        extra["matrix_pipe_alone_random_operands"] = mfma_pipe_bench(dev, True)
        extra["matrix_pipe_alone_constant_operands"] = mfma_pipe_bench(dev, False)
    if want("gemv_stream"):
        extra["gemv_stream"] = gemv_stream_bench(dev)
    if want("scan"):
        extra["hgrn_scan"] = scan_bench(dev)
    if want("norms"):
        extra["norms"] = norm_bench(dev)
    if "link_trace" in only:
        extra["link_trace"] = link_trace_bench(model, dev)
    if want("sampling"):
        extra["sampling"] = sampler_bench(model, dev)
    if want("loss"):
        extra["cross_entropy"] = loss_bench(dev)
    if want("train"):
        extra["training_step"] = train_bench(model, dev)
    if extra:
        result["extra"] = extra
    del model, eng, eng1
    torch.cuda.empty_cache()
    result["cpu_baseline"] = cpu_baseline(args.shape) if want("cpu") else None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
