"""Whole-model single-token decode step as one HIP graph.

At batch 1 the 4L fused BitLinears of the layers run as ONE persistent launch (mmf_decode_layers: resident
workgroups hand activations to each other as tagged words), followed by the lm_head launch and the argmax.

The module path (HGRNBitForCausalLM.forward with T = 1) issues the same kernels through
nn.Module calls and fresh output tensors; at batch 1 that host work dwarfs the ~40 us the
weights take to stream.  DecodeEngine lays the step out once over static buffers, records it
into a graph (torch.cuda.CUDAGraph = hipGraph) and replays it per token: embedding gather ->
L x [RMSNorm, i/f/g BitLinear, gate + recurrence step, gated norm, o_proj BitLinear,
residual RMSNorm, gate_proj BitLinear, swiglu, down_proj BitLinear (+residual)] -> final
norm -> lm_head BitLinear -> argmax.  The argmax writes the token buffer the next replay's
embedding reads, so consecutive steps need no host round trip.

Every launch is the same C-ABI call with the same arithmetic as the module path, so the two
produce identical bits (tests/test_gpu_model.py checks that).
"""
import ctypes
import warnings
from typing import List, Optional

import torch

from . import _lib as L
from . import functional as F_


class _Phase(ctypes.Structure):
    """One fused BitLinear of mmf_decode_layers' device table (include/mmf.h)."""
    _fields_ = [("w1", ctypes.c_void_p), ("norm_w", ctypes.c_void_p), ("packed", ctypes.c_void_p), ("wdeq", ctypes.c_void_p),
                ("lb", ctypes.c_void_p), ("state", ctypes.c_void_p), ("inv_K", ctypes.c_double), ("eps", ctypes.c_float),
                ("eps1", ctypes.c_float), ("K", ctypes.c_int), ("N", ctypes.c_int), ("seg_rows", ctypes.c_int),
                ("pad", ctypes.c_int)]


class DecodeEngine:
    SPIN = 1 << 15      # polling rounds a resident workgroup waits for its input before it gives up (mmf_decode_layers)

    @classmethod
    def for_model(cls, model, batch_size: int, use_graph: bool = True, fuse: bool = True, resident: Optional[bool] = None):
        engines = model.__dict__.setdefault("_decode_engines", {})
        key = (batch_size, use_graph, fuse, resident)
        eng = engines.get(key)
        if eng is None or eng.stale():
            eng = cls(model, batch_size, use_graph, fuse, resident)
            engines[key] = eng
        return eng

    def __init__(self, model, batch_size: int, use_graph: bool = True, fuse: bool = True, resident: Optional[bool] = None):
        cfg = model.config
        if getattr(cfg, "use_short_conv", False):
            raise NotImplementedError("DecodeEngine has no convolution state: models with use_short_conv decode through "
                                      "the module path (generate() does so by itself)")
        self.lib = L.load()
        self.model = model
        self.B = B = batch_size
        emb = model.model.embeddings.weight
        self.dev = dev = L.require_gpu(emb)
        self.dtype = dt = emb.dtype
        self.dt_id = L.dtype_id(dt)
        self.H = H = cfg.hidden_size
        self.V = cfg.vocab_size
        self.L = len(model.model.layers)
        self.eps = float(cfg.rms_norm_eps)
        self.use_graph = use_graph
        self._version_key = self._param_versions()

        attn0 = model.model.layers[0].attn
        self.D = D = attn0.input_dim
        self.I = I = model.model.layers[0].mlp.intermediate_size
        lbs = model.model.lower_bound_rows() if cfg.use_lower_bound else None

        def z(*shape, dtype=dt):
            return torch.zeros(*shape, dtype=dtype, device=dev)

        # ---- per-layer operands (references keep the packed weights alive)
        self.layers = []
        for li, blk in enumerate(model.model.layers):
            a, m = blk.attn, blk.mlp
            ent = {
                "attn_norm": blk.attn_norm.weight.detach(), "mlp_norm": blk.mlp_norm.weight.detach(),
                "g_norm": a.g_norm.weight.detach(), "g_eps": float(a.g_norm.eps),
                "ifg": a._stacked_ifg(),
                "projs": [(p.packed_weight(), p.norm.weight.detach(), self._eps_of(p)) for p in (a.i_proj, a.f_proj, a.g_proj)],
                "o": (a.o_proj.packed_weight(), a.o_proj.norm.weight.detach(), self._eps_of(a.o_proj)),
                "gate": (m.gate_proj.packed_weight(), m.gate_proj.norm.weight.detach(), self._eps_of(m.gate_proj)),
                "down": (m.down_proj.packed_weight(), m.down_proj.norm.weight.detach(), self._eps_of(m.down_proj)),
                "lb": lbs[li].contiguous() if (lbs is not None and li > 0) else None,
                "state": z(B, D, dtype=torch.float32),
            }
            for p in (a.i_proj, a.f_proj, a.g_proj, a.o_proj, m.gate_proj, m.down_proj):
                if p.bias is not None:
                    raise NotImplementedError("DecodeEngine: BitLinear bias is not on the model path")
            self.layers.append(ent)
        self.final_norm = model.model.norm.weight.detach()
        self.head = (model.lm_head.packed_weight(), model.lm_head.norm.weight.detach(), self._eps_of(model.lm_head))
        self.table = emb.detach()

        # ---- static activation buffers
        self.tok = torch.zeros(B, dtype=torch.int64, device=dev)
        self.h = z(B, H)            # residual stream
        self.hn = z(B, H)
        self.ifg = z(B, 3 * D)
        self.o = z(B, D)
        self.o2 = z(B, D)
        self.a = z(B, H)
        self.res = z(B, H)
        self.y = z(B, 2 * I)
        self.zb = z(B, I)
        self.logits = z(B, self.V)
        kmax = max(H, D, I)
        self.q = torch.zeros(self.lib.mmf_codes_bytes(B, kmax, 1), dtype=torch.int8, device=dev)
        self.deq = z(B, dtype=torch.float32)
        self.qsum = torch.zeros(B, dtype=torch.int32, device=dev)
        self.gemv = B <= F_.GEMV_MAX_M
        self.fused = fuse and self._can_fuse()
        self.fused_mfma = fuse and self._can_fuse_mfma()
        # resident=None: the one-launch layer chain whenever the model fits it; True insists; False never
        self.resident = self.fused and resident is not False and self._can_run_resident()
        if resident and not self.resident:
            raise L.MMFError("DecodeEngine: this model / batch / device does not fit the resident layer chain")
        if self.resident:
            self._build_resident()
        self.graph = None

    @staticmethod
    def _eps_of(p):
        return float(p.norm.eps if getattr(p, "fused_eps", None) is None else p.fused_eps)

    def _param_versions(self):
        return tuple((p.data_ptr(), p._version) for p in self.model.parameters())

    def stale(self):
        return self._param_versions() != self._version_key

    # ------------------------------------------------------------------ launches
    def _bitlinear(self, x, pw_nw_eps, out, n_k, addend=None):
        pw, nw, eps = pw_nw_eps
        lib, s, B = self.lib, L.stream(), self.B
        n, k = n_k
        nw_id = L.dtype_id(nw.dtype)
        if self.gemv and k <= lib.mmf_bitlinear_gemv_max_k():
            L.check(lib.mmf_bitlinear_gemv(x.data_ptr(), nw.data_ptr(), pw.packed.data_ptr(), pw.wdeq.data_ptr(),
                                           pw.seg_rows, None, L.ptr(addend), out.data_ptr(), B, k, n, eps, self.dt_id,
                                           nw_id, s), "mmf_bitlinear_gemv")
        else:
            L.check(lib.mmf_rmsnorm_quant(x.data_ptr(), None, nw.data_ptr(), self.q.data_ptr(), self.deq.data_ptr(),
                                          self.qsum.data_ptr(), None, B, k, eps, self.dt_id, self.dt_id, nw_id, 1, s),
                    "mmf_rmsnorm_quant")
            L.check(lib.mmf_bitlinear_mfma(self.q.data_ptr(), self.deq.data_ptr(), self.qsum.data_ptr(),
                                           pw.packed.data_ptr(), pw.wdeq.data_ptr(), pw.seg_rows, None, L.ptr(addend),
                                           out.data_ptr(), n, B, k, n, self.dt_id, -1, s), "mmf_bitlinear_mfma")

    # prologue / epilogue ids of mmf_bitlinear_gemv_fused
    PLAIN, NORM, RESNORM, GATEDNORM, SWIGLU = 0, 1, 2, 3, 4
    E_PLAIN, E_STEP, E_SWIGLU = 0, 1, 2

    def _fused(self, pro, epi, x, ldx, aux, ldaux, res_out, w1, eps1, pw_nw_eps, out, g_out, lb, state, n, k,
               addend=None):
        pw, nw, eps = pw_nw_eps
        L.check(self.lib.mmf_bitlinear_gemv_fused(
            pro, epi, x.data_ptr(), ldx, L.ptr(aux), ldaux, L.ptr(res_out), L.ptr(w1), eps1, nw.data_ptr(), eps,
            pw.packed.data_ptr(), pw.wdeq.data_ptr(), pw.seg_rows, None, L.ptr(addend), out.data_ptr(), L.ptr(g_out),
            L.ptr(lb), L.ptr(state), self.B, k, n, self.dt_id, L.dtype_id(nw.dtype), L.stream()), "mmf_bitlinear_gemv_fused")

    # ------------------------------------------------------------------ resident layer chain (batch 1)
    def _can_run_resident(self):
        props = torch.cuda.get_device_properties(self.dev)
        return (self.B == 1 and self.dtype in (torch.bfloat16, torch.float16) and self.final_norm.dtype == self.dtype
                and self.D == self.H and self.H % 128 == 0 and self.I % 128 == 0 and self.H <= 4096 and self.I <= 8192
                and props.multi_processor_count >= 256)

    def _build_resident(self):
        H, D, I = self.H, self.D, self.I
        assert self.lib.mmf_decode_layers_phase_bytes() == ctypes.sizeof(_Phase)
        table = (_Phase * (4 * self.L + 1))()            # the last record is the final norm + lm_head

        def fill(rec, w1, eps1, pw_nw_eps, k, n, lb=None, state=None):
            pw, nw, eps = pw_nw_eps
            rec.w1 = w1.data_ptr() if w1 is not None else None
            rec.norm_w, rec.packed, rec.wdeq = nw.data_ptr(), pw.packed.data_ptr(), pw.wdeq.data_ptr()
            rec.lb = lb.data_ptr() if lb is not None else None
            rec.state = state.data_ptr() if state is not None else None
            rec.inv_K, rec.eps, rec.eps1, rec.K, rec.N, rec.seg_rows = 1.0 / k, eps, eps1, k, n, pw.seg_rows

        for li, ent in enumerate(self.layers):
            fill(table[4 * li], ent["attn_norm"], self.eps, (ent["ifg"], ent["projs"][0][1], ent["projs"][0][2]), H, 3 * D,
                 ent["lb"], ent["state"])
            fill(table[4 * li + 1], ent["g_norm"], ent["g_eps"], ent["o"], D, H)
            fill(table[4 * li + 2], ent["mlp_norm"], self.eps, ent["gate"], H, 2 * I)
            fill(table[4 * li + 3], None, 0.0, ent["down"], I, H)
        fill(table[4 * self.L], self.final_norm, self.eps, self.head, H, self.V)
        raw = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8)
        self.phases = raw.to(self.dev)
        # tagged hand-off words: every row in `copies` copies (one per XCD), [copies, n] each, in the kernel's order
        R = self.lib.mmf_decode_layers_copies()
        sizes = [H, H, D, D, H, I]                          # h0, h1, o, g, attn, z
        words = torch.zeros(self.lib.mmf_decode_layers_words(H, D, I), dtype=torch.int32, device=self.dev)
        self.words, off = [], 0
        for n in sizes:
            self.words.append(words[off:off + R * n].view(R, n))
            off += R * n
        assert off == words.numel()
        self._words = words
        self.am_words = torch.zeros(256, dtype=torch.int64, device=self.dev)
        self.epoch = torch.zeros(1, dtype=torch.int32, device=self.dev)
        self.err = torch.zeros(1, dtype=torch.int32, device=self.dev)

    def _launch_layers(self, with_head: bool, trace: Optional[torch.Tensor] = None, delay: int = 6):
        head = self.phases.data_ptr() + 4 * self.L * ctypes.sizeof(_Phase) if with_head else None
        args = (self.phases.data_ptr(), self.L, self.table.data_ptr(), self.tok.data_ptr(), self.V, self._words.data_ptr(),
                self.h.data_ptr(), head, self.logits.data_ptr(), self.am_words.data_ptr(), self.tok.data_ptr(),
                self.epoch.data_ptr(), self.err.data_ptr())
        if trace is None:
            L.check(self.lib.mmf_decode_layers(*args, self.H, self.D, self.I, self.SPIN, self.dt_id, L.stream()), "mmf_decode_layers")
        else:
            L.check(self.lib.mmf_decode_layers_traced(*args, trace.data_ptr(), self.H, self.D, self.I, self.SPIN, delay, self.dt_id,
                                                      L.stream()), "mmf_decode_layers_traced")

    def link_trace(self, delay: int = 6) -> torch.Tensor:
        """One resident step with the kernel's cycle trace on: int64 [256 workgroups, 128 links, 12 stamps] (see
        mmf_decode_layers_traced in include/mmf_diag.h), on the host."""
        assert self.resident
        t = torch.zeros(self.lib.mmf_decode_layers_trace_words(), dtype=torch.int64, device=self.dev)
        self._launch_layers(True, trace=t, delay=delay)
        torch.cuda.synchronize(self.dev)
        return t.view(256, 128, 12).cpu()

    def _launch_step_resident(self):
        self._launch_layers(True)       # the whole step: final norm, lm_head and argmax are the launch's last two links

    def resident_ok(self) -> bool:
        """False once a wait inside the resident layer chain ran out of polling rounds (host synchronisation)."""
        return not self.resident or int(self.err.item()) == 0

    def _reset_resident(self):
        """Bring the hand-off words back to their initial state.  A launch whose wait timed out may have had a late
        workgroup read the tag base after workgroup 0 advanced it (the base is only published safely when every poll
        succeeded), and so have left words that carry tags of the NEXT launch; a later launch would accept them as its
        own.  With every word, the tag base and the error word zero the next launch starts like the first one.  The
        caller has synchronised with the device (it has read the error word)."""
        self._words.zero_()
        self.am_words.zero_()
        self.epoch.zero_()
        self.err.zero_()

    def check(self):
        """Raise if a wait inside the resident layer chain timed out since the engine was built: its workgroups were
        not all resident at once (other work held CUs), so the steps since then are invalid.  One host synchronisation;
        callers run it once per generation, not per step.  The engine is reset and can be used again."""
        if not self.resident_ok():
            self._reset_resident()
            raise L.MMFError("DecodeEngine: a wait inside the resident layer chain timed out (were other kernels running "
                             "on this device?); the tokens of this generation are invalid. Build the engine with "
                             "resident=False to decode with one launch per BitLinear.")

    def _launch_step_fused(self, ends=True):
        """Batch <= GEMV_MAX_M: four launches per layer, every elementwise op folded into a GEMV.
        ends=False leaves out the embedding gather and the argmax (the 4L+1 GEMV launches only)."""
        lib, s, B, H, D, I = self.lib, L.stream(), self.B, self.H, self.D, self.I
        if ends:
            L.check(lib.mmf_embedding(self.table.data_ptr(), self.tok.data_ptr(), self.h.data_ptr(), B, H, self.V,
                                      self.dt_id, s), "mmf_embedding")
        g_buf = self.ifg.view(-1)[:B * D].view(B, D)
        for ent in self.layers:
            self._fused(self.NORM, self.E_STEP, self.h, H, None, 0, None, ent["attn_norm"], self.eps,
                        (ent["ifg"], ent["projs"][0][1], ent["projs"][0][2]), self.o, g_buf, ent["lb"], ent["state"],
                        3 * D, H)
            self._fused(self.GATEDNORM, self.E_PLAIN, g_buf, D, self.o, D, None, ent["g_norm"], ent["g_eps"], ent["o"],
                        self.a, None, None, None, H, D)
            self._fused(self.RESNORM, self.E_SWIGLU, self.a, H, self.h, H, self.res, ent["mlp_norm"], self.eps,
                        ent["gate"], self.zb, None, None, None, 2 * I, H)
            self._fused(self.PLAIN, self.E_PLAIN, self.zb, I, None, 0, None, None, 0.0, ent["down"], self.h, None, None,
                        None, H, I, addend=self.res)
        self._fused(self.NORM, self.E_PLAIN, self.h, H, None, 0, None, self.final_norm, self.eps, self.head, self.logits,
                    None, None, None, self.V, H)
        if ends:
            L.check(lib.mmf_argmax(self.logits.data_ptr(), self.V, B, self.V, self.tok.data_ptr(), self.dt_id, s),
                    "mmf_argmax")

    def fused_step_bytes(self, with_head: bool = True):
        """Algorithmic bytes of the 4L (+1 with head) fused BitLinears of one batch-B step: 2-bit weights once, plus
        each link's activation / norm-weight / state reads and its outputs."""
        B, H, D, I, V, e = self.B, self.H, self.D, self.I, self.V, self.h.element_size()
        per_layer = ((3 * D * H + H * D + 2 * I * H + H * I) // 4        # packed weights of i/f/g, o, gate, down
                     + B * (H * e + 2 * D * e + 8 * D) + 2 * H * e + 4 * D  # A: x; o, g out; state rd+wr; two norm weights, lb
                     + B * (2 * D * e + H * e) + 2 * D * e                  # B: g, o in; a out; two norm weights
                     + B * (2 * H * e + H * e + I * e) + 2 * H * e          # C: a, h in; res, z out; two norm weights
                     + B * (I * e + 2 * H * e) + I * e)                     # D: z, res in; h out; norm weight
        head = V * H // 4 + B * (H * e + V * e) + 2 * H * e
        return self.L * per_layer + (head if with_head else 0)

    def _qfused(self, pro, x, ldx, aux, ldaux, aux2, ldaux2, res_out, w1, eps1, nw, eps, lb, state, k):
        L.check(self.lib.mmf_rmsnorm_quant_fused(
            pro, x, ldx, aux, ldaux, aux2, ldaux2, L.ptr(res_out), L.ptr(w1), eps1, nw.data_ptr(), eps, L.ptr(lb),
            L.ptr(state), self.q.data_ptr(), self.deq.data_ptr(), self.qsum.data_ptr(), self.B, k, self.dt_id,
            L.dtype_id(nw.dtype), L.stream()), "mmf_rmsnorm_quant_fused")

    def _mfma(self, pw, out, n, k, addend=None):
        L.check(self.lib.mmf_bitlinear_mfma(self.q.data_ptr(), self.deq.data_ptr(), self.qsum.data_ptr(),
                                            pw.packed.data_ptr(), pw.wdeq.data_ptr(), pw.seg_rows, None, L.ptr(addend),
                                            out.data_ptr(), n, self.B, k, n, self.dt_id, -1, L.stream()), "mmf_bitlinear_mfma")

    def _launch_step_mfma_fused(self):
        """Batch > GEMV_MAX_M: eight launches per layer -- each BitLinear is a fused prologue+quantiser row kernel
        (norm / recurrence step + gated norm / residual norm / swiglu folded in) and a matrix-core contraction."""
        lib, s, B, H, D, I = self.lib, L.stream(), self.B, self.H, self.D, self.I
        esz = self.h.element_size()
        L.check(lib.mmf_embedding(self.table.data_ptr(), self.tok.data_ptr(), self.h.data_ptr(), B, H, self.V,
                                  self.dt_id, s), "mmf_embedding")
        ifg, y = self.ifg.data_ptr(), self.y.data_ptr()
        for ent in self.layers:
            nw, eps = ent["projs"][0][1], ent["projs"][0][2]
            self._qfused(1, self.h.data_ptr(), H, None, 0, None, 0, None, ent["attn_norm"], self.eps, nw, eps, None, None, H)
            self._mfma(ent["ifg"], self.ifg, 3 * D, H)
            self._qfused(3, ifg, 3 * D, ifg + D * esz, 3 * D, ifg + 2 * D * esz, 3 * D, None, ent["g_norm"], ent["g_eps"],
                         ent["o"][1], ent["o"][2], ent["lb"], ent["state"], D)
            self._mfma(ent["o"][0], self.a, H, D)
            self._qfused(2, self.a.data_ptr(), H, self.h.data_ptr(), H, None, 0, self.res, ent["mlp_norm"], self.eps,
                         ent["gate"][1], ent["gate"][2], None, None, H)
            self._mfma(ent["gate"][0], self.y, 2 * I, H)
            self._qfused(4, y, 2 * I, y + I * esz, 2 * I, None, 0, None, None, 0.0, ent["down"][1], ent["down"][2], None, None, I)
            self._mfma(ent["down"][0], self.h, H, I, addend=self.res)
        self._qfused(1, self.h.data_ptr(), H, None, 0, None, 0, None, self.final_norm, self.eps, self.head[1], self.head[2],
                     None, None, H)
        self._mfma(self.head[0], self.logits, self.V, H)
        L.check(lib.mmf_argmax(self.logits.data_ptr(), self.V, B, self.V, self.tok.data_ptr(), self.dt_id, s), "mmf_argmax")

    def _can_fuse_mfma(self):
        same_dt = all(t.dtype == self.final_norm.dtype for e in self.layers
                      for t in (e["attn_norm"], e["mlp_norm"], e["g_norm"], e["o"][1], e["gate"][1], e["down"][1],
                                e["projs"][0][1])) and self.head[1].dtype == self.final_norm.dtype
        return (not self.gemv and same_dt and all(e["ifg"] is not None for e in self.layers)
                and max(self.H, self.D, self.I) <= 8192 and (3 * self.D) % 8 == 0 and (2 * self.I) % 8 == 0)

    def _can_fuse(self):
        kmax = self.lib.mmf_bitlinear_gemv_max_k()
        same_dt = all(t.dtype == self.final_norm.dtype for e in self.layers
                      for t in (e["attn_norm"], e["mlp_norm"], e["g_norm"], e["o"][1], e["gate"][1], e["down"][1],
                                e["projs"][0][1])) and self.head[1].dtype == self.final_norm.dtype
        return (self.gemv and same_dt and all(e["ifg"] is not None for e in self.layers)
                and max(self.H, self.D, self.I) <= kmax and self.D % 32 == 0 and self.I % 32 == 0)

    def _launch_step(self):
        if self.resident:
            return self._launch_step_resident()
        if self.fused:
            return self._launch_step_fused()
        if self.fused_mfma:
            return self._launch_step_mfma_fused()
        lib, s, B, H, D, I = self.lib, L.stream(), self.B, self.H, self.D, self.I
        dt, esz = self.dt_id, self.h.element_size()
        wid = L.dtype_id(self.final_norm.dtype)
        L.check(lib.mmf_embedding(self.table.data_ptr(), self.tok.data_ptr(), self.h.data_ptr(), B, H, self.V, dt, s),
                "mmf_embedding")
        for ent in self.layers:
            L.check(lib.mmf_rmsnorm(self.h.data_ptr(), None, ent["attn_norm"].data_ptr(), self.hn.data_ptr(), None, B, H,
                                    self.eps, dt, dt, wid, s), "mmf_rmsnorm")
            if ent["ifg"] is not None:
                self._bitlinear(self.hn, (ent["ifg"], ent["projs"][0][1], ent["projs"][0][2]), self.ifg, (3 * D, H))
                ip, fp, gp, ld = self.ifg.data_ptr(), self.ifg.data_ptr() + D * esz, self.ifg.data_ptr() + 2 * D * esz, 3 * D
            else:
                # three separate projections into the three column blocks of a [3, B, D] layout
                bufs = self.ifg.view(3, B, D)
                for j in range(3):
                    self._bitlinear(self.hn, ent["projs"][j], bufs[j], (D, H))
                ip, fp, gp, ld = bufs[0].data_ptr(), bufs[1].data_ptr(), bufs[2].data_ptr(), D
            L.check(lib.mmf_hgrn_step(ip, ld, fp, ld, L.ptr(ent["lb"]), None, ent["state"].data_ptr(), self.o.data_ptr(),
                                      B, D, dt, s), "mmf_hgrn_step")
            L.check(lib.mmf_rmsnorm_swishgate(gp, ld, self.o.data_ptr(), None, ent["g_norm"].data_ptr(),
                                              self.o2.data_ptr(), None, B, D, ent["g_eps"], dt, dt, wid, s),
                    "mmf_rmsnorm_swishgate")
            self._bitlinear(self.o2, ent["o"], self.a, (H, D))
            L.check(lib.mmf_rmsnorm(self.a.data_ptr(), self.h.data_ptr(), ent["mlp_norm"].data_ptr(), self.hn.data_ptr(),
                                    self.res.data_ptr(), B, H, self.eps, dt, dt, wid, s), "mmf_rmsnorm")
            self._bitlinear(self.hn, ent["gate"], self.y, (2 * I, H))
            L.check(lib.mmf_swiglu(self.y.data_ptr(), 2 * I, self.y.data_ptr() + I * esz, 2 * I, self.zb.data_ptr(), B, I,
                                   dt, s), "mmf_swiglu")
            self._bitlinear(self.zb, ent["down"], self.h, (H, I), addend=self.res)
        L.check(lib.mmf_rmsnorm(self.h.data_ptr(), None, self.final_norm.data_ptr(), self.hn.data_ptr(), None, B, H,
                                self.eps, dt, dt, wid, s), "mmf_rmsnorm")
        self._bitlinear(self.hn, self.head, self.logits, (self.V, H))
        L.check(lib.mmf_argmax(self.logits.data_ptr(), self.V, B, self.V, self.tok.data_ptr(), dt, s), "mmf_argmax")

    def _capture(self):
        # warm-up launches on a side stream (module loading, attribute setting), then record
        saved = [e["state"].clone() for e in self.layers]
        tok = self.tok.clone()
        side = torch.cuda.Stream(device=self.dev)
        side.wait_stream(torch.cuda.current_stream(self.dev))
        with torch.cuda.stream(side):
            self._launch_step()
        torch.cuda.current_stream(self.dev).wait_stream(side)
        torch.cuda.synchronize(self.dev)
        if self.resident and not self.resident_ok():
            # the workgroups were not all resident at once (another stream or process holds CUs): use the launch chain
            warnings.warn("DecodeEngine: the resident layer chain timed out waiting for its workgroups; "
                          "falling back to one launch per BitLinear")
            self.resident = False
            self._reset_resident()
            for e, sv in zip(self.layers, saved):
                e["state"].copy_(sv)
            self.tok.copy_(tok)
            with torch.cuda.stream(side):
                self._launch_step()
            torch.cuda.current_stream(self.dev).wait_stream(side)
            torch.cuda.synchronize(self.dev)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._launch_step()
        torch.cuda.synchronize(self.dev)
        for e, sv in zip(self.layers, saved):     # undo the warm-up step's state update
            e["state"].copy_(sv)
        self.tok.copy_(tok)
        self.graph = g

    # ------------------------------------------------------------------ public
    def load_state(self, states: Optional[List[torch.Tensor]]):
        """Set the per-layer recurrent states ([B, *, D] tensors, or None for zeros)."""
        for i, e in enumerate(self.layers):
            if states is None:
                e["state"].zero_()
            else:
                e["state"].copy_(states[i].reshape(self.B, self.D).to(torch.float32))

    def export_state(self):
        return [e["state"].clone() for e in self.layers]

    def advance(self):
        """One decode step from the token buffer; leaves logits in self.logits and the greedy
        next token in the token buffer (no host synchronisation)."""
        with torch.cuda.device(self.dev):
            if not self.use_graph:
                self._launch_step()
                return
            if self.graph is None:
                self._capture()
            self.graph.replay()

    def step(self, tokens: torch.Tensor) -> torch.Tensor:
        """Feed `tokens` [B]; returns the logits buffer [B, V] (overwritten by the next step)."""
        self.tok.copy_(tokens.reshape(self.B))
        self.advance()
        return self.logits

    def greedy(self, first_tokens: torch.Tensor, n_steps: int) -> torch.Tensor:
        """Run n_steps self-feeding greedy steps starting from first_tokens [B]; returns the
        [B, n_steps] tokens chosen after each step.  One host synchronisation at the end."""
        out = torch.empty(n_steps, self.B, dtype=torch.int64, device=self.dev)
        self.tok.copy_(first_tokens.reshape(self.B))
        for t in range(n_steps):
            self.advance()
            out[t].copy_(self.tok)
        self.check()
        return out.t().contiguous()
