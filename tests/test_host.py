"""Host-side checks that need no GPU: the shared library loads and exports every symbol the public header
declares, argument validation, the cache and config mirrors, and loud failure on CPU tensors."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    """Every function the two public headers declare: the drop-in boundary (mmf.h) and the measuring aids (mmf_diag.h)."""
    syms = set()
    for name in ("mmf.h", "mmf_diag.h"):
        text = open(os.path.join(ROOT, "include", name)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        syms |= set(re.findall(r"\b(mmf_[a-z0-9_]+)\s*\(", text))
    return sorted(syms)


def test_library_exports_every_declared_symbol():
    from matmulfreellm_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m matmulfreellm_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    syms = header_symbols()
    assert len(syms) >= 18
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/ but not exported"
    assert sorted(_lib.SIGNATURES) == syms, "ctypes signature table and header disagree"


def test_size_helpers_need_no_gpu():
    from matmulfreellm_amd import _lib
    lib = _lib.load()
    assert lib.mmf_packed_bytes(2048, 2048) == 2048 * 2048 // 4
    assert lib.mmf_packed_bytes(33, 129) == 2 * 2 * 1024                # padded to 64 x 256
    assert lib.mmf_codes_bytes(5, 300, 0) == 5 * 384 and lib.mmf_codes_bytes(5, 300, 1) == 32 * 384
    assert lib.mmf_ternarize_workspace_bytes() == 8192
    assert lib.mmf_bitlinear_gemv_max_k() == 8192


def test_argument_errors_are_codes_not_crashes():
    from matmulfreellm_amd import _lib
    lib = _lib.load()
    assert lib.mmf_rmsnorm(None, None, None, None, None, 4, 64, 1e-6, 1, 1, 1, None) == -1       # null x
    assert lib.mmf_rmsnorm(None, None, None, None, None, 0, 64, 1e-6, 1, 1, 1, None) == 0        # empty is fine
    assert lib.mmf_hgrn_chunk(None, None, None, None, None, 0, 0, 64, 100, 1, None, None) == -1        # chunk > 64
    assert lib.mmf_bitlinear_mfma(None, None, None, None, None, 32, None, None, None, 8, 4, 64, 16, 1, -1, None) == -1


def test_cpu_tensors_fail_loudly():
    import matmulfreellm_amd as mm
    from matmulfreellm_amd._lib import MMFError
    with pytest.raises(MMFError):
        mm.RMSNorm(64)(torch.randn(2, 64))
    with pytest.raises(MMFError):
        mm.FusedBitLinear(64, 32)(torch.randn(2, 64))
    with pytest.raises(MMFError):
        mm.fused_recurrent_hgrn(torch.randn(1, 1, 4, 8), torch.rand(1, 1, 4, 8))
    with pytest.raises(MMFError):
        mm.swiglu(torch.randn(4), torch.randn(4))


def test_recurrent_cache_semantics():
    from matmulfreellm_amd import RecurrentCache
    c = RecurrentCache.from_legacy_cache([(torch.zeros(2, 1, 4),), (torch.zeros(2, 1, 4),)])
    assert len(c) == 2 and c.get_seq_length() == 0
    s0 = c[0][0]
    c.update((torch.ones(2, 1, 4),), 0)
    assert c.get_seq_length() == 0 and torch.equal(s0, torch.ones(2, 1, 4))      # copied in place
    c.update((torch.ones(2, 1, 4),), 1)
    assert c.get_seq_length() == 1                                                 # counted at the last layer
    with pytest.raises(KeyError):
        c[2]
    c.reorder_cache(torch.tensor([1, 0]))
    assert isinstance(c.to_legacy_cache(), tuple) and c.get_max_length() is None


def test_config_and_module_tree_mirror_the_reference():
    import matmulfreellm_amd as mm
    cfg = mm.HGRNBitConfig()
    assert (cfg.vocab_size, cfg.hidden_size, cfg.num_hidden_layers, cfg.num_heads, cfg.use_lower_bound,
            cfg.rms_norm_eps, cfg.attn_mode, cfg.model_type) == (32000, 2048, 24, 1, True, 1e-6, "fused_recurrent", "hgrn_bit")
    with torch.device("meta"):
        model = mm.HGRNBitForCausalLM(mm.HGRNBitConfig(hidden_size=512, num_hidden_layers=2))
    keys = set(model.state_dict().keys())
    for k in ["model.embeddings.weight", "model.lower_bounds", "model.layers.0.attn_norm.weight",
              "model.layers.1.attn.i_proj.weight", "model.layers.1.attn.f_proj.norm.weight",
              "model.layers.0.attn.g_norm.weight", "model.layers.0.attn.o_proj.weight", "model.layers.0.mlp_norm.weight",
              "model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.down_proj.norm.weight", "model.norm.weight",
              "lm_head.weight", "lm_head.norm.weight"]:
        assert k in keys, k
    assert model.model.layers[0].mlp.intermediate_size == 1536
    assert tuple(model.model.layers[0].mlp.gate_proj.weight.shape) == (3072, 512)
    assert model.lm_head.norm.eps == 1e-8


def test_layer_norm_linear_quant_fn_rejects_unsupported_forms():
    import matmulfreellm_amd as mm
    x, w = torch.randn(2, 64), torch.randn(8, 64)
    with pytest.raises(NotImplementedError):           # the LayerNorm form has no backward
        mm.layer_norm_linear_quant_fn(x.clone().requires_grad_(), torch.ones(64), None, w, None, is_rms_norm=False)
    with pytest.raises(RuntimeError):                  # and, like every op here, no CPU path
        mm.layer_norm_linear_quant_fn(x, torch.ones(64), None, w, None, is_rms_norm=False)
    with pytest.raises(NotImplementedError):           # a norm bias exists for the LayerNorm form only
        mm.layer_norm_linear_quant_fn(x, torch.ones(64), torch.zeros(64), w, None, is_rms_norm=True)
    attn = mm.HGRNBitAttention(hidden_size=64, num_heads=1, use_short_conv=True, share_conv_kernel=False)
    assert isinstance(attn.i_conv1d, mm.ShortConvolution) and attn.state_size() == 64 + 3 * 64 * 4
    assert [tuple(s.shape) for s in attn.init_state(2)] == [(2, 64, 4), (2, 64, 4), (2, 1, 64)]


def test_division_free_quotient_is_the_correctly_rounded_one():
    """The kernels' rstd uses q = s*y; q = fma(fma(-q,K,s), y, q) twice with y = RN(1/K) in place of
    the fp64 division s / K (csrc/mmf_common.h, mmf_rstd).  Check the sequence against exact
    rational arithmetic: it must give the correctly rounded quotient, i.e. what `/` gives."""
    from fractions import Fraction
    import random

    def fma(a, b, c):
        return float(Fraction(a) * Fraction(b) + Fraction(c))       # one rounding, like the hardware's

    rng = random.Random(7)
    for K in (1, 3, 7, 11, 100, 127, 2048, 5632, 8191, 4096, 33, 999, 65537, 100003):
        y, Kd = 1.0 / K, float(K)
        for _ in range(1500):
            s = rng.random() * 10.0 ** rng.randint(-20, 12)
            q = s * y
            q = fma(fma(-q, Kd, s), y, q)
            q = fma(fma(-q, Kd, s), y, q)
            assert q == s / Kd, (K, s)


def test_reference_format_checkpoint_round_trip(tmp_path):
    """save_pretrained / from_pretrained keep the reference's state-dict keys and values (no GPU needed:
    nothing is packed until a BitLinear runs)."""
    import matmulfreellm_amd as mm
    cfg = mm.HGRNBitConfig(vocab_size=64, hidden_size=64, num_hidden_layers=2)
    torch.manual_seed(0)
    m = mm.HGRNBitForCausalLM(cfg)
    m.save_pretrained(tmp_path)
    m2 = mm.HGRNBitForCausalLM.from_pretrained(tmp_path)
    a, b = m.state_dict(), m2.state_dict()
    assert set(a) == set(b)
    assert all(torch.equal(a[k], b[k]) for k in a)
    for key in ("model.embeddings.weight", "model.lower_bounds", "model.layers.0.attn.i_proj.weight",
                "model.layers.0.attn.i_proj.norm.weight", "model.layers.1.mlp.down_proj.norm.weight", "lm_head.weight"):
        assert key in a


def test_packed_checkpoint_loader_rejects_foreign_files(tmp_path):
    import matmulfreellm_amd as mm
    from matmulfreellm_amd import checkpoint as ck
    from safetensors.torch import save_file
    cfg = mm.HGRNBitConfig(vocab_size=64, hidden_size=64, num_hidden_layers=1)
    cfg.save_pretrained(tmp_path)
    save_file({"x": torch.zeros(1)}, str(tmp_path / ck.PACKED_FILE), metadata={"format": "something-else"})
    with pytest.raises(ValueError):
        ck.load_packed(tmp_path, device="cpu")
    save_file({"x": torch.zeros(1)}, str(tmp_path / ck.PACKED_FILE), metadata={"format": ck.FORMAT})
    with pytest.raises(KeyError):
        ck.load_packed(tmp_path, device="cpu")


def test_rejected_shapes_and_pointers_return_their_code_before_any_launch():
    """MMF_ERR_ARG -1, MMF_ERR_WIDE -2, MMF_ERR_ALIGN -3 (include/mmf.h): every check below sits in front of the
    first kernel launch, so the calls are safe without a GPU (the fake non-null pointers are never dereferenced)."""
    from matmulfreellm_amd import _lib
    lib = _lib.load()
    P = 4096                                                    # a non-null, 16-byte aligned stand-in
    # fused GEMV: row too wide for one workgroup's passes; misaligned packed weights; bad prologue / epilogue ids
    gemv = lambda pro, epi, k, packed=P, n=32, ldx=None: lib.mmf_bitlinear_gemv_fused(
        pro, epi, P, ldx if ldx is not None else k, None, 0, None, None, 0.0, P, 1e-8, packed, P, 32, None, None, P, None, None,
        None, 1, k, n, 1, 1, None)
    assert gemv(0, 0, 9000) == -2
    assert gemv(0, 0, 2048, packed=P + 8) == -3
    assert gemv(7, 0, 2048) == -1 and gemv(0, 3, 2048) == -1
    assert gemv(2, 0, 2048) == -1                               # residual prologue without its second operand
    assert gemv(0, 0, 2048, ldx=100) == -1                      # row stride shorter than the row
    assert gemv(0, 1, 2048, n=100) == -1                        # the recurrence-step epilogue wants N = 3 * 32 * j
    assert lib.mmf_bitlinear_gemv_fused(0, 0, P, 64, None, 0, None, None, 0.0, P, 1e-8, P, P, 32, None, None, P, None, None,
                                        None, 0, 64, 32, 1, 1, None) == 0      # no rows: nothing to do
    # fused quantiser
    fq = lambda pro, k: lib.mmf_rmsnorm_quant_fused(pro, P, k, P, k, None, 0, None, P, 1e-6, P, 1e-8, None, None, P, P, P, 3, k,
                                                    1, 1, None)
    assert fq(9, 2048) == -1 and fq(-1, 2048) == -1              # 0 is the plain prologue
    assert fq(1, 20000) == -2
    assert lib.mmf_rmsnorm_quant_fused(1, P + 2, 2048, None, 0, None, 0, None, P, 1e-6, P, 1e-8, None, None, P, P, P, 3, 2048,
                                       1, 1, None) == -3
    # matrix cores: segments must be whole 32-row blocks
    assert lib.mmf_bitlinear_mfma(P, P, P, P, P, 33, None, None, P, 64, 8, 128, 64, 1, -1, None) == -1
    # scans: too many (batch, head) pairs for one grid; a 64-step chunk that does not fit 32-bit offsets
    assert lib.mmf_hgrn_recurrent(P, P, None, P, None, 70000, 4, 64, 1, None) == -1
    assert lib.mmf_hgrn_recurrent(P, P, None, P, None, 1, 4, 1 << 24, 1, None) == -2
    assert lib.mmf_hgrn_recurrent(None, None, None, None, None, 0, 4, 64, 1, None) == 0
    # gate math: row stride shorter than the row
    assert lib.mmf_hgrn_gate(P, 32, P, 64, None, None, P, P, 2, 64, 1, None) == -1
    # resident layer chain: D must equal H, rows are whole k-blocks, 16-bit activations only, bounded widths, aligned rows
    # arguments: phases, n_layers, table, tok, vocab, words, h_out, head, logits, am_words, tok_out, epoch, err, H, D, I, spin, dtype
    layers = lambda h, d, i, dtype=1, words=P, spin=100: lib.mmf_decode_layers(P, 2, P, P, 1000, words, P, None, None, None, None, P, P,
                                                                             h, d, i, spin, dtype, None)
    assert layers(512, 256, 1536) == -1 and layers(500, 500, 1536) == -1 and layers(512, 512, 1500) == -1
    assert layers(512, 512, 1536, dtype=0) == -1 and layers(512, 512, 1536, spin=0) == -1
    assert layers(4224, 4224, 4096) == -2 and layers(2048, 2048, 8320) == -2
    assert layers(512, 512, 1536, words=P + 4) == -3
    assert lib.mmf_decode_layers(None, 2, P, P, 1000, P, P, None, None, None, None, P, P, 512, 512, 1536, 100, 1, None) == -1
    assert lib.mmf_decode_layers(P, 2, P, P, 1000, P, P, P, None, P, P, P, P, 512, 512, 1536, 100, 1,
                                 None) == -1                      # a head record without its logits buffer
    assert lib.mmf_decode_layers_traced(P, 2, P, P, 1000, P, P, None, None, None, None, P, P, None, 512, 512, 1536, 100, 6, 1,
                                        None) == -1               # the traced form needs its trace buffer
    assert lib.mmf_decode_layers_copies() == 8
    assert lib.mmf_decode_layers_words(512, 512, 1536) == 8 * (5 * 512 + 1536)
    assert lib.mmf_decode_layers_trace_words() == 256 * 128 * 12
    assert lib.mmf_decode_layers_phase_bytes() == 80


def test_generation_mixin_wiring():
    """The causal LM is a transformers GenerationMixin model that brings its own cache: transformers must not
    build a key/value cache for it, prepare_inputs_for_generation feeds only the new tokens once state exists,
    and a call on CPU tensors reaches the HIP-only forward (there is no CPU path to fall back to)."""
    import pytest
    from transformers.generation import GenerationMixin
    from matmulfreellm_amd.modeling_hgrn_bit import HGRNBitForCausalLM
    from matmulfreellm_amd.configuration_hgrn_bit import HGRNBitConfig
    from matmulfreellm_amd.cache import RecurrentCache
    from matmulfreellm_amd._lib import MMFError
    model = HGRNBitForCausalLM(HGRNBitConfig(vocab_size=64, hidden_size=64, num_hidden_layers=2, num_heads=1))
    assert isinstance(model, GenerationMixin) and model.can_generate()
    assert model._is_stateful and not model._supports_default_dynamic_cache()
    ids = torch.arange(10).view(2, 5)
    mask = torch.ones(2, 5, dtype=torch.long)
    first = model.prepare_inputs_for_generation(ids, attention_mask=mask, use_cache=True, logits_to_keep=1,
                                                is_first_iteration=True)
    assert first["input_ids"].shape == (2, 5) and first["past_key_values"] is None and first["logits_to_keep"] == 1
    cache = RecurrentCache()
    for layer in range(2):
        cache.update((torch.zeros(2, 64),), layer)
    for kw in ({"next_sequence_length": 1}, {}, {"next_sequence_length": 2}):
        step = model.prepare_inputs_for_generation(ids, past_key_values=cache, attention_mask=mask, use_cache=True, **kw)
        n = kw.get("next_sequence_length", 1)
        assert torch.equal(step["input_ids"], ids[:, -n:]) and step["attention_mask"].shape == (2, n)
        assert step["past_key_values"] is cache
    with pytest.raises(MMFError):
        model.generate(ids, attention_mask=mask, max_new_tokens=2, num_beams=2, pad_token_id=0)
    with pytest.raises(MMFError):
        model.generate(ids, max_new_tokens=2)
