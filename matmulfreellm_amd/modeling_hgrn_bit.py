"""HGRNBit model family on the HIP kernels.

Same module tree, parameter names and forward semantics as
mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py (MLP :29-59, Block :62-113, PreTrainedModel
:116-156, Model :159-278, ForCausalLM :281-409), so a checkpoint's state dict loads as is.
Differences, all on the host side:
  * the recurrent state cache is this package's RecurrentCache; ``generate()`` runs a greedy / top-p loop
    owned by the class on the captured decode graph for the arguments the reference's generate.py uses, and
    hands every other call (beams, logits processors, stopping criteria, streamers, a GenerationConfig) to
    transformers' GenerationMixin, which the class inherits explicitly (transformers >= 5 no longer gives
    PreTrainedModel a generate());
  * ``logits_to_keep`` lets a caller ask for the last positions' logits only (the
    reference projects all T positions through the 32000-wide head);
  * ``labels`` gives the evaluation loss (forward only, fp32): there is no backward.
"""
from __future__ import annotations

import math
import warnings
from typing import List, Optional, Tuple, Union

import torch
import torch.nn as nn
from transformers.generation import GenerationMixin
from transformers.modeling_outputs import BaseModelOutputWithPast, CausalLMOutputWithPast
from transformers.modeling_utils import PreTrainedModel

from . import functional as F_
from .activations import swiglu
from .attention import HGRNBitAttention
from .autograd import module_needs_grad
from .bitlinear import FusedBitLinear as BitLinear
from .cache import RecurrentCache
from .configuration_hgrn_bit import HGRNBitConfig
from .layernorm import RMSNorm


def lower_bound_schedule(lower_bounds: torch.Tensor) -> torch.Tensor:
    """softmax over layers, cumulative sum, minus the first row (modeling_hgrn_bit.py:231-233).

    Evaluated in fp32 on the host so the values do not depend on a device reduction order;
    returns an fp32 [L, H] tensor on the parameter's device."""
    lb = lower_bounds.detach().to(device="cpu", dtype=torch.float32).softmax(0)
    lb = lb.cumsum(0) - lb[0]
    return lb.to(lower_bounds.device)


class HGRNBitMLP(nn.Module):

    def __init__(self, hidden_size: int, hidden_ratio: Optional[int] = None, intermediate_size: Optional[int] = None,
                 hidden_act: str = "swish", bitlinear_eps: Optional[float] = 1e-6):
        super().__init__()
        self.hidden_size = hidden_size
        if hidden_ratio is None:
            hidden_ratio = 4
        if intermediate_size is None:
            intermediate_size = int(hidden_size * hidden_ratio * 2 / 3)
            intermediate_size = 256 * ((intermediate_size + 256 - 1) // 256)
        self.hidden_ratio = hidden_ratio
        self.intermediate_size = intermediate_size
        if hidden_act not in ("swish", "silu"):
            raise NotImplementedError(f"hidden_act={hidden_act!r}: the fused gate is swish")
        self.gate_proj = BitLinear(self.hidden_size, self.intermediate_size * 2, bias=False, fused_eps=bitlinear_eps)
        self.down_proj = BitLinear(self.intermediate_size, self.hidden_size, bias=False, fused_eps=bitlinear_eps)

    def forward(self, x, residual=None, pre_norm=None):
        """down_proj(swiglu(gate, y)) as mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:55-59.

        The swiglu is folded into down_proj's quantiser.  With ``residual`` the block's closing add is
        fused into down_proj's epilogue; with ``pre_norm`` (the block's mlp_norm) x is the attention
        output and the residual add + RMSNorm in front of gate_proj (:107) is folded into gate_proj."""
        inter = self.intermediate_size
        if module_needs_grad(self, x, residual):
            # the reference's composition (:55-59) through the autograd Functions; the block's norm and residual as :107-109
            from .activations import swiglu
            if pre_norm is not None:
                x, residual = pre_norm(x, residual, True)
            y = self.gate_proj(x)
            z = self.down_proj(swiglu(y[..., :inter], y[..., inter:]))
            return z if residual is None else residual + z
        rows = x.numel() // x.shape[-1]
        # long prompts: the tiled gate/up contraction applies the swiglu itself and down_proj quantises its result
        in_epilogue = (self.gate_proj.bias is None and x.is_cuda
                       and F_.swiglu_epilogue_fits(rows, self.gate_proj.packed_weight(), x.dtype))
        epilogue = "swiglu" if in_epilogue else None
        if pre_norm is not None:
            y, residual = self.gate_proj.forward_fused(x, ("resnorm", residual, pre_norm.weight, pre_norm.eps), epilogue=epilogue)
        elif in_epilogue:
            y = self.gate_proj.forward_fused(x, None, epilogue=epilogue)
        else:
            y = self.gate_proj(x)
        addend = residual.contiguous() if residual is not None else None
        if in_epilogue:
            return self.down_proj.forward_fused(y, None, addend=addend)
        return self.down_proj.forward_fused(y[..., :inter], ("swiglu", y[..., inter:]), addend=addend)


class HGRNBitBlock(nn.Module):

    def __init__(self, config: HGRNBitConfig, layer_idx: int):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.attn_norm = RMSNorm(hidden_size=config.hidden_size, eps=config.rms_norm_eps)
        self.attn = HGRNBitAttention(
            mode=config.attn_mode, hidden_size=config.hidden_size, num_heads=config.num_heads,
            expand_ratio=config.expand_ratio, use_short_conv=config.use_short_conv, conv_size=config.conv_size,
            share_conv_kernel=config.share_conv_kernel, layernorm_eps=config.rms_norm_eps, layer_idx=layer_idx,
            bitlinear_eps=getattr(config, "bitlinear_eps", 1e-6))
        self.mlp_norm = RMSNorm(hidden_size=config.hidden_size, eps=config.rms_norm_eps)
        self.mlp = HGRNBitMLP(hidden_size=config.hidden_size, hidden_ratio=config.hidden_ratio,
                              intermediate_size=config.intermediate_size, hidden_act=config.hidden_act,
                              bitlinear_eps=getattr(config, "bitlinear_eps", 1e-6))

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_values=None, use_cache: Optional[bool] = False, output_attentions: Optional[bool] = False,
                lower_bound: Optional[torch.Tensor] = None, **kwargs):
        # the reference's op sequence (:97-111) with every norm folded into the BitLinear that consumes it
        residual = hidden_states
        hidden_states, attentions, past_key_values = self.attn(
            hidden_states=hidden_states, attention_mask=attention_mask, past_key_values=past_key_values,
            use_cache=use_cache, output_attentions=output_attentions, lower_bound=lower_bound, input_norm=self.attn_norm)
        hidden_states = self.mlp(hidden_states, residual=residual, pre_norm=self.mlp_norm)   # = residual' + mlp(norm(residual'))
        return hidden_states, attentions, past_key_values


class HGRNBitPreTrainedModel(PreTrainedModel):
    config_class = HGRNBitConfig
    base_model_prefix = "model"
    supports_gradient_checkpointing = False
    _no_split_modules = ["HGRNBitBlock"]

    def _init_weights(self, module: nn.Module, rescale_prenorm_residual: bool = True, num_residuals_per_layer: int = 2):
        if isinstance(module, (nn.Linear, nn.Conv1d)):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.initializer_range)
            if module.bias is not None:
                nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.initializer_range)
            if module.padding_idx is not None:
                module.weight.data[module.padding_idx].zero_()
        elif isinstance(module, HGRNBitModel) and getattr(module, "lower_bounds", None) is not None:
            nn.init.zeros_(module.lower_bounds)
        if hasattr(module, "weight") and module.weight is not None and type(module).__name__ in (
                "RMSNorm", "FusedRMSNormSwishGate"):
            nn.init.ones_(module.weight)
        if rescale_prenorm_residual:
            for name, p in module.named_parameters():
                if name in ["o_proj.weight", "down_proj.weight"]:
                    with torch.no_grad():
                        p /= math.sqrt(num_residuals_per_layer * self.config.num_hidden_layers)


class HGRNBitModel(HGRNBitPreTrainedModel):

    def __init__(self, config: HGRNBitConfig):
        super().__init__(config)
        self.padding_idx = config.pad_token_id
        self.vocab_size = config.vocab_size
        self.embeddings = nn.Embedding(config.vocab_size, config.hidden_size, self.padding_idx)
        if config.use_lower_bound:
            self.lower_bounds = nn.Parameter(torch.zeros(config.num_hidden_layers, config.hidden_size))
        self.layers = nn.ModuleList([HGRNBitBlock(config, i) for i in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.gradient_checkpointing = False
        self._lb_key, self._lb = None, None
        self.post_init()

    def get_input_embeddings(self):
        return self.embeddings

    def set_input_embeddings(self, value):
        self.embeddings = value

    def lower_bound_rows(self):
        """fp32 [L, H] lower bounds, recomputed only when the parameter changes."""
        p = self.lower_bounds
        key = (p.data_ptr(), p._version, p.device)
        if key != self._lb_key:
            self._lb_key, self._lb = key, lower_bound_schedule(p)
        return self._lb

    def forward(self, input_ids: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None,
                inputs_embeds: Optional[torch.FloatTensor] = None, past_key_values=None,
                use_cache: Optional[bool] = None, output_attentions: Optional[bool] = None,
                output_hidden_states: Optional[bool] = None, return_dict: Optional[bool] = None
                ) -> Union[Tuple, BaseModelOutputWithPast]:
        """With gradients enabled and a parameter or the input embeddings requiring one -- in train or eval mode, as the
        reference -- the forward runs the reference's op-by-op composition through the autograd Functions
        (matmulfreellm_amd/autograd.py); everything else (torch.no_grad(), generate()) runs the fused inference launches
        without a graph."""
        train = module_needs_grad(self, inputs_embeds)
        with torch.enable_grad() if train else torch.no_grad():
            return self._forward(train, input_ids, attention_mask, inputs_embeds, past_key_values, use_cache,
                                 output_attentions, output_hidden_states, return_dict)

    def _forward(self, train, input_ids, attention_mask, inputs_embeds, past_key_values, use_cache, output_attentions,
                 output_hidden_states, return_dict):
        if output_attentions:
            warnings.warn("`HGRNBitModel` does not `output_attentions` now, setting it to `False`.")
        output_attentions = False
        output_hidden_states = bool(output_hidden_states) if output_hidden_states is not None else \
            bool(getattr(self.config, "output_hidden_states", False))
        use_cache = use_cache if use_cache is not None else (self.config.use_cache if not train else False)
        return_dict = return_dict if return_dict is not None else bool(getattr(self.config, "return_dict", True))

        if input_ids is not None and inputs_embeds is not None:
            raise ValueError("You cannot specify both input_ids and inputs_embeds at the same time")
        elif input_ids is not None:
            batch_size = input_ids.shape[0]
        elif inputs_embeds is not None:
            batch_size = inputs_embeds.shape[0]
        else:
            raise ValueError("You have to specify either input_ids or inputs_embeds")

        if inputs_embeds is None:
            inputs_embeds = self.embeddings(input_ids) if train else F_.embedding(self.embeddings.weight, input_ids)
        hidden_states = inputs_embeds
        if train:
            use_cache = False                                    # whole sequences, no recurrent-state cache

        if use_cache:
            if past_key_values is None:
                past_key_values = [layer.attn.init_state(batch_size) for layer in self.layers]
            if not isinstance(past_key_values, RecurrentCache):
                past_key_values = RecurrentCache.from_legacy_cache(past_key_values)

        all_hidden_states = () if output_hidden_states else None
        if not self.config.use_lower_bound:
            lower_bounds = None
        elif train:                                              # differentiable (modeling_hgrn_bit.py:231-233)
            lower_bounds = self.lower_bounds.float().softmax(0)
            lower_bounds = lower_bounds.cumsum(0) - lower_bounds[0]
        else:
            lower_bounds = self.lower_bound_rows()
        for i, layer in enumerate(self.layers):
            if output_hidden_states:
                all_hidden_states += (hidden_states,)
            lower_bound = lower_bounds[i] if lower_bounds is not None else None
            hidden_states, _, past_key_values = layer(
                hidden_states, attention_mask=attention_mask, past_key_values=past_key_values, use_cache=use_cache,
                output_attentions=False, lower_bound=lower_bound)

        hidden_states = self.norm(hidden_states)
        if output_hidden_states:
            all_hidden_states += (hidden_states,)

        next_cache = past_key_values if use_cache else None
        if not return_dict:
            return tuple(x for x in [hidden_states, next_cache, all_hidden_states] if x is not None)
        return BaseModelOutputWithPast(last_hidden_state=hidden_states, past_key_values=next_cache,
                                       hidden_states=all_hidden_states, attentions=None)


class HGRNBitForCausalLM(HGRNBitPreTrainedModel, GenerationMixin):
    _tied_weights_keys = {}
    # the recurrent state cannot be rolled back to an earlier position: GenerationMixin refuses assisted decoding
    _is_stateful = True

    @classmethod
    def _supports_default_dynamic_cache(cls) -> bool:
        """GenerationMixin must not build a key/value cache: the first forward creates the RecurrentCache."""
        return False

    def __init__(self, config):
        super().__init__(config)
        self.model = HGRNBitModel(config)
        self.vocab_size = config.vocab_size
        self.lm_head = BitLinear(config.hidden_size, config.vocab_size, bias=False, fused_eps=getattr(config, "bitlinear_eps", 1e-6))
        self.post_init()

    def get_input_embeddings(self):
        return self.model.embeddings

    def set_input_embeddings(self, value):
        self.model.embeddings = value

    def get_output_embeddings(self):
        return self.lm_head

    def set_output_embeddings(self, new_embeddings):
        self.lm_head = new_embeddings

    def set_decoder(self, decoder):
        self.model = decoder

    def get_decoder(self):
        return self.model

    def prepare_inputs_for_generation(self, input_ids: torch.LongTensor = None, past_key_values=None,
                                      attention_mask: Optional[torch.Tensor] = None,
                                      inputs_embeds: Optional[torch.Tensor] = None,
                                      next_sequence_length: Optional[int] = None,
                                      is_first_iteration: Optional[bool] = None, **kwargs):
        """modeling_hgrn_bit.py:326-354: once a cache holds state, only the new tokens are fed.

        Called by GenerationMixin with the whole sequence so far and a mask of the same length.
        ``next_sequence_length`` (transformers >= 5) says how many trailing tokens are new; older
        releases do not pass it and always mean one."""
        has_state = past_key_values is not None and len(past_key_values) > 0
        if has_state:
            if not isinstance(past_key_values, RecurrentCache):
                past_key_values = RecurrentCache.from_legacy_cache(past_key_values, input_ids.shape[1] - 1)
            n_new = next_sequence_length if next_sequence_length is not None else 1
            input_ids = input_ids[:, -n_new:]
            if attention_mask is not None:
                attention_mask = attention_mask[:, -n_new:]
        elif next_sequence_length is not None:
            input_ids = input_ids[:, -next_sequence_length:]
            if attention_mask is not None:
                attention_mask = attention_mask[:, -next_sequence_length:]
        if inputs_embeds is not None and not has_state:
            model_inputs = {"inputs_embeds": inputs_embeds}
        else:
            model_inputs = {"input_ids": input_ids.contiguous()}
        model_inputs.update({"past_key_values": past_key_values, "use_cache": kwargs.get("use_cache"),
                             "attention_mask": attention_mask})
        if kwargs.get("logits_to_keep") is not None:
            model_inputs["logits_to_keep"] = kwargs["logits_to_keep"]
        return model_inputs

    def forward(self, input_ids: torch.LongTensor = None, attention_mask: Optional[torch.Tensor] = None,
                inputs_embeds: Optional[torch.Tensor] = None, past_key_values=None,
                labels: Optional[torch.LongTensor] = None, use_cache: Optional[bool] = None,
                output_attentions: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                return_dict: Optional[bool] = None, logits_to_keep: int = 0) -> Union[Tuple, CausalLMOutputWithPast]:
        train = module_needs_grad(self, inputs_embeds)
        with torch.enable_grad() if train else torch.no_grad():
            return self._forward(train, input_ids, attention_mask, inputs_embeds, past_key_values, labels, use_cache,
                                 output_attentions, output_hidden_states, return_dict, logits_to_keep)

    def _forward(self, train, input_ids, attention_mask, inputs_embeds, past_key_values, labels, use_cache, output_attentions,
                 output_hidden_states, return_dict, logits_to_keep):
        if labels is not None:
            logits_to_keep = 0                           # the loss scores every position
        return_dict = return_dict if return_dict is not None else bool(getattr(self.config, "return_dict", True))
        outputs = self.model(input_ids=input_ids, attention_mask=attention_mask, inputs_embeds=inputs_embeds,
                             past_key_values=past_key_values, use_cache=use_cache,
                             output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                             return_dict=True)
        hidden_states = outputs.last_hidden_state
        if logits_to_keep:
            hidden_states = hidden_states[:, -logits_to_keep:, :]
        logits = self.lm_head(hidden_states)
        loss = None
        if labels is not None:
            # as mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:388-397: position t is scored against token t + 1
            labels = labels.to(logits.device)
            targets = torch.cat((labels[..., 1:], torch.full_like(labels[:, :1], -100)), 1)
            if train:
                # FusedCrossEntropyLoss(inplace_backward=True) as :389-391 (nn.CrossEntropyLoss gives the same value)
                from .autograd import FusedCrossEntropyLoss
                loss = FusedCrossEntropyLoss(inplace_backward=True)(logits.view(-1, logits.shape[-1]), targets.view(-1))
            else:
                loss = F_.cross_entropy(logits, targets, ignore_index=-100)
        if not return_dict:
            return tuple(x for x in (loss, logits, outputs.past_key_values, outputs.hidden_states) if x is not None)
        return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=outputs.past_key_values,
                                      hidden_states=outputs.hidden_states, attentions=None)

    # ------------------------------------------------------------------ generation
    @torch.no_grad()
    def generate(self, input_ids: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None,
                 max_new_tokens: Optional[int] = None, max_length: Optional[int] = None, do_sample: bool = False,
                 top_p: float = 1.0, temperature: float = 1.0, top_k: Optional[int] = None,
                 eos_token_id: Optional[int] = None,
                 pad_token_id: Optional[int] = None, use_graph: bool = True, resident: Optional[bool] = None,
                 generator: Optional[torch.Generator] = None, **kwargs) -> torch.LongTensor:
        """Greedy (default) or top-p sampling; returns [B, T + new] token ids like HF's generate.

        With the arguments above (what the reference's generate.py passes), prefill runs the module path with
        last-position logits only and decode runs the captured whole-step HIP graph of DecodeEngine when
        use_graph is set.  Sampling draws every token with one launch of the top-p kernel (functional.sample_top_p)
        on the step's logits and feeds it back without a host round trip; the uniform numbers of the whole run are
        drawn up front from `generator` (torch.rand), and the logits are bit-identical to the module path's, so a
        seeded generator gives the same tokens either way (not the tokens torch.multinomial would draw from the
        same seed).  top_k, when not given, is the generation config's, else transformers' default of 50 (what the
        reference's call, which passes none, samples with); top_k=0 switches the limit off.  Rows that
        have produced eos_token_id (default: the generation config's) are filled with pad_token_id (eos_token_id
        when not given); generation ends early once every row has.  At batch 1 the whole decode step is one resident
        launch when the model fits it; resident=False keeps one launch per fused BitLinear.

        Any further keyword (num_beams, repetition_penalty, logits_processor, stopping_criteria, streamer,
        generation_config, return_dict_in_generate, ...) sends the whole call to
        transformers' GenerationMixin.generate, which steps the module path through
        prepare_inputs_for_generation and the RecurrentCache."""
        gen_cfg = getattr(self, "generation_config", None)
        if eos_token_id is None and gen_cfg is not None:
            eos_token_id = gen_cfg.eos_token_id          # as GenerationMixin does: the model's own end-of-sequence id
            if pad_token_id is None:
                pad_token_id = gen_cfg.pad_token_id
        if kwargs or input_ids is None or not isinstance(eos_token_id, (int, type(None))):
            hf = dict(kwargs)
            for name, value, default in (("attention_mask", attention_mask, None), ("max_new_tokens", max_new_tokens, None),
                                         ("max_length", max_length, None), ("top_p", top_p, 1.0),
                                         ("temperature", temperature, 1.0), ("top_k", top_k, None),
                                         ("eos_token_id", eos_token_id, None),
                                         ("pad_token_id", pad_token_id, None)):
                if value is not None and not (isinstance(default, float) and value == default):
                    hf[name] = value
            return GenerationMixin.generate(self, input_ids, do_sample=do_sample, **hf)
        if max_new_tokens is None:
            max_new_tokens = (max_length - input_ids.shape[1]) if max_length is not None else 20
        if max_new_tokens <= 0:
            return input_ids
        B = input_ids.shape[0]
        out = self(input_ids=input_ids, attention_mask=attention_mask, use_cache=True, logits_to_keep=1)
        cache = out.past_key_values
        logits = out.logits[:, -1, :]
        tokens = [input_ids]
        finished = torch.zeros(B, dtype=torch.bool, device=input_ids.device)
        engine = None
        if use_graph and max_new_tokens > 1 and not self.config.use_short_conv:   # the graph engine has no convolution state
            from .decode import DecodeEngine
            engine = DecodeEngine.for_model(self, B, resident=resident)
            engine.load_state([c[-1] for c in cache])
        choose = None
        if do_sample:
            temperature = max(float(temperature), 1e-6)
            if top_k is None:
                top_k = getattr(gen_cfg, "top_k", None)
                top_k = 50 if top_k is None else top_k               # transformers' default generation parameter
            top_k = max(int(top_k), 0)
            # every uniform number of the run is drawn here, so the random stream does not depend on the path taken
            g_dev = generator.device if generator is not None else input_ids.device
            uniforms = torch.rand(max_new_tokens, B, generator=generator, device=g_dev).to(input_ids.device)
            if logits.shape[-1] <= F_.sample_top_p_max_vocab():
                choose = lambda lg, step, out=None: F_.sample_top_p(lg, top_p, temperature, uniforms[step], out=out,
                                                                    top_k=top_k)
            else:
                choose = lambda lg, step, out=None: _sample_top_p(lg.float(), top_p, temperature, uniforms[step], out,
                                                                  top_k=top_k)
        first = choose(logits, 0) if do_sample else F_.argmax(logits)
        if engine is not None:
            pick = (lambda step: choose(engine.logits, step, engine.tok)) if do_sample else None
            new = _self_feeding(engine, first, max_new_tokens, eos_token_id, pad_token_id, pick=pick)
            engine.check()
            return torch.cat([input_ids, new], dim=1)
        nxt = first
        for step in range(max_new_tokens):
            if step > 0:
                out = self(input_ids=nxt.view(B, 1), past_key_values=cache, use_cache=True)
                cache = out.past_key_values
                logits = out.logits[:, -1, :]
                nxt = choose(logits, step) if do_sample else F_.argmax(logits)
            if eos_token_id is not None:
                nxt = torch.where(finished, torch.full_like(nxt, eos_token_id if pad_token_id is None else pad_token_id), nxt)
                finished |= nxt == eos_token_id
            tokens.append(nxt.view(B, 1))
            if eos_token_id is not None and bool(finished.all()):
                break
        return torch.cat(tokens, dim=1)


def _self_feeding(engine, first, max_new_tokens, eos_token_id, pad_token_id, chunk=32, pick=None):
    """Decoding without a host round trip per token: every replay of the engine's graph leaves its argmax in the
    token buffer the next replay embeds; pick(step), when given, replaces that token by one drawn from the step's
    logits (sampling) before it is recorded.  The end-of-sequence test looks at a whole chunk of steps at a time;
    the steps decoded past the point where every row had finished are cut off, and a finished row's later tokens
    are replaced by the padding id, so the result is the one of the token-by-token loop."""
    B = first.shape[0]
    buf = torch.empty(max_new_tokens, B, dtype=torch.int64, device=first.device)
    buf[0].copy_(first)
    engine.tok.copy_(first.reshape(B))
    produced = 1
    while produced < max_new_tokens:
        n = min(chunk, max_new_tokens - produced)
        for _ in range(n):
            engine.advance()
            if pick is not None:
                pick(produced)
            buf[produced].copy_(engine.tok)
            produced += 1
        if eos_token_id is not None and bool((buf[:produced] == eos_token_id).any(0).all()):
            break
    seq = buf[:produced].t()                                                    # [B, produced]
    if eos_token_id is None:
        return seq.contiguous()
    is_eos = seq == eos_token_id
    after = (is_eos.cumsum(1) - is_eos.long()) > 0                              # strictly after a row's first eos
    seq = torch.where(after, torch.full_like(seq, eos_token_id if pad_token_id is None else pad_token_id), seq)
    if bool(is_eos.any(1).all()):                                               # every row finished: stop where the last one did
        last = int(is_eos.long().argmax(1).max()) + 1
        seq = seq[:, :last]
    return seq.contiguous()


def _sample_top_p(logits, top_p, temperature, u, out=None, top_k=0):
    """Vocabularies wider than the sampling kernel holds: the same top-k limit, nucleus and inverse CDF (kept tokens in
    index order, one uniform number per row) with library calls in fp32."""
    logits = logits / temperature
    if 0 < top_k < logits.shape[-1]:
        kth = torch.topk(logits, top_k, dim=-1).values[..., -1:]
        logits = logits.masked_fill(logits < kth, float("-inf"))
    probs = torch.softmax(logits, dim=-1)
    sp, si = torch.sort(probs, dim=-1, descending=True)
    keep_sorted = (sp.cumsum(-1) - sp) < max(float(top_p), 0.0)
    keep_sorted[..., 0] = True                                   # at least the most probable token
    keep = torch.zeros_like(keep_sorted).scatter_(-1, si, keep_sorted)
    cdf = (probs * keep).cumsum(-1)
    target = u.to(cdf.dtype).clamp(0.0, 1.0).reshape(-1, 1) * cdf[..., -1:]
    tok = torch.searchsorted(cdf, target, right=True).squeeze(-1).clamp_(max=logits.shape[-1] - 1)
    if out is not None:
        out.copy_(tok)
        return out
    return tok
