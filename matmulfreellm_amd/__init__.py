"""MI355X-native inference hot path of the MatMul-free LM (BitLinear + HGRN).

Same public names as the reference package ``mmfreelm``; every op runs a hand-written HIP
kernel for gfx950 through the C ABI in include/mmf.h (lib/libmmf_hip.so).  There is no CPU
path: tensors must live on a ROCm device.

Name map (reference module -> here):
    mmfreelm.ops.fusedbitnet      FusedBitLinear, BitLinear, layer_norm_linear_quant_fn,
                                  activation_quant, weight_quant          -> .bitlinear
    mmfreelm.modules.layernorm    RMSNorm, rms_norm_fn                     -> .layernorm
    mmfreelm.modules.fused_norm_gate  FusedRMSNormSwishGate                -> .fused_norm_gate
    mmfreelm.modules.activations  swiglu                                   -> .activations
    mmfreelm.ops.hgrn             fused_recurrent_hgrn, chunk_hgrn         -> .hgrn
    mmfreelm.layers.hgrn_bit      HGRNBitAttention                         -> .attention
    mmfreelm.models.hgrn_bit      HGRNBitConfig, HGRNBitModel, HGRNBitForCausalLM -> .modeling_hgrn_bit
    mmfreelm.models.utils         RecurrentCache                           -> .cache
    mmfreelm.modules.convolution  ShortConvolution                         -> .convolution
"""
from .activations import swiglu
from .bitlinear import (BitLinear, FusedBitLinear, activation_quant, layer_norm_linear_quant_fn, weight_quant)
from .cache import RecurrentCache
from .convolution import ShortConvolution
from .fused_norm_gate import FusedRMSNormSwishGate
from .hgrn import chunk_hgrn, fused_recurrent_hgrn
from .layernorm import RMSNorm, rms_norm_fn

__version__ = "0.1"

_LAZY = {"HGRNBitAttention": ".attention", "HGRNBitConfig": ".configuration_hgrn_bit",
         "HGRNBitModel": ".modeling_hgrn_bit", "HGRNBitForCausalLM": ".modeling_hgrn_bit",
         "HGRNBitBlock": ".modeling_hgrn_bit", "HGRNBitMLP": ".modeling_hgrn_bit", "DecodeEngine": ".decode",
         "save_packed": ".checkpoint", "load_packed": ".checkpoint", "load_pretrained": ".checkpoint", "pack_all": ".checkpoint"}

__all__ = ["swiglu", "BitLinear", "FusedBitLinear", "activation_quant", "weight_quant", "layer_norm_linear_quant_fn",
           "RecurrentCache", "ShortConvolution", "FusedRMSNormSwishGate", "chunk_hgrn", "fused_recurrent_hgrn", "RMSNorm", "rms_norm_fn",
           *_LAZY]

_registered = False


def register_auto_classes():
    """AutoConfig / AutoModel / AutoModelForCausalLM registration (mmfreelm/models/hgrn_bit/__init__.py:8-10)."""
    global _registered
    if _registered:
        return
    from transformers import AutoConfig, AutoModel, AutoModelForCausalLM

    from .configuration_hgrn_bit import HGRNBitConfig
    from .modeling_hgrn_bit import HGRNBitForCausalLM, HGRNBitModel
    for fn, args in ((AutoConfig.register, (HGRNBitConfig.model_type, HGRNBitConfig)),
                     (AutoModel.register, (HGRNBitConfig, HGRNBitModel)),
                     (AutoModelForCausalLM.register, (HGRNBitConfig, HGRNBitForCausalLM))):
        try:
            fn(*args)
        except ValueError:
            pass   # already registered by an earlier import
    _registered = True


def __getattr__(name):
    # the model classes pull in transformers (seconds to import); load them on first use
    if name in _LAZY:
        import importlib
        mod = importlib.import_module(_LAZY[name], __name__)
        if name in ("HGRNBitConfig", "HGRNBitModel", "HGRNBitForCausalLM"):
            register_auto_classes()
        return getattr(mod, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
