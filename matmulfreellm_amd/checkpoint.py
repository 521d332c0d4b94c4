"""Checkpoints for the MI355X path.

Two on-disk forms of an HGRNBit model:

* the reference's own: Hugging Face ``save_pretrained`` / ``from_pretrained`` with the latent
  (fp16 / bf16 / fp32) BitLinear weights under the reference's state-dict keys
  (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:51-52,67-79,166-170,288; mmfreelm/layers/hgrn_bit.py:56-70;
  mmfreelm/ops/fusedbitnet.py:556).  ``load_pretrained`` reads such a directory and packs every
  BitLinear once, at load, instead of on first use.
* a packed form (``save_packed`` / ``load_packed``): for each BitLinear the 2-bit codes exactly as
  the kernels read them from HBM plus the de-quantisation scale, everything else (embedding, norm
  weights, lower bounds) unchanged.  A packed model holds no latent weights: the 1.3B model is
  0.33 GB of codes instead of 2.6 GB of bf16, loads without a ternarisation pass and can only run
  inference.

Files: ``config.json`` (the reference's config) and ``model.packed.safetensors``.
"""
import json
import os

import torch
import torch.nn as nn

from . import functional as F_
from .bitlinear import BitLinear

PACKED_FILE = "model.packed.safetensors"
FORMAT = "mmf-packed-1"        # layout of the codes: 1 KiB blocks of 32 rows x 128 inputs, see include/mmf.h


def _bitlinears(model):
    return [(name, mod) for name, mod in model.named_modules() if isinstance(mod, BitLinear)]


def pack_all(model):
    """Ternarise + pack every BitLinear of ``model`` now (they are packed lazily otherwise)."""
    for _, mod in _bitlinears(model):
        mod.packed_weight()
    return model


def load_pretrained(directory, device="cuda", dtype=None, **kw):
    """``HGRNBitForCausalLM.from_pretrained`` of a reference-format directory, moved to ``device`` and packed."""
    from .modeling_hgrn_bit import HGRNBitForCausalLM
    model = HGRNBitForCausalLM.from_pretrained(directory, **kw)
    if dtype is not None:
        model = model.to(dtype)
    return pack_all(model.to(device).eval())


def save_packed(model, directory):
    """Write ``model`` (on a ROCm device) as config.json + model.packed.safetensors."""
    from safetensors.torch import save_file
    os.makedirs(directory, exist_ok=True)
    tensors, meta, latent = {}, {"format": FORMAT}, set()
    for name, mod in _bitlinears(model):
        pw = mod.packed_weight()
        tensors[name + ".packed"] = pw.packed.detach().reshape(-1).cpu()
        tensors[name + ".wdeq"] = pw.wdeq.detach().cpu()
        meta[name] = json.dumps({"n": pw.n, "k": pw.k, "seg_rows": pw.seg_rows, "dtype": str(mod.weight.dtype)})
        latent.add(name + ".weight")
    for key, t in model.state_dict().items():
        if key not in latent:
            tensors[key] = t.detach().cpu().contiguous()
    save_file(tensors, os.path.join(directory, PACKED_FILE), metadata=meta)
    model.config.save_pretrained(directory)
    return os.path.join(directory, PACKED_FILE)


def _assign(model, key, tensor):
    mod_name, _, leaf = key.rpartition(".")
    mod = model.get_submodule(mod_name) if mod_name else model
    if leaf in mod._parameters:
        mod._parameters[leaf] = nn.Parameter(tensor, requires_grad=False)
    elif leaf in mod._buffers:
        mod._buffers[leaf] = tensor
    else:
        raise KeyError(f"unexpected tensor {key!r} in packed checkpoint")


def load_packed(directory, device="cuda"):
    """Build an inference-only HGRNBitForCausalLM from ``save_packed`` output.  BitLinear latent weights
    stay on the meta device (no memory); their packed codes go straight to ``device``."""
    from safetensors import safe_open
    from .configuration_hgrn_bit import HGRNBitConfig
    from .modeling_hgrn_bit import HGRNBitForCausalLM
    device = torch.device(device)
    cfg = HGRNBitConfig.from_pretrained(directory)
    with torch.device("meta"):
        model = HGRNBitForCausalLM(cfg)
    mods = dict(_bitlinears(model))
    with safe_open(os.path.join(directory, PACKED_FILE), framework="pt", device="cpu") as f:
        meta = f.metadata() or {}
        if meta.get("format") != FORMAT:
            raise ValueError(f"{directory}: not a {FORMAT} checkpoint (format={meta.get('format')!r})")
        keys = set(f.keys())
        for name, mod in mods.items():
            if name not in meta or name + ".packed" not in keys:
                raise KeyError(f"packed checkpoint lacks BitLinear {name!r}")
            info = json.loads(meta[name])
            if (info["n"], info["k"]) != (mod.out_features, mod.in_features):
                raise ValueError(f"{name}: checkpoint holds {info['n']}x{info['k']}, model wants "
                                 f"{mod.out_features}x{mod.in_features}")
            pw = F_.PackedWeight(f.get_tensor(name + ".packed").to(device), f.get_tensor(name + ".wdeq").to(device),
                                 info["n"], info["k"], info["seg_rows"])
            dt = getattr(torch, info["dtype"].replace("torch.", ""))
            mod.weight = nn.Parameter(torch.empty(info["n"], info["k"], dtype=dt, device="meta"), requires_grad=False)
            mod._pack.freeze(pw)
            keys -= {name + ".packed", name + ".wdeq"}
        for key in sorted(keys):
            _assign(model, key, f.get_tensor(key).to(device))
    left = [n for n, p in model.named_parameters() if p.is_meta and not any(n == b + ".weight" for b in mods)]
    if left:
        raise KeyError(f"packed checkpoint lacks {left[:4]}{'...' if len(left) > 4 else ''}")
    return model.eval()
