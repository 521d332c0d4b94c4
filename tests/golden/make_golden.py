"""Writes tests/golden/config1_{fp32,bf16}.npz and config1_eps1e-8_{fp32,bf16}.npz from the CPU oracle (spec arithmetic).

The reference ships no tests or fixtures for this path, so these vectors pin the oracle itself against
drift and give the GPU tests a committed target: seeded random-init model (vocab 32000, hidden 512,
4 layers), a seeded 128-token prompt, then
  argmax      [128]  greedy choice at every prompt position (lowest index on ties)
  probe_idx   [64]   fixed vocabulary indices
  probe_bits  [128, 64] uint32 bit patterns of the fp32-cast logits at those indices
  greedy      [12]   tokens of a 12-step greedy continuation
The first pair runs every BitLinear's inner norm at eps 1e-6 (what the reference's FusedBitLinear forward really uses,
mmfreelm/ops/fusedbitnet.py:602-610 with the default of :520), the second at 1e-8 (the eps its un-fused BitLinear
states, :551; the model is built with HGRNBitConfig(bitlinear_eps=1e-8) to match).
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import model as om  # noqa: E402

V, H, L, T, NEW = 32000, 512, 4, 128, 12


def vectors(dtype, bitlinear_eps=1e-6):
    params = om.init_params(V, H, L, seed=0, dtype=dtype)
    torch.manual_seed(1)
    ids = torch.randint(0, V, (1, T))
    logits, _ = om.forward(params, ids, L, mode="spec", bitlinear_eps=bitlinear_eps)
    probe = torch.arange(64) * 499 + 7
    toks, _ = om.greedy(params, ids, L, NEW, mode="spec", bitlinear_eps=bitlinear_eps)
    return {"prompt": ids[0].numpy().astype(np.int64),
            "argmax": om.argmax_lowest(logits.float())[0].numpy().astype(np.int64),
            "probe_idx": probe.numpy().astype(np.int64),
            "probe_bits": logits[0][:, probe].float().contiguous().numpy().view(np.uint32),
            "greedy": toks[0].numpy().astype(np.int64)}


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for tag, eps in (("", 1e-6), ("eps1e-8_", 1e-8)):
        for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
            np.savez_compressed(os.path.join(here, f"config1_{tag}{name}.npz"), **vectors(dt, eps))
            print("wrote", f"config1_{tag}{name}.npz")
