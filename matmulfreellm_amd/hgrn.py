"""fused_recurrent_hgrn / chunk_hgrn (interfaces of mmfreelm/ops/hgrn/recurrent_fuse.py:176 and chunk.py:287)."""
from typing import Optional, Tuple

import torch

from . import functional as F_


def fused_recurrent_hgrn(x: torch.Tensor, g: torch.Tensor, initial_state: Optional[torch.Tensor] = None,
                         output_final_state: bool = False) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """h_t = g_t * h_{t-1} + x_t with g the decay in (0, 1).  x, g: [B, H, T, D]; state [B, H, D].

    The final state is returned in fp32 (the reference returns it in x.dtype)."""
    if initial_state is not None:
        initial_state = initial_state.detach()
    from .autograd import FusedRecurrentHGRNFn, needs_grad
    if needs_grad(x, g):
        return FusedRecurrentHGRNFn.apply(x, g, initial_state, output_final_state)
    return F_.hgrn_recurrent(x, g, initial_state, output_final_state)


def chunk_hgrn(x: torch.Tensor, g: torch.Tensor, initial_state: Optional[torch.Tensor] = None,
               output_final_state: bool = False, chunk_size: int = 64) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """h_t = exp(g_t) * h_{t-1} + x_t with g the LOG decay (<= 0).  Same shapes; fp32 final state."""
    if initial_state is not None:
        initial_state = initial_state.detach()
    from .autograd import ChunkHGRNFn, needs_grad
    if needs_grad(x, g):
        return ChunkHGRNFn.apply(x, g, initial_state, output_final_state, chunk_size)
    return F_.hgrn_chunk(x, g, initial_state, output_final_state, chunk_size)
