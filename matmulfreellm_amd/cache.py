"""RecurrentCache: per-layer recurrent state for decoding (interface of mmfreelm/models/utils.py:11-104).

Stands alone instead of deriving from transformers' Cache, whose constructor and legacy
conversion helpers changed incompatibly between transformers 4.x and 5.x.
"""
from typing import Any, Dict, List, Optional, Tuple

import torch


class RecurrentCache:
    """A list of per-layer state tuples; the first update appends, later ones copy in place."""

    def __init__(self, seen_tokens: int = 0):
        self.states: List[Tuple[torch.Tensor, ...]] = []
        self._seen_tokens = seen_tokens

    def __getitem__(self, layer_idx: int):
        if layer_idx < len(self):
            return self.states[layer_idx]
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        for state in self.states:
            yield state

    def __len__(self):
        return len(self.states)

    def update(self, state, layer_idx: int, cache_kwargs: Optional[Dict[str, Any]] = None):
        if isinstance(state, torch.Tensor):
            state = (state,)
        if len(self.states) <= layer_idx:
            self.states.append(state)
        else:
            for i, s in enumerate(state):
                if self.states[layer_idx][i].data_ptr() != s.data_ptr():
                    self.states[layer_idx][i].copy_(s)
            if layer_idx == len(self) - 1:
                self._seen_tokens += 1
        return state

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if len(self.states) <= layer_idx:
            return 0
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        return None

    def reorder_cache(self, beam_idx: torch.LongTensor):
        for layer_idx in range(len(self.states)):
            self.states[layer_idx] = tuple(s.index_select(0, beam_idx.to(s.device)) for s in self.states[layer_idx])

    def to_legacy_cache(self):
        return tuple(self.states)

    @classmethod
    def from_legacy_cache(cls, past_key_values=None, seen_tokens: int = 0):
        cache = cls(seen_tokens)
        if past_key_values is not None:
            for layer_idx in range(len(past_key_values)):
                cache.update(past_key_values[layer_idx], layer_idx)
        return cache
