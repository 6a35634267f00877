"""Names of the reference's HF monkey-patch decoder (obkv_accel/decode_hook.py).

In the reference both entry points raise ``NotImplementedError`` before doing any work
(decode_hook.py:243, :481) because the hook predates the three-zone cache; the live decode
path is ``fast_decode``.  The same behaviour is kept so callers see the same error.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .packing import DualZoneCache


class PackedCacheWrapper:
    """Duck-typed cache facade answering the length queries HF's model loop makes
    (decode_hook.py:86-197)."""

    def __init__(self, dual_cache: DualZoneCache):
        self.dual_cache = dual_cache
        self._num_layers = len(dual_cache.packed)

    def get_seq_length(self, layer_idx: int = 0) -> int:
        pl = self.dual_cache.packed[layer_idx]
        t_old = pl.T_eff_k if pl.T_eff_k > 0 else pl.T_eff
        new_k = self.dual_cache.new_both_k[layer_idx]
        return t_old + (new_k.shape[2] if new_k is not None else 0)

    def get_max_length(self) -> Optional[int]:
        return None

    def get_max_cache_shape(self) -> Optional[int]:
        return None

    def get_mask_sizes(self, cache_position, layer_idx: int = 0):
        return self.get_seq_length(layer_idx) + int(cache_position.shape[0]), 0

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        return key_states, value_states

    @property
    def is_sliding(self):
        return [False] * self._num_layers

    def __len__(self) -> int:
        return self._num_layers

    def __getitem__(self, idx):
        return self.dual_cache.new_both_k[idx], self.dual_cache.new_both_v[idx]


def make_packed_decode_forward(layer_idx: int, dual_cache: DualZoneCache):
    raise NotImplementedError(
        "decode_hook.make_packed_decode_forward is incompatible with TriZoneCache; "
        "use fast_decode.trizone_attention / trizone_attention_fused.")


def greedy_decode_packed(model, dual_cache: DualZoneCache, next_token_logits: torch.Tensor,
                         max_new_tokens: int, eos_token_ids: Sequence[int],
                         primary_device: torch.device, decode_position_start: int) -> List[int]:
    raise NotImplementedError(
        "decode_hook.greedy_decode_packed is incompatible with TriZoneCache; "
        "use fast_decode.trizone_attention / trizone_attention_fused.")
