"""Per-sequence state of layer-list models: latent pages + state slots.

Two pools, both handed out and taken back by the engine as sequences
come and go:

* :class:`LatentCachePool` — paged rows for every attention layer that owns
  a cache: ``[latent | rotated key part]`` for latent attention (layers
  that read another layer's cache own none), ``[keys of all kv heads |
  values of all kv heads]`` for grouped-query attention. Block ids come
  from the same refcounting :class:`BlockAllocator` as the dense models'
  K/V pool, so a forked candidate shares its prompt's full pages.
* :class:`StateSlotPool` — fixed-size fp32 state per live sequence: the
  last ``taps - 1`` inputs of every short convolution (the block's own, or
  a delta-rule layer's over its q/k/v channels) and the state of every
  recurrent layer (a vector for minGRU, a matrix per head for the delta
  rule). A slot is zeroed when it is handed out, so whatever its previous
  owner left cannot leak.
"""

from __future__ import annotations

from typing import Dict, List

import torch

from ..models.hybrid import (DeltaRuleSpec, HybridSpec, LatentAttentionSpec,
                             MinGRUSpec, SinkAttentionSpec)
from .kvcache import BlockAllocator


class LatentCachePool:
    def __init__(self, spec: HybridSpec, num_blocks: int, block_size: int,
                 dtype: torch.dtype, device):
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.allocator = BlockAllocator(num_blocks)
        # one page past the allocator's range that no sequence ever owns:
        # padding rows of a captured decode step write there
        self.scratch_block = num_blocks
        # layer index -> [(num_blocks + 1) * block_size, kv_rank + rot_dim]
        self.rows: Dict[int, torch.Tensor] = {}
        for i, ls in enumerate(spec.layers):
            m = ls.mixer
            if self._owns_rows(m):
                self.rows[i] = torch.zeros((num_blocks + 1) * block_size, m.cache_width,
                                           dtype=dtype, device=device)

    @staticmethod
    def _owns_rows(m) -> bool:
        return (isinstance(m, SinkAttentionSpec)
                or (isinstance(m, LatentAttentionSpec) and m.kv_from is None))

    def layer_rows(self, spec: HybridSpec, layer: int) -> torch.Tensor:
        m = spec.layers[layer].mixer
        src = getattr(m, "kv_from", None)
        return self.rows[layer if src is None else src]

    @staticmethod
    def blocks_for(num_tokens: int, block_size: int) -> int:
        return (num_tokens + block_size - 1) // block_size

    @staticmethod
    def bytes_per_block(spec: HybridSpec, block_size: int, dtype) -> int:
        w = sum(ls.mixer.cache_width for ls in spec.layers
                if LatentCachePool._owns_rows(ls.mixer))
        return max(1, w) * block_size * torch.tensor([], dtype=dtype).element_size()

    def copy_block(self, src: int, dst: int) -> None:
        bs = self.block_size
        for t in self.rows.values():
            t[dst * bs:(dst + 1) * bs].copy_(t[src * bs:(src + 1) * bs])


class StateSlotPool:
    def __init__(self, spec: HybridSpec, num_slots: int, device):
        self.num_slots = num_slots
        self.scratch_slot = num_slots     # never handed out (padding rows)
        D, k = spec.width, max(spec.conv_taps - 1, 0)
        # conv tails: one tensor per layer, [slots + 1, taps-1, width] fp32
        self.tails: List[torch.Tensor] = [
            torch.zeros(num_slots + 1, k, D, dtype=torch.float32, device=device)
            for _ in spec.layers]
        # recurrent state: layer index -> [slots + 1, state size] fp32
        self.recurrent: Dict[int, torch.Tensor] = {
            i: torch.zeros(num_slots + 1, ls.mixer.state_size, dtype=torch.float32,
                           device=device)
            for i, ls in enumerate(spec.layers)
            if isinstance(ls.mixer, (MinGRUSpec, DeltaRuleSpec))}
        # a mixer's own short convolution: layer index ->
        # [slots + 1, taps - 1, channels] fp32
        self.mixer_tails: Dict[int, torch.Tensor] = {
            i: torch.zeros(num_slots + 1, ls.mixer.taps - 1, ls.mixer.conv_channels,
                           dtype=torch.float32, device=device)
            for i, ls in enumerate(spec.layers)
            if isinstance(ls.mixer, DeltaRuleSpec)}
        self._free = list(range(num_slots - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def _tensors(self):
        return (list(self.tails) + list(self.recurrent.values())
                + list(self.mixer_tails.values()))

    def alloc(self) -> int:
        if not self._free:
            raise MemoryError("state slot pool exhausted")
        s = self._free.pop()
        for t in self._tensors():
            t[s].zero_()
        return s

    def free(self, slot: int) -> None:
        assert slot not in self._free
        self._free.append(slot)

    def copy(self, src: int, dst: int) -> None:
        for t in self._tensors():
            t[dst].copy_(t[src])

    def reset(self) -> None:
        self._free = list(range(self.num_slots - 1, -1, -1))
