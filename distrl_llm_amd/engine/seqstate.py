"""Per-sequence state of layer-list models: latent pages + state slots.

Two pools, both handed out and taken back by the engine as sequences
come and go:

* :class:`LatentCachePool` — paged rows for every attention layer that owns
  a cache: ``[latent | rotated key part]`` for latent attention (layers
  that read another layer's cache own none), ``[keys of all kv heads |
  values of all kv heads]`` for grouped-query attention. Block ids come
  from the same refcounting :class:`BlockAllocator` as the dense models'
  K/V pool, so a forked candidate shares its prompt's full pages.
  Tensors are keyed by mixer unit: the layer index, or (layer, side) for
  the two sides of a parallel pair.
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
                             MinGRUSpec, SigmoidAttentionSpec,
                             SinkAttentionSpec, WindowAttentionSpec,
                             mixer_units)
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
        # mixer unit -> [(num_blocks + 1) * block_size, cache row width]
        self.rows: Dict[object, torch.Tensor] = {}
        for i, m in mixer_units(spec):
            if self._owns_rows(m):
                self.rows[i] = torch.zeros((num_blocks + 1) * block_size, m.cache_width,
                                           dtype=dtype, device=device)

    @staticmethod
    def _owns_rows(m) -> bool:
        return (isinstance(m, (SinkAttentionSpec, SigmoidAttentionSpec,
                               WindowAttentionSpec))
                or (isinstance(m, LatentAttentionSpec) and m.kv_from is None))

    def layer_rows(self, spec: HybridSpec, layer: int) -> torch.Tensor:
        return self.unit_rows(layer, spec.layers[layer].mixer)

    def unit_rows(self, key, m) -> torch.Tensor:
        src = getattr(m, "kv_from", None)
        return self.rows[key if src is None else src]

    @staticmethod
    def blocks_for(num_tokens: int, block_size: int) -> int:
        return (num_tokens + block_size - 1) // block_size

    @staticmethod
    def bytes_per_block(spec: HybridSpec, block_size: int, dtype) -> int:
        w = sum(m.cache_width for _, m in mixer_units(spec)
                if LatentCachePool._owns_rows(m))
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
        # recurrent state: mixer unit -> [slots + 1, state size] fp32
        self.recurrent: Dict[object, torch.Tensor] = {
            i: torch.zeros(num_slots + 1, m.state_size, dtype=torch.float32,
                           device=device)
            for i, m in mixer_units(spec)
            if isinstance(m, (MinGRUSpec, DeltaRuleSpec))}
        # a mixer's own short convolution: mixer unit ->
        # [slots + 1, taps - 1, channels] fp32
        self.mixer_tails: Dict[object, torch.Tensor] = {
            i: torch.zeros(num_slots + 1, m.taps - 1, m.conv_channels,
                           dtype=torch.float32, device=device)
            for i, m in mixer_units(spec)
            if isinstance(m, DeltaRuleSpec)}
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
