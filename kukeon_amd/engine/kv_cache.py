"""Paged KV cache for MI355X (288 GB HBM3E per GPU).

Layout per layer: k/v [num_blocks, Hk, BLOCK=16, D] bf16 — token-major rows
with D contiguous so the decode kernel's cooperative 16 B/lane stage is
coalesced.  One big [L, ...] allocation per side keeps the allocator trivial
and lets the engine size it against free HBM at init (kukeon capability map:
the reference has no GPU plane; this implements BASELINE.json's "paged KV
sized for 288 GB HBM").
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch


class BlockAllocator:
    """Free-list block allocator (exact, O(1) alloc/free)."""

    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> List[int]:
        if n > len(self._free):
            raise MemoryError(
                f"KV cache exhausted: want {n} blocks, {len(self._free)} free")
        out = self._free[-n:][::-1]
        del self._free[-n:]
        return out

    def free(self, blocks: List[int]) -> None:
        self._free.extend(reversed(blocks))


class SequenceKV:
    """Per-sequence block list + logical length."""

    def __init__(self, block_size: int):
        self.block_size = block_size
        self.blocks: List[int] = []
        self.num_tokens = 0
        # last sampled token of the previous turn: sampled but never run
        # through the model, so the next turn's prefill must include it
        self.pending_token = None
        # slot of this sequence in the engine's StatePool (-1: none held)
        self.state_slot = -1
        # every token whose K/V lives in the cache, in order — the replay
        # source for preemption-by-recompute
        self.history = []

    def blocks_needed(self, new_tokens: int) -> int:
        total = self.num_tokens + new_tokens
        need = (total + self.block_size - 1) // self.block_size
        return max(0, need - len(self.blocks))

    def slots_for(self, new_tokens: int) -> List[int]:
        """Flat slot ids for the next new_tokens positions (after extend)."""
        out = []
        for i in range(new_tokens):
            p = self.num_tokens + i
            out.append(self.blocks[p // self.block_size] * self.block_size +
                       p % self.block_size)
        return out


class PagedKVCache:
    def __init__(self, num_layers: int, num_blocks: int, num_kv_heads: int,
                 block_size: int, head_dim: int, device, dtype=torch.bfloat16):
        self.num_layers = num_layers
        self.num_blocks = num_blocks
        self.block_size = block_size
        shape = (num_layers, num_blocks, num_kv_heads, block_size, head_dim)
        # zeros, NOT empty: attention masks out-of-range tail-block tokens
        # by score (-inf -> weight 0), but their V still enters the
        # accumulation as 0*value — uninitialized bytes can decode to NaN
        # bf16 and 0*NaN poisons the whole row. Zero-init guarantees every
        # slot is 0.0 or a previously written finite value.
        self.k = torch.zeros(shape, dtype=dtype, device=device)
        self.v = torch.zeros(shape, dtype=dtype, device=device)
        self.allocator = BlockAllocator(num_blocks)

    @staticmethod
    def blocks_from_bytes(free_bytes: int, num_layers: int, num_kv_heads: int,
                          block_size: int, head_dim: int,
                          dtype_bytes: int = 2) -> int:
        per_block = 2 * num_layers * num_kv_heads * block_size * head_dim * dtype_bytes
        return max(1, free_bytes // per_block)


@dataclass
class LayerKVSpec:
    """Cache geometry of one layer. A layer with `share_from` set keeps no
    pages of its own: it reads the pages of that (earlier) layer."""
    kv_heads: int
    k_width: int
    v_width: int
    share_from: Optional[int] = None


class LayeredKVCache:
    """Paged cache whose layers differ in shape (key rows wider than value
    rows, per-layer head counts) and may share pages across layers. A layer
    whose spec is None keeps no pages at all (a recurrent mixer); a spec
    with `v_width == 0` keeps one row per token (a latent cache from which
    keys and values are both expanded).

    One allocator serves all layers: block id b names the page
    [b, kv_heads, block_size, width] in every layer's pool, so a sequence
    holds ONE block list. `k[i]` / `v[i]` of a sharing layer alias the
    owner's tensors.
    """

    def __init__(self, specs: Sequence[LayerKVSpec], num_blocks: int,
                 block_size: int, device, dtype=torch.bfloat16):
        self.specs = list(specs)
        self.num_layers = len(self.specs)
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.k: List[torch.Tensor] = [None] * self.num_layers
        self.v: List[torch.Tensor] = [None] * self.num_layers
        for i, sp in enumerate(self.specs):
            if sp is None or sp.share_from is not None:
                continue
            # zeros: masked-out tail slots are never read as garbage
            self.k[i] = torch.zeros(num_blocks, sp.kv_heads, block_size,
                                    sp.k_width, dtype=dtype, device=device)
            self.v[i] = torch.zeros(num_blocks, sp.kv_heads, block_size,
                                    sp.v_width, dtype=dtype, device=device)
        for i, sp in enumerate(self.specs):
            if sp is None or sp.share_from is None:
                continue
            j = sp.share_from
            if not (0 <= j < i) or self.specs[j] is None or \
                    self.specs[j].share_from is not None:
                raise ValueError(
                    f"layer {i} shares the cache of layer {j}, which must be "
                    "an earlier layer with pages of its own")
            own = self.specs[j]
            if (own.kv_heads, own.k_width, own.v_width) != \
                    (sp.kv_heads, sp.k_width, sp.v_width):
                raise ValueError(
                    f"layer {i} and the layer {j} it shares with differ in "
                    "cache shape")
            self.k[i], self.v[i] = self.k[j], self.v[j]
        self.allocator = BlockAllocator(num_blocks)

    @property
    def nbytes(self) -> int:
        return sum(self.k[i].nbytes + self.v[i].nbytes
                   for i, sp in enumerate(self.specs)
                   if sp is not None and sp.share_from is None)

    @staticmethod
    def blocks_from_bytes(free_bytes: int, specs: Sequence[LayerKVSpec],
                          block_size: int, dtype_bytes: int = 2) -> int:
        per_block = sum(sp.kv_heads * block_size * (sp.k_width + sp.v_width)
                        for sp in specs
                        if sp is not None and sp.share_from is None) \
            * dtype_bytes
        return max(1, free_bytes // max(1, per_block))


class StatePool:
    """Fixed-size slots of per-sequence carried state (tails of short
    convolutions, recurrent state): one fp32 tensor [slots, *shape] per
    layer that carries state, None for the others; a layer that carries
    several pieces (a convolution tail AND a recurrent state) gives a list
    of shapes and gets a tuple of tensors. A sequence holds one
    slot index for all layers; a slot's content is only meaningful to the
    sequence that wrote it, and a sequence that starts at position 0 never
    reads what the slot held before."""

    def __init__(self, layer_shapes: Sequence[Optional[Tuple[int, ...]]],
                 num_slots: int, device, dtype=torch.float32):
        self.num_slots = num_slots
        def make(shp):
            if shp is None:
                return None
            if len(shp) and isinstance(shp[0], (tuple, list)):
                return tuple(make(one) for one in shp)
            return torch.zeros((num_slots,) + tuple(shp), dtype=dtype,
                               device=device)

        self.layers: list = [make(shp) for shp in layer_shapes]
        self._free: List[int] = list(range(num_slots - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise MemoryError("state slots exhausted")
        return self._free.pop()

    def free(self, slot: int) -> None:
        if slot >= 0:
            self._free.append(slot)
