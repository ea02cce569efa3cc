"""Paged KV cache + block allocator.

Layout per layer: [num_blocks, num_kv_heads, block_size, head_dim] — a
(block, kv_head) pair is a contiguous [block_size, head_dim] tile, which is
what one workgroup of the CDNA4 decode kernel streams with coalesced
dwordx4 loads (PagedAttention equivalent).

Sizing: the engine claims ``gpu_memory_utilization`` × free HBM after
weights are resident (MI355X: 288 GB per GPU, so 9B-bf16 leaves ~240 GB of
KV — tens of thousands of 8k contexts; the scheduler, not memory, is the
usual admission limit)."""

from __future__ import annotations

import logging
from typing import List, Optional, Tuple

import torch

logger = logging.getLogger(__name__)


class KVCache:
    """Uniform models pass (num_layers, num_kv_heads, head_dim); models whose
    layers differ pass ``layout``: one (kv_heads, k_dim, v_dim) per layer, or
    None for a layer that caches no keys (its k/v entries are None); v_dim 0
    means the layer's values are read out of its key rows (latent caches), so
    only k is allocated. All layers share block ids, so one block table
    serves every layer."""

    def __init__(
        self,
        num_layers: int,
        num_blocks: int,
        num_kv_heads: int,
        block_size: int,
        head_dim: int,
        device: torch.device,
        dtype: torch.dtype,
        layout: Optional[List[Optional[Tuple[int, int, int]]]] = None,
    ):
        if layout is None:
            layout = [(num_kv_heads, head_dim, head_dim)] * num_layers
        self.layout = list(layout)
        self.num_layers = len(self.layout)
        self.num_blocks = num_blocks
        self.block_size = block_size
        # per-sequence recurrent state of the same model (set by the engine
        # for models with recurrent layers): one cache object reaches forward
        self.recurrent: Optional["RecurrentStateCache"] = None
        self.k: List[Optional[torch.Tensor]] = []
        self.v: List[Optional[torch.Tensor]] = []
        for entry in self.layout:
            if entry is None:
                self.k.append(None)
                self.v.append(None)
                continue
            heads, k_dim, v_dim = entry
            self.k.append(
                torch.zeros(num_blocks, heads, block_size, k_dim, device=device, dtype=dtype)
            )
            self.v.append(
                torch.zeros(num_blocks, heads, block_size, v_dim, device=device, dtype=dtype)
                if v_dim else None
            )

    @staticmethod
    def block_bytes(num_layers, num_kv_heads, block_size, head_dim, dtype) -> int:
        elem = torch.tensor([], dtype=dtype).element_size()
        return 2 * num_layers * num_kv_heads * block_size * head_dim * elem

    @staticmethod
    def layout_block_bytes(layout, block_size, dtype) -> int:
        elem = torch.tensor([], dtype=dtype).element_size()
        return sum(h * block_size * (kd + vd) * elem for (h, kd, vd) in
                   (e for e in layout if e is not None))

    @classmethod
    def num_blocks_for_budget(
        cls, budget_bytes: int, num_layers, num_kv_heads, block_size, head_dim, dtype
    ) -> int:
        per_block = cls.block_bytes(num_layers, num_kv_heads, block_size, head_dim, dtype)
        return max(budget_bytes // per_block, 0)


class BlockAllocator:
    """Free-list allocator over block ids [0, num_blocks)."""

    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def can_allocate(self, n: int) -> bool:
        return len(self._free) >= n

    def allocate(self, n: int) -> Optional[List[int]]:
        if len(self._free) < n:
            return None
        if n == 0:
            return []
        blocks = self._free[-n:][::-1]
        del self._free[-n:]
        return blocks

    def free(self, blocks: List[int]) -> None:
        self._free.extend(reversed(blocks))


def blocks_needed(num_tokens: int, block_size: int) -> int:
    return (num_tokens + block_size - 1) // block_size


class RecurrentStateCache:
    """Per-sequence recurrent state, one fp32 tensor [num_slots + 1, *shape]
    per recurrent layer (None for the others). A layer that carries several
    states (a scan's state and the tail of its short convolution, say) names
    a list of shapes and gets a list of tensors. A sequence owns one slot id
    across all layers from admission to release; slot ``num_slots`` is a
    scratch row for the padding rows of a captured decode graph. Slots are
    never cleared: a sequence's first portion starts from zero by itself."""

    def __init__(self, layout: List[Optional[Tuple[int, ...]]], num_slots: int,
                 device: torch.device):
        self.layout = list(layout)
        self.num_slots = num_slots
        self.pad_slot = num_slots

        def make(shape):
            return torch.zeros(num_slots + 1, *shape, device=device, dtype=torch.float32)

        self.state: List[Optional[torch.Tensor]] = [
            None if entry is None
            else [make(shape) for shape in entry] if isinstance(entry, list)
            else make(entry)
            for entry in self.layout
        ]

    def _tensors(self):
        for s in self.state:
            if s is None:
                continue
            yield from (s if isinstance(s, list) else [s])

    @property
    def active(self) -> bool:
        return any(True for _ in self._tensors())

    def bytes(self) -> int:
        return sum(t.numel() * 4 for t in self._tensors())


class SlotAllocator:
    """Free-list over state slot ids [0, num_slots); lowest id first, so
    released slots are handed out again at once."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free: List[int] = list(range(num_slots - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> Optional[int]:
        return self._free.pop() if self._free else None

    def free(self, slot: int) -> None:
        if slot < 0 or slot >= self.num_slots or slot in self._free:
            raise ValueError(f"bad state slot release: {slot}")
        self._free.append(slot)
