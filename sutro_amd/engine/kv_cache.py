"""Paged KV cache: block allocator + per-layer page tensors, plus the
fixed-size recurrent state of layers that carry one (slot per sequence).

Layout (per layer, K and V separate):
    cache[num_blocks, num_kv_heads, block_size, head_dim]

chosen so a decode wave reads one page's (head, pos, :) rows as contiguous
16-byte vectors along head_dim, and the RoPE+cache-write kernel scatters each
new token's K/V row with a single dwordx4-per-lane store.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch


class BlockAllocator:
    """Free-list allocator over KV page indices."""

    def __init__(self, num_blocks: int) -> None:
        self.num_blocks = num_blocks
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, n: int) -> List[int]:
        if n > len(self._free):
            raise MemoryError(f"KV cache exhausted: need {n} blocks, have {len(self._free)}")
        return [self._free.pop() for _ in range(n)]

    def free(self, blocks: List[int]) -> None:
        self._free.extend(reversed(blocks))


class RecurrentStateCache:
    """Per-sequence fixed-size state of recurrent mixers, one slot a sequence.

    For every layer that carries state (`shapes[i]` = (channels, taps, heads,
    dk, dv), else None):
        conv[i]  [slots, taps-1, channels] fp32 — the last taps-1 inputs of the
                 layer's short filters, oldest first;
        ssm[i]   [slots, heads, dk, dv] fp32 — the delta-rule memory.
    A layer may instead describe its state as a dict name -> per-slot shape;
    it then gets fp32 tensors named[i][name] of shape [slots, *shape] (the
    mLSTM keeps its matrix memory and its stabiliser this way).
    A slot is not cleared when it is handed out again: the kernels start from
    zero whenever a sequence's first token (position 0) is in the batch.
    Slot 0 is reserved as scratch for padded graph rows."""

    def __init__(self, num_slots: int, shapes: Sequence, device: str) -> None:
        self.num_slots = num_slots + 1
        self.conv: List[Optional[torch.Tensor]] = []
        self.ssm: List[Optional[torch.Tensor]] = []
        self.named: List[Optional[Dict[str, torch.Tensor]]] = []
        for sh in shapes:
            if sh is None or isinstance(sh, dict):
                self.conv.append(None)
                self.ssm.append(None)
                self.named.append(None if sh is None else {
                    k: torch.zeros((self.num_slots,) + tuple(v),
                                   dtype=torch.float32, device=device)
                    for k, v in sh.items()})
                continue
            self.named.append(None)
            ch, taps, heads, dk, dv = sh
            self.conv.append(torch.zeros(self.num_slots, max(1, taps - 1), ch,
                                         dtype=torch.float32, device=device))
            self.ssm.append(torch.zeros(self.num_slots, heads, dk, dv,
                                        dtype=torch.float32, device=device))
        self.scratch_slot = 0
        self._free: List[int] = list(range(self.num_slots - 1, 0, -1))
        self.slots: Dict[int, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self, req_id: int) -> int:
        slot = self.slots.get(req_id)
        if slot is None:
            if not self._free:
                raise MemoryError("recurrent state slots exhausted")
            slot = self._free.pop()
            self.slots[req_id] = slot
        return slot

    def release(self, req_id: int) -> None:
        slot = self.slots.pop(req_id, None)
        if slot is not None:
            self._free.append(slot)


class PagedKVCache:
    def __init__(
        self,
        num_layers: int,
        num_blocks: int,
        num_kv_heads: int,
        block_size: int,
        head_dim: int,
        dtype: torch.dtype,
        device: str,
        layer_shapes: Optional[Sequence[Optional[Tuple[int, int, int]]]] = None,
        state: Optional[RecurrentStateCache] = None,
    ) -> None:
        """`layer_shapes`, when given, sizes every layer by itself:
        (kv_heads, key_dim, value_dim), or None for a layer without keys
        (its k_cache/v_cache entries are None). `state` ties recurrent-state
        slots to the life of a sequence's pages."""
        self.num_layers = num_layers
        self.num_blocks = num_blocks
        self.num_kv_heads = num_kv_heads
        self.block_size = block_size
        self.head_dim = head_dim
        if layer_shapes is None:
            layer_shapes = [(num_kv_heads, head_dim, head_dim)] * num_layers
        self.layer_shapes = list(layer_shapes)
        self.k_cache: List[Optional[torch.Tensor]] = []
        self.v_cache: List[Optional[torch.Tensor]] = []
        for sh in self.layer_shapes:
            if sh is None:
                self.k_cache.append(None)
                self.v_cache.append(None)
                continue
            kvh, kd, vd = sh
            self.k_cache.append(torch.zeros((num_blocks, kvh, block_size, kd),
                                            dtype=dtype, device=device))
            self.v_cache.append(torch.zeros((num_blocks, kvh, block_size, vd),
                                            dtype=dtype, device=device))
        self.allocator = BlockAllocator(num_blocks)
        self.state = state
        # per-sequence block tables (python side; tensorized per step)
        self.block_tables: Dict[int, List[int]] = {}

    def blocks_needed(self, seq_len: int) -> int:
        return (seq_len + self.block_size - 1) // self.block_size

    def can_grow(self, req_id: int, new_len: int) -> bool:
        have = len(self.block_tables.get(req_id, []))
        if (self.state is not None and req_id not in self.state.slots
                and self.state.num_free == 0):
            return False
        return self.blocks_needed(new_len) - have <= self.allocator.num_free

    def grow(self, req_id: int, new_len: int) -> None:
        """Ensure the sequence has pages covering new_len tokens."""
        if self.state is not None:
            self.state.acquire(req_id)
        table = self.block_tables.setdefault(req_id, [])
        need = self.blocks_needed(new_len) - len(table)
        if need > 0:
            table.extend(self.allocator.allocate(need))

    def release(self, req_id: int) -> None:
        table = self.block_tables.pop(req_id, None)
        if table:
            self.allocator.free(table)
        if self.state is not None:
            self.state.release(req_id)

    def slot(self, req_id: int, pos: int) -> int:
        """Flat slot index for token position `pos` of a sequence."""
        table = self.block_tables[req_id]
        return table[pos // self.block_size] * self.block_size + pos % self.block_size
