"""Paged caches: one page pool (block table, free list, per-sequence ownership) under every cache layout of the package.

A sequence lives in a slot (a row of the block table); a page holds `block` consecutive positions of one sequence in every layer.
Pages are handed out on demand, given back when a sequence ends and used again (last freed, first reused), so which pages and
which slot a sequence gets depends on what ran before it - the kernels find a position through the table only."""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch


class PagePool:
    def __init__(self, num_blocks: int, block: int, max_seqs: int, max_blocks_per_seq: int, device, position_limit: int = 0):
        self.block, self.device, self.num_blocks, self.max_seqs = int(block), device, int(num_blocks), int(max_seqs)
        self.max_blocks_per_seq = int(max_blocks_per_seq)
        self.position_limit = int(position_limit)     # 0: bounded by the table's width only
        self._bt_host = torch.full((max_seqs, self.max_blocks_per_seq), -1, dtype=torch.int32)
        self.block_table = self._bt_host.to(device)
        self._free = list(range(num_blocks - 1, -1, -1))
        self._owned: Dict[int, int] = {}

    @property
    def free_blocks(self) -> int:
        return len(self._free)

    def blocks_of(self, slot: int) -> List[int]:
        return [int(b) for b in self._bt_host[slot, : self._owned.get(slot, 0)]]

    def blocks_for(self, length: int) -> int:
        return (length + self.block - 1) // self.block

    def reserve(self, slot: int, length: int):
        """Make sure sequence `slot` owns blocks for positions [0, length). Host bookkeeping + one small upload."""
        need = (length + self.block - 1) // self.block
        have = self._owned.get(slot, 0)
        if need <= have:
            return
        if need > self.max_blocks_per_seq:
            limit = self.position_limit or self.max_blocks_per_seq * self.block
            raise RuntimeError(f"sequence length {length} exceeds max_pos {limit}")
        if need - have > len(self._free):
            raise RuntimeError("paged KV cache exhausted")
        for b in range(have, need):
            self._bt_host[slot, b] = self._free.pop()
        self._owned[slot] = need
        self.block_table[slot].copy_(self._bt_host[slot], non_blocking=True)

    def free(self, slot: int):
        for b in range(self._owned.pop(slot, 0)):
            self._free.append(int(self._bt_host[slot, b]))
            self._bt_host[slot, b] = -1
        self.block_table[slot].copy_(self._bt_host[slot], non_blocking=True)


class PagedKVCache(PagePool):
    """Per-layer K and V in the reference layout (num_blocks, 16, kv_heads, head_dim) + int32 block table (core/kv_cache.py:84-107)."""

    def __init__(self, cfg, num_blocks: int, max_seqs: int, device, dtype=torch.float32):
        super().__init__(num_blocks, cfg.kv_block, max_seqs, (cfg.max_pos + cfg.kv_block - 1) // cfg.kv_block, device, position_limit=cfg.max_pos)
        self.cfg, self.dtype = cfg, dtype
        shape = (num_blocks, cfg.kv_block, cfg.num_kv_heads, cfg.head_dim)
        self.k = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(cfg.num_layers)]
        self.v = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(cfg.num_layers)]


class LatentCache(PagePool):
    """One row per token and layer (latent attention: the normalised latent and the rotated shared key part, side by side):
    rows[l] is (num_blocks, block, widths[l]); layers may differ in width.  A sequence may hold the whole pool."""

    def __init__(self, widths: Sequence[int], num_blocks: int, max_seqs: int, device, dtype=torch.bfloat16, block: int = 16):
        super().__init__(num_blocks, block, max_seqs, max(1, num_blocks), device)
        self.dtype, self.widths = dtype, [int(w) for w in widths]
        self.rows = [torch.zeros((num_blocks, block, w), dtype=dtype, device=device) for w in self.widths]


class HybridCache(PagePool):
    """Cache of a model whose layers keep different things: pages of key rows for attention layers (one row per token, which is also
    the value, and the reciprocal root mean square of that row as a separate fp32 number), and per-slot state for recurrent layers
    (fp32, one entry per sequence, overwritten by every step).  specs[l] = {"rows": width} and / or {"state": {name: shape}};
    "kscale": False leaves the per-token number out (rows that hold keys and values as they are); {"rows_of": j} makes layer l read the
    rows of the earlier layer j (a layer that attends over another layer's keys and values holds none of its own).
    seq_state: per-slot state of the model as a whole, {name: (shape, dtype)}.  Recurrent state needs no clearing when a slot is used
    again: the kernels take it as empty for a row at position 0.  position_limit > 0 bounds a sequence's length (a model with a table
    of positions)."""

    def __init__(self, specs: Sequence[dict], num_blocks: int, max_seqs: int, device, dtype=torch.bfloat16, block: int = 16, seq_state=None,
                 position_limit: int = 0):
        per_seq = max(1, num_blocks) if position_limit <= 0 else max(1, min(num_blocks, (position_limit + block - 1) // block))
        super().__init__(num_blocks, block, max_seqs, per_seq, device, position_limit=position_limit)
        self.dtype = dtype
        self.rows: List = []
        self.kscale: List = []
        self.state: List[Dict[str, torch.Tensor]] = []
        for sp in specs:
            if sp.get("rows_of") is not None:
                j = int(sp["rows_of"])
                if not 0 <= j < len(self.rows) or self.rows[j] is None:
                    raise ValueError(f"layer {len(self.rows)} reads the rows of layer {j}, which has none")
                self.rows.append(self.rows[j])
                self.kscale.append(self.kscale[j])
                self.state.append({k: torch.zeros((max_seqs, *shape), dtype=torch.float32, device=device) for k, shape in (sp.get("state") or {}).items()})
                continue
            w = int(sp.get("rows", 0))
            self.rows.append(torch.zeros((num_blocks, block, w), dtype=dtype, device=device) if w else None)
            self.kscale.append(torch.zeros((num_blocks, block), dtype=torch.float32, device=device) if w and sp.get("kscale", True) else None)
            self.state.append({k: torch.zeros((max_seqs, *shape), dtype=torch.float32, device=device) for k, shape in (sp.get("state") or {}).items()})
        self.seq_state = {k: torch.zeros((max_seqs, *shape), dtype=dt, device=device) for k, (shape, dt) in (seq_state or {}).items()}

    def _state_tensors(self) -> List[torch.Tensor]:
        return [t for d in self.state for t in d.values()] + list(self.seq_state.values())

    def snapshot(self) -> List[torch.Tensor]:
        """Copies of every per-slot state tensor (not of the pages: writing a position's key again changes nothing)."""
        return [t.clone() for t in self._state_tensors()]

    def restore(self, held: List[torch.Tensor]) -> None:
        for t, h in zip(self._state_tensors(), held):
            t.copy_(h)
