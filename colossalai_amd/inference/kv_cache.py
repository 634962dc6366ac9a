"""Paged KV cache manager (reference: colossalai/inference/kv_cache/
kvcache_manager.py — vLLM-style block pool, MI355X sizing).

One K and one V pool per layer, shaped [num_blocks, block_size, Hkv, D]
(block_size a power of two so the decode kernel folds addressing into
shift/mask). 288 GB HBM3E holds ~1.5M tokens of llama-7B KV at bf16, so
the default pool is sized generously and admission control, not eviction,
is the knob. Blocks are handed out from a free list; sequences own a
block-id list that becomes a row of the [B, max_blocks] block-table tensor
fed to ``decode_attention_paged``.
"""

from typing import Dict, List, Optional

import torch

__all__ = ["KVCacheManager"]


class KVCacheManager:
    def __init__(
        self,
        num_layers: int,
        num_kv_heads: int,
        head_dim: int,
        num_blocks: int = 2048,
        block_size: int = 16,
        device=None,
        dtype=torch.bfloat16,
        layer_shapes: Optional[List[Optional[tuple]]] = None,
        layer_sources: Optional[List[Optional[int]]] = None,
        layer_summaries: Optional[List[Optional[int]]] = None,
    ):
        """``layer_shapes`` (optional) gives each layer its own
        ``(kv_heads, key_dim, value_dim)`` or ``None`` for a layer that keeps no
        keys (a recurrent layer of a hybrid model); without it every layer gets
        ``(num_kv_heads, head_dim, head_dim)``. ``layer_sources`` (optional)
        names, for a layer that projects no keys of its own, the layer whose
        pools it reads: ``k_pools[i]`` / ``v_pools[i]`` are then that layer's
        tensors (no second copy; the pages and page tables are shared by all
        layers anyway), and the layer's own shape entry must be ``None``.
        ``layer_summaries`` (optional) gives, for a layer whose attention also reads
        one mean key and value per block of ``P`` positions, that ``P``: the layer
        gets a second, small pair of pools ``k_summaries[i]`` / ``v_summaries[i]``
        ``[num_blocks, rows, Hkv, D]`` with ``rows = summary_rows_per_page(block_size, P)``;
        summary ``b`` of a sequence lives in its page ``b // rows`` at row ``b % rows``,
        so the sequence's page table addresses both pools and freeing its pages
        frees its summaries."""
        assert block_size & (block_size - 1) == 0, "block_size must be a power of two"
        self.num_layers = num_layers
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.device = device or ("cuda" if torch.cuda.is_available() else "cpu")
        if layer_shapes is None:
            layer_shapes = [(num_kv_heads, head_dim, head_dim)] * num_layers
        assert len(layer_shapes) == num_layers
        self.layer_shapes = list(layer_shapes)
        self.k_pools = [
            None if s is None else torch.zeros(num_blocks, block_size, s[0], s[1], device=self.device, dtype=dtype)
            for s in layer_shapes
        ]
        self.v_pools = [
            None if s is None else torch.zeros(num_blocks, block_size, s[0], s[2], device=self.device, dtype=dtype)
            for s in layer_shapes
        ]
        self.layer_sources = list(layer_sources) if layer_sources is not None else [None] * num_layers
        assert len(self.layer_sources) == num_layers
        for i, src in enumerate(self.layer_sources):
            if src is not None:
                assert layer_shapes[i] is None, f"layer {i} reads layer {src}'s pools and keeps none of its own"
                assert self.layer_sources[src] is None and self.k_pools[src] is not None, \
                    f"layer {i} reads keys of layer {src}, which keeps none"
                self.k_pools[i], self.v_pools[i] = self.k_pools[src], self.v_pools[src]
        self.layer_summaries = list(layer_summaries) if layer_summaries is not None else [None] * num_layers
        assert len(self.layer_summaries) == num_layers
        self.k_summaries: List[Optional[torch.Tensor]] = [None] * num_layers
        self.v_summaries: List[Optional[torch.Tensor]] = [None] * num_layers
        for i, P in enumerate(self.layer_summaries):
            if P is None:
                continue
            from ..ops.paged_attention import summary_rows_per_page

            s = layer_shapes[i]
            assert s is not None and P >= 1, f"layer {i} summarises keys it does not keep"
            rows = summary_rows_per_page(block_size, int(P))
            self.k_summaries[i] = torch.zeros(num_blocks, rows, s[0], s[1], device=self.device, dtype=dtype)
            self.v_summaries[i] = torch.zeros(num_blocks, rows, s[0], s[2], device=self.device, dtype=dtype)
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))
        self._tables: Dict[int, List[int]] = {}  # seq id -> block ids

    # ------------------------------------------------------------- accounting
    @property
    def free_blocks(self) -> int:
        return len(self._free)

    def blocks_needed(self, num_tokens: int) -> int:
        return (num_tokens + self.block_size - 1) // self.block_size

    def can_allocate(self, num_tokens: int) -> bool:
        return self.blocks_needed(num_tokens) <= self.free_blocks

    # ------------------------------------------------------------- allocation
    def has(self, seq_id) -> bool:
        return seq_id in self._tables

    def allocate(self, seq_id: int, num_tokens: int) -> None:
        need = self.blocks_needed(num_tokens)
        assert need <= self.free_blocks, "KV pool exhausted"
        self._tables[seq_id] = [self._free.pop() for _ in range(need)]

    def extend(self, seq_id: int, new_len: int) -> None:
        """Grow seq's table to cover new_len tokens (decode append)."""
        table = self._tables[seq_id]
        while len(table) * self.block_size < new_len:
            assert self._free, "KV pool exhausted"
            table.append(self._free.pop())

    def free(self, seq_id: int) -> None:
        self._free.extend(reversed(self._tables.pop(seq_id, [])))

    def table(self, seq_id: int) -> List[int]:
        return self._tables[seq_id]

    def block_tables_tensor(self, seq_ids: List[int]) -> torch.Tensor:
        mb = max(len(self._tables[s]) for s in seq_ids)
        bt = torch.zeros(len(seq_ids), mb, dtype=torch.int32, device=self.device)
        for i, s in enumerate(seq_ids):
            ids = self._tables[s]
            bt[i, : len(ids)] = torch.tensor(ids, dtype=torch.int32, device=self.device)
        return bt

    # ---------------------------------------------------------------- writes
    def write_prefill(self, layer: int, seq_id: int, k: torch.Tensor, v: torch.Tensor) -> None:
        """k/v [S, Hkv, D] for one sequence's prompt."""
        S = k.shape[0]
        bs = self.block_size
        table = self._tables[seq_id]
        for bi in range((S + bs - 1) // bs):
            lo, hi = bi * bs, min((bi + 1) * bs, S)
            self.k_pools[layer][table[bi], : hi - lo] = k[lo:hi]
            self.v_pools[layer][table[bi], : hi - lo] = v[lo:hi]

    def write_token(self, layer: int, seq_id: int, pos: int, k: torch.Tensor, v: torch.Tensor) -> None:
        """k/v [Hkv, D] for the token at position pos."""
        bs = self.block_size
        blk = self._tables[seq_id][pos // bs]
        self.k_pools[layer][blk, pos % bs] = k
        self.v_pools[layer][blk, pos % bs] = v

    # ----------------------------------------------------------------- reads
    def gather_contiguous(self, layer: int, seq_id: int, length: int):
        """CPU/reference path: materialize [length, Hkv, D] K and V."""
        table = self._tables[seq_id]
        nb = self.blocks_needed(length)
        idx = torch.tensor(table[:nb], dtype=torch.long, device=self.device)
        k = self.k_pools[layer][idx].reshape(-1, *self.k_pools[layer].shape[2:])[:length]
        v = self.v_pools[layer][idx].reshape(-1, *self.v_pools[layer].shape[2:])[:length]
        return k, v
