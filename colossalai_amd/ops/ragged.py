"""Ragged serving batch descriptor shared by the sequence-state ops.

One engine step runs ``N`` new tokens that belong to ``B`` live sequences:
a prompt portion of any length next to single decode tokens. Every op that
carries per-sequence memory (paged keys/values, recurrent matrices, the tail
of a short convolution, the previous token of a token shift) takes this
descriptor instead of a dense ``[B, S]`` layout, so that a result never
depends on how a prompt was cut or on what else shares the step.
"""

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

__all__ = ["RaggedBatch"]


@dataclass
class RaggedBatch:
    # device tensors (int32)
    cu: torch.Tensor          # [B + 1] offsets of each sequence's new tokens in the flat token axis
    start: torch.Tensor       # [B] tokens the sequence already holds (= position of its first new token)
    slots: torch.Tensor       # [B] state slot of each sequence
    tok_seq: torch.Tensor     # [N] which sequence (0..B-1) a token belongs to
    positions: torch.Tensor   # [N] absolute position of a token in its sequence
    block_tables: Optional[torch.Tensor]  # [B, max_blocks] page ids (None when no layer keeps keys)
    kv_rows: Optional[torch.Tensor]       # [N] flat pool row (page * page_size + offset) of each token
    # host mirrors
    cu_host: List[int]
    start_host: List[int]
    slots_host: List[int]
    page_size: int = 0
    _dense: Optional[tuple] = None  # memo of dense_context()
    _scan_chunks: Optional[tuple] = None  # memo of the selective scan's chunk tables

    @property
    def num_seqs(self) -> int:
        return len(self.start_host)

    @property
    def num_tokens(self) -> int:
        return self.cu_host[-1]

    @property
    def max_new(self) -> int:
        return max(self.cu_host[i + 1] - self.cu_host[i] for i in range(self.num_seqs))

    @property
    def num_tiles32(self) -> int:
        """32-token tiles of the prompt portions (0 for a pure decode step):
        the grid of the matrix-core attention kernel."""
        if self.max_new == 1:
            return 0
        return sum((self.cu_host[i + 1] - self.cu_host[i] + 31) // 32 for i in range(self.num_seqs))

    @property
    def num_tiles128(self) -> int:
        """128-token tiles of the prompt portions (0 for a pure decode step): the grid of the matrix-core attention
        kernel when every key head has a single query head."""
        if self.max_new == 1:
            return 0
        return sum((self.cu_host[i + 1] - self.cu_host[i] + 127) // 128 for i in range(self.num_seqs))

    @property
    def max_total(self) -> int:
        """Longest sequence after this step (cached + new tokens)."""
        return max(self.start_host[i] + self.cu_host[i + 1] - self.cu_host[i] for i in range(self.num_seqs))

    def dense_context(self):
        """For ops that lay the whole context of the step's sequences (cached and new tokens) out densely, each
        sequence padded to whole pages: ``(rows, tables, total)`` with ``rows`` [total] the pool row of every place
        of that layout (a padding place repeats the sequence's last row) and ``tables`` [B, max_pages] int32 the page
        table of the dense layout itself (consecutive pages, sequence after sequence). Built on the device from
        the step's own index vectors, once per step."""
        if self._dense is None:
            ps, dev = self.page_size, self.cu.device
            shift = ps.bit_length() - 1
            lens = [self.start_host[i] + self.cu_host[i + 1] - self.cu_host[i] for i in range(self.num_seqs)]
            pages = [(n + ps - 1) // ps for n in lens]
            first, total_pages = [], 0
            for n in pages:
                first.append(total_pages)
                total_pages += n
            width = max(pages)
            host = torch.tensor([first, pages, lens], dtype=torch.int32).to(dev)   # one copy
            first_d, pages_d, lens_d = host[0].long(), host[1].long(), host[2].long()
            total = total_pages * ps
            seq = torch.repeat_interleave(torch.arange(self.num_seqs, device=dev), pages_d * ps, output_size=total)
            pos = torch.arange(total, device=dev) - first_d[seq] * ps
            pos = torch.minimum(pos, lens_d[seq] - 1)
            rows = (self.block_tables[seq, pos >> shift].long() << shift) + (pos & (ps - 1))
            cols = torch.arange(width, device=dev)
            tables = torch.where(cols[None, :] < pages_d[:, None], first_d[:, None] + cols[None, :], 0).int()
            self._dense = (rows, tables.contiguous(), total)
        return self._dense

    @classmethod
    def build(cls, new_counts: Sequence[int], starts: Sequence[int], slots: Sequence[int], device,
              tables: Optional[Sequence[Sequence[int]]] = None, page_size: int = 0) -> "RaggedBatch":
        cu = [0]
        for n in new_counts:
            assert n > 0, "a sequence in a step brings at least one token"
            cu.append(cu[-1] + n)
        tok_seq, pos, rows = [], [], []
        for i, n in enumerate(new_counts):
            tok_seq += [i] * n
            pos += list(range(starts[i], starts[i] + n))
            if tables is not None:
                t = tables[i]
                assert len(t) * page_size >= starts[i] + n, "block table does not cover the new tokens"
                rows += [t[p // page_size] * page_size + p % page_size for p in range(starts[i], starts[i] + n)]
        # one host-to-device copy for all index vectors of the step; the fields are views into it
        B = len(new_counts)
        parts = [cu, list(starts), list(slots), tok_seq, pos]
        width = 0
        if tables is not None:
            width = max(len(t) for t in tables)
            parts += [[p for t in tables for p in list(t) + [0] * (width - len(t))], rows]
        flat = [v for part in parts for v in part]
        buf = torch.tensor(flat, dtype=torch.int32).to(device)
        sizes = [len(part) for part in parts]
        views, at = [], 0
        for n in sizes:
            views.append(buf[at : at + n])
            at += n
        return cls(
            cu=views[0], start=views[1], slots=views[2], tok_seq=views[3], positions=views[4],
            block_tables=views[5].view(B, width) if tables is not None else None,
            kv_rows=views[6] if tables is not None else None,
            cu_host=cu, start_host=list(starts), slots_host=list(slots), page_size=page_size,
        )
