"""Attention whose keys and values are up-projections of one cached latent.

A token caches a single row ``[c | r]``: the RMS-normed latent ``c`` (``rank``
channels) and one rotated key part ``r`` (``R`` channels) that all heads share.
Head ``h`` has the key ``[U_k^h c | r]`` and the value ``U_v^h c``; its score with
a query ``[q_h | s_h]`` (``s_h`` rotated) is

    q_h . (U_k^h c) + s_h . r  =  ((U_k^h)^T q_h) . c + s_h . r,

so with the query carried into the latent space (``absorb_queries``) attention
runs as multi-query attention over the cached rows themselves — one key head of
``rank + R`` channels whose first ``rank`` channels are also the value — and
the per-head value ``U_v^h (sum_j p_j c_j)`` is taken after the weighted sum
(``expand_values``). The paged-attention op does the middle part; its value pool
is a view of the key pool.

That form reads ``rank + R`` channels per key and head, which is what a decode
step wants (the cache is read once for all heads) and more arithmetic than the
per-head form. For prompt portions in bfloat16 whose per-head sizes fit the
matrix-core attention kernel, ``latent_attention`` instead up-projects the
latents of the step's sequences (cached tokens included) into per-head keys
``[U_k^h c | r]`` and values in a dense scratch layout and runs ordinary
multi-head attention over it (``expanded_attention``); the cache itself still
holds latents only.

``latent_kv_write`` forms a step's rows (norm of the latent part, rotation of
the shared key part) and scatters them into the pool in one launch.
"""

from typing import Optional

import dataclasses

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip
from .group_norm import grouped_rms_norm_ref
from .paged_attention import paged_attention
from .pair_rotary import rotate_pairs, rotate_pairs_ref
from .ragged import RaggedBatch

__all__ = ["latent_kv_write", "latent_kv_write_ref", "absorb_queries", "expand_values", "latent_attention",
           "expanded_attention", "expands"]

# per-head key size (plain + rotated) and value size up to which prompt portions take the per-head form: what the
# matrix-core attention kernel tiles
EXPAND_MAX_HEAD = 128


def latent_kv_write_ref(dkv, norm_w, eps: float, freqs, pool, batch: RaggedBatch):
    rank = norm_w.numel()
    c = grouped_rms_norm_ref(dkv[:, :rank], norm_w, 1, eps, None, torch.float32)
    r = rotate_pairs_ref(dkv[:, None, rank:].float(), batch.positions, freqs)[:, 0]
    rows = batch.kv_rows.long()
    pool.view(-1, pool.shape[-1])[rows] = torch.cat([c, r], -1).to(pool.dtype)


def latent_kv_write(dkv, norm_w, eps: float, freqs, pool, batch: RaggedBatch):
    """dkv [N, rank + R] (rows may be strided): the first ``rank`` channels are RMS-normed with ``norm_w`` (float32
    statistics), the last ``R`` rotated pair-wise by the tokens' positions; the row goes to ``batch.kv_rows`` of
    ``pool`` [pages, page_size, 1, rank + R]."""
    assert pool.shape[2] == 1 and pool.shape[3] == dkv.shape[1]
    if use_hip(dkv):
        serving_kernels().latent_kv_write(dkv, norm_w, eps, freqs, batch.positions, pool, batch.kv_rows)
        return
    latent_kv_write_ref(dkv, norm_w, eps, freqs, pool, batch)


def absorb_queries(q, w_uk, positions, freqs, rank: int):
    """q [N, H, D + R] (``D`` plain, ``R`` rotated channels per head), w_uk [H, D, rank] -> [N, H, rank + R]:
    ``(U_k^h)^T q_h`` next to the rotated ``s_h``."""
    N, H, DR = q.shape
    D = w_uk.shape[1]
    out = torch.empty(N, H, rank + DR - D, dtype=q.dtype, device=q.device)
    torch.bmm(q[:, :, :D].transpose(0, 1), w_uk, out=out[:, :, :rank].transpose(0, 1))
    rotate_pairs(q[:, :, D:], positions, freqs, out=out[:, :, rank:])
    return out


def expand_values(o, w_uv):
    """o [N, H, rank] (weighted sums of latents), w_uv [H, Dv, rank] -> [N, H * Dv]."""
    N, H, _ = o.shape
    out = torch.empty(N, H, w_uv.shape[1], dtype=o.dtype, device=o.device)
    torch.bmm(o.transpose(0, 1), w_uv.transpose(1, 2), out=out.transpose(0, 1))
    return out.view(N, -1)


def expands(q, w_uk, w_uv, batch: RaggedBatch) -> bool:
    """Whether a step takes the per-head form: bfloat16 on the GPU, a prompt portion in the step, head sizes the
    matrix-core kernel tiles."""
    Dk, Dv = q.shape[2], w_uv.shape[1]
    return (use_hip(q) and q.dtype == torch.bfloat16 and batch.num_tiles32 > 0 and Dk % 8 == 0 and Dv % 8 == 0
            and Dk <= EXPAND_MAX_HEAD and Dv <= EXPAND_MAX_HEAD)


def expanded_attention(q, w_uk, w_uv, pool, batch: RaggedBatch, scale: float, freqs, rank: int,
                       gate: Optional[torch.Tensor] = None, window: int = 0, keep_first: int = 0):
    """The per-head form: keys ``[U_k^h c | r]`` and values ``U_v^h c`` of every token the step's sequences hold,
    laid out densely (``RaggedBatch.dense_context``), then multi-head attention over that layout. q [N, H, D + R]
    un-rotated (its rotated part is turned in place). Returns [N, H * Dv]."""
    N, H, DR = q.shape
    D, Dv = w_uk.shape[1], w_uv.shape[1]
    rows, tables, total = batch.dense_context()
    ctx = pool.view(-1, pool.shape[-1]).index_select(0, rows)                     # [total, rank + R]
    keys = torch.empty(total, H, DR, dtype=q.dtype, device=q.device)
    torch.bmm(ctx[:, :rank].unsqueeze(0).expand(H, total, rank), w_uk.transpose(1, 2),
              out=keys[:, :, :D].transpose(0, 1))
    keys[:, :, D:] = ctx[:, None, rank:]
    values = torch.mm(ctx[:, :rank], w_uv.reshape(H * Dv, rank).t())              # [total, H * Dv]
    rotate_pairs(q[:, :, D:], batch.positions, freqs, out=q[:, :, D:])
    ps = batch.page_size
    dense = dataclasses.replace(batch, block_tables=tables, kv_rows=None, _dense=None)
    o = paged_attention(q, keys.view(total // ps, ps, H, DR), values.view(total // ps, ps, H, Dv), dense, scale,
                        window, keep_first, None, gate)
    return o.reshape(N, H * Dv)


def latent_attention(q, w_uk, w_uv, pool, batch: RaggedBatch, scale: float, freqs, rank: int,
                     gate: Optional[torch.Tensor] = None, window: int = 0, keep_first: int = 0):
    """Causal softmax attention of a ragged step over latent rows already in ``pool``. q [N, H, D + R] un-rotated;
    ``gate`` [N, H] logits of a per-head sigmoid output gate. Returns [N, H * Dv]."""
    if expands(q, w_uk, w_uv, batch):
        return expanded_attention(q, w_uk, w_uv, pool, batch, scale, freqs, rank, gate, window, keep_first)
    qa = absorb_queries(q, w_uk, batch.positions, freqs, rank)
    o = paged_attention(qa, pool, pool[..., :rank], batch, scale, window, keep_first, None, gate)
    return expand_values(o, w_uv)
