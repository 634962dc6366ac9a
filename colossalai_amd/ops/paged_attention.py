"""Attention of a ragged serving batch over paged keys and values.

Prompt portions and single decode tokens run in one call: each new token
attends over the pages of its own sequence, which already hold this step's
keys (``paged_kv_write`` runs first). Masking and bias are parameters:

* causal, optionally limited to a sliding ``window`` (query ``i`` sees key
  ``j`` when ``i - j < window``) with the first ``keep_first`` positions always
  visible (attention sinks that keep their true positions);
* an optional per-head linear distance penalty ``slopes[h] * (i - j)`` taken
  off the scaled score;
* an optional per-head output gate ``sigmoid(gate[n, h])``;
* an optional soft cap ``softcap * tanh(score / softcap)`` on the scaled score
  (before the distance penalty);
* an optional *sink*: one more place of score 0 in the softmax denominator that
  carries no value, ``p_j = exp(s_j) / (1 + sum exp(s_j))``, so a query may
  attend to nothing; with ``sink_logits`` the place has a learned score per
  head instead of 0, ``p_j = exp(s_j) / (exp(sink_h) + sum exp(s_j))``;
* an optional additive distance table ``dist_bias[min(i - j, rows - 1), h]``
  (after scale and cap; ``distance_bias_table`` fills one from a bucketed
  table of learned rows);
* optional *block summaries* of what lies before the window: with
  ``pooled = (key summaries, value summaries, P)`` a query at position ``i``
  with window ``w`` also sees one key and value for every block of ``P``
  positions ``[bP, bP + P)`` that ends at or before ``i - w``; the summaries are
  the means of the block's cached keys and values (``paged_pool_write``), they
  share the softmax with the window's keys and get no distance terms;
* optional *talking heads*: the softmax weights of the heads are mixed,
  ``p'_h = sum_g talk[h, g] p_g``, before head ``h`` applies them to the values
  of its own key/value head.

Scores, softmax weights and the accumulation are float32. Key and value head
sizes may differ; query head ``h`` reads key/value head ``h // (H / G)``.
"""

import math
from typing import Optional, Tuple

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip
from .ragged import RaggedBatch

__all__ = ["paged_kv_write", "paged_attention", "paged_attention_ref", "distance_slopes", "distance_bias_table",
           "summary_rows_per_page", "paged_pool_write", "paged_pool_write_ref", "mix_values"]


def distance_slopes(num_heads: int, device=None) -> torch.Tensor:
    """Geometric head slopes 2^(-8 (h + 1) / H)."""
    h = torch.arange(1, num_heads + 1, dtype=torch.float64)
    return torch.pow(2.0, -8.0 * h / num_heads).to(torch.float32).to(device)


def distance_bias_table(rows: torch.Tensor, far: float, length: int) -> torch.Tensor:
    """Per-distance bias ``[length, H]`` (float32) from a bucketed table ``rows`` [B, H]: distances below ``B // 2``
    have a row each, the rows above are spread logarithmically up to distance ``far``, the last row serves every
    larger distance: ``bucket(n) = n`` for ``n < B/2``, else
    ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(far / (B/2)) * (B - B/2)))``. The attention op clamps a distance
    to ``length - 1``, so ``length`` is the window, or ``ceil(far) + 1`` without one."""
    B = rows.shape[0]
    half = B // 2
    n = torch.arange(max(int(length), 1), dtype=torch.float64)
    if half > 0 and far > half:
        log_part = half + torch.floor(torch.log(n.clamp(min=half) / half) / math.log(far / half) * (B - half))
    else:
        log_part = torch.full_like(n, B - 1)
    bucket = torch.where(n < half, n, log_part.clamp(max=B - 1)).long()
    return rows.float()[bucket.to(rows.device)].contiguous()


def summary_rows_per_page(page_size: int, block: int) -> int:
    """Rows per page of a block-summary pool: summary ``b`` of a sequence lives in the sequence's page
    ``b // rows`` at row ``b % rows``; with ``rows >= page_size / block`` (rounded up to a power of two) that page is
    one the sequence already owns when the block is complete."""
    need = (page_size + block - 1) // block
    rows = 1
    while rows < need:
        rows <<= 1
    return rows


def paged_pool_write_ref(kpool, vpool, ksum, vsum, batch: RaggedBatch, block: int):
    ps, R = kpool.shape[1], ksum.shape[1]
    for i in range(batch.num_seqs):
        s0, n = batch.start_host[i], batch.cu_host[i + 1] - batch.cu_host[i]
        table = batch.block_tables[i].long()
        for b in range(s0 // block, (s0 + n) // block):
            pos = torch.arange(b * block, (b + 1) * block, device=kpool.device)
            pg, off = table[pos // ps], pos % ps
            ksum[table[b // R], b % R] = kpool[pg, off].float().mean(0).to(ksum.dtype)
            vsum[table[b // R], b % R] = vpool[pg, off].float().mean(0).to(vsum.dtype)


def paged_pool_write(kpool, vpool, ksum, vsum, batch: RaggedBatch, block: int):
    """Refresh the block summaries this step completes: for every sequence and every block ``b`` of ``block``
    positions whose last position is among the step's new tokens, the float32 means of the block's cached keys and
    values go to row ``b`` of the summary pools ([pages, rows_per_page, G, D] / [.., Dv], addressed through the
    sequence's own page table). Runs after ``paged_kv_write`` and before the attention of the same step."""
    if use_hip(kpool):
        most = max((batch.start_host[i] + batch.cu_host[i + 1] - batch.cu_host[i]) // block - batch.start_host[i] // block
                   for i in range(batch.num_seqs))
        if most > 0:
            serving_kernels().paged_pool_write(kpool, vpool, ksum, vsum, batch.block_tables, batch.cu, batch.start,
                                               block, most)
        return
    paged_pool_write_ref(kpool, vpool, ksum, vsum, batch, block)


def mix_values(v, v_first, lam: float):
    """``(1 - lam) v + lam v_first`` in float32, rounded once to v's dtype; v, v_first [N, C] (rows may be strided)."""
    if use_hip(v):
        return serving_kernels().lerp_rows(v, v_first, float(lam))
    return torch.lerp(v.float(), v_first.float(), float(lam)).to(v.dtype)


def paged_kv_write(k, v, kpool, vpool, batch: RaggedBatch):
    """k [N, G, D], v [N, G, Dv] -> rows ``batch.kv_rows`` of the pools
    ([pages, page_size, G, D] / [.., Dv])."""
    if use_hip(k):
        serving_kernels().paged_kv_write(k, v, kpool, vpool, batch.kv_rows)
        return
    rows = batch.kv_rows.long()
    kpool.view(-1, *kpool.shape[2:])[rows] = k.to(kpool.dtype)
    vpool.view(-1, *vpool.shape[2:])[rows] = v.to(vpool.dtype)


def paged_attention_ref(q, kpool, vpool, batch: RaggedBatch, scale: float, window: int = 0, keep_first: int = 0,
                        slopes: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                        softcap: float = 0.0, sink: bool = False, sink_logits: Optional[torch.Tensor] = None,
                        dist_bias: Optional[torch.Tensor] = None, pooled: Optional[Tuple] = None,
                        talk: Optional[torch.Tensor] = None):
    N, H, D = q.shape
    G, Dv = vpool.shape[2], vpool.shape[3]
    ps = kpool.shape[1]
    out = torch.empty(N, H, Dv, dtype=torch.float32, device=q.device)
    for i in range(batch.num_seqs):
        lo, hi, s0 = batch.cu_host[i], batch.cu_host[i + 1], batch.start_host[i]
        L = s0 + hi - lo
        pages = batch.block_tables[i, : (L + ps - 1) // ps].long()
        kk = kpool[pages].reshape(-1, G, D)[:L].float().repeat_interleave(H // G, 1)   # [L, H, D]
        vv = vpool[pages].reshape(-1, G, Dv)[:L].float().repeat_interleave(H // G, 1)
        qi = torch.arange(s0, L, device=q.device)[:, None]
        kj = torch.arange(L, device=q.device)[None, :]
        dist = (qi - kj).float()
        s = torch.einsum("nhd,lhd->hnl", q[lo:hi].float(), kk) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if slopes is not None:
            s = s - slopes.float()[:, None, None] * dist
        if dist_bias is not None:
            rows_of = dist.clamp(min=0, max=dist_bias.shape[0] - 1).long()
            s = s + dist_bias.float()[rows_of].permute(2, 0, 1)
        seen = kj <= qi
        if window > 0:
            seen = seen & ((qi - kj < window) | (kj < keep_first))
        s = s.masked_fill(~seen, float("-inf"))
        n_sum = 0
        if pooled is not None:  # one summary per block that ends at or before i - window, ahead of the keys
            ksum, vsum, P = pooled
            R = ksum.shape[1]
            n_sum = max(0, (L - window) // P)
            if n_sum:
                b = torch.arange(n_sum, device=q.device)
                pg = batch.block_tables[i].long()[b // R]
                ks = ksum[pg, b % R].float().repeat_interleave(H // G, 1)        # [n_sum, H, D]
                vs = vsum[pg, b % R].float().repeat_interleave(H // G, 1)
                s2 = torch.einsum("nhd,lhd->hnl", q[lo:hi].float(), ks) * scale
                if softcap > 0:
                    s2 = softcap * torch.tanh(s2 / softcap)
                seen2 = (b[None, :] * P + P - 1) <= (qi - window)
                s = torch.cat([s2.masked_fill(~seen2, float("-inf")), s], -1)
                vv = torch.cat([vs, vv], 0)
        if sink_logits is not None:  # a column without a value whose score is learned per head
            s = torch.cat([s, sink_logits.float()[:, None, None].expand(H, hi - lo, 1)], -1)
        elif sink:  # a zero-score column without a value
            s = torch.cat([s, torch.zeros_like(s[..., :1])], -1)
        p = torch.softmax(s, -1)[..., : L + n_sum]
        if talk is not None:
            p = torch.einsum("hg,gnl->hnl", talk.float(), p)
        out[lo:hi] = torch.einsum("hnl,lhv->nhv", p, vv)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.to(q.dtype)


def paged_attention(q, kpool, vpool, batch: RaggedBatch, scale: float, window: int = 0, keep_first: int = 0,
                    slopes: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                    softcap: float = 0.0, sink: bool = False, sink_logits: Optional[torch.Tensor] = None,
                    dist_bias: Optional[torch.Tensor] = None, pooled: Optional[Tuple] = None,
                    talk: Optional[torch.Tensor] = None):
    """q [N, H, D]; returns [N, H, Dv] in q's dtype. ``window == 0`` means no
    window; ``gate`` [N, H] logits or None; ``softcap == 0`` means no cap;
    ``sink_logits`` [H] float32; ``dist_bias`` [rows, H] float32; ``pooled`` =
    (key summaries, value summaries, block) needs a window; ``talk`` [H, H]."""
    assert pooled is None or window > 0, "block summaries stand for what a window no longer shows"
    if use_hip(q) and (sink_logits is not None or dist_bias is not None or pooled is not None or talk is not None):
        # With talking heads the kernels hand back every query head's weights applied to every key/value head's
        # values, O[n, g, c] (float32): the mix is linear, so out[n, h] = sum_g talk[h, g] O[n, g, kv(h)]
        ksum, vsum, block = pooled if pooled is not None else (None, None, 0)
        o = serving_kernels().paged_attention_ext(q, kpool, vpool, batch.block_tables, batch.cu, batch.start,
                                                  batch.tok_seq, batch.positions, scale, window, keep_first, slopes,
                                                  gate, float(softcap), bool(sink), sink_logits, dist_bias, ksum, vsum,
                                                  int(block), talk is not None, batch.num_tiles32, batch.num_tiles128)
        if talk is None:
            return o
        return serving_kernels().talk_mix(o, talk, q.dtype)
    if use_hip(q):
        return serving_kernels().paged_attention(q, kpool, vpool, batch.block_tables, batch.cu, batch.start,
                                                 batch.tok_seq, batch.positions, scale, window, keep_first,
                                                 slopes, gate, batch.num_tiles32, float(softcap), bool(sink),
                                                 batch.num_tiles128)
    return paged_attention_ref(q, kpool, vpool, batch, scale, window, keep_first, slopes, gate, softcap, sink,
                               sink_logits, dist_bias, pooled, talk)
