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
  attend to nothing.

Scores, softmax weights and the accumulation are float32. Key and value head
sizes may differ; query head ``h`` reads key/value head ``h // (H / G)``.
"""

from typing import Optional

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip
from .ragged import RaggedBatch

__all__ = ["paged_kv_write", "paged_attention", "paged_attention_ref", "distance_slopes"]


def distance_slopes(num_heads: int, device=None) -> torch.Tensor:
    """Geometric head slopes 2^(-8 (h + 1) / H)."""
    h = torch.arange(1, num_heads + 1, dtype=torch.float64)
    return torch.pow(2.0, -8.0 * h / num_heads).to(torch.float32).to(device)


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
                        softcap: float = 0.0, sink: bool = False):
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
        seen = kj <= qi
        if window > 0:
            seen = seen & ((qi - kj < window) | (kj < keep_first))
        s = s.masked_fill(~seen, float("-inf"))
        if sink:  # a zero-score column without a value
            s = torch.cat([s, torch.zeros_like(s[..., :1])], -1)
        p = torch.softmax(s, -1)[..., :L]
        out[lo:hi] = torch.einsum("hnl,lhv->nhv", p, vv)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.to(q.dtype)


def paged_attention(q, kpool, vpool, batch: RaggedBatch, scale: float, window: int = 0, keep_first: int = 0,
                    slopes: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                    softcap: float = 0.0, sink: bool = False):
    """q [N, H, D]; returns [N, H, Dv] in q's dtype. ``window == 0`` means no
    window; ``gate`` [N, H] logits or None; ``softcap == 0`` means no cap."""
    if use_hip(q):
        return serving_kernels().paged_attention(q, kpool, vpool, batch.block_tables, batch.cu, batch.start,
                                                 batch.tok_seq, batch.positions, scale, window, keep_first,
                                                 slopes, gate, batch.num_tiles32, float(softcap), bool(sink),
                                                 batch.num_tiles128)
    return paged_attention_ref(q, kpool, vpool, batch, scale, window, keep_first, slopes, gate, softcap, sink)
