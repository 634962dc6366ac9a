"""Mixture-of-experts feed-forward of the serving path: a group-limited top-k
router and the experts' two-matrix feed-forward over a flat token batch.

``grouped_topk_route`` turns float32 router logits into expert ids and mixing
weights:

* score ``s = sigmoid(z)``; the *choice* score is ``s + correction`` (a
  per-expert selection bias), the mixing weights use ``s`` alone;
* the ``E`` experts form ``group_count`` runs of neighbours; a group is worth the
  sum of its ``group_top`` largest choice scores and only the ``group_keep``
  best groups stay in the running (the others count as minus infinity, so a
  negative choice score inside a kept group still beats them);
* the ``top`` largest remaining choice scores are chosen (ties go to the lower
  index) and their plain scores are divided by their sum plus ``renorm_eps``.

With ``score="softmax"`` the scores are the softmax of the logits over all
experts, and with ``renorm=False`` the chosen scores are the mixing weights as
they are.

``routed_expert_ffn`` runs ``down_e(act(up_e(h)))`` for each token's chosen
experts and forms ``base + sum_j weight_j * y_j`` in float32. On the GPU nothing
of a bfloat16 step goes to the host: a small step (decode tokens) streams just
the chosen experts' weights through matrix-vector kernels; a larger one sorts
the (token, expert) pairs by expert on the device and runs each of the two
products for all experts in one grouped matrix-core launch that reads the
experts' row ranges from a device-side offsets vector. Float32 serving and
sizes the grouped kernel does not tile take one library product per expert
after a host-side count.
"""

from typing import Optional

import torch
import torch.nn.functional as F

from ._kernels import serving_kernels, use_serving_hip as use_hip
from .activation import relu_squared

__all__ = ["grouped_topk_route", "grouped_topk_route_ref", "routed_expert_ffn", "routed_expert_ffn_ref"]

# (token, expert) pairs up to which the matrix-vector kernels are used (measured crossover, 32 experts of 1024 x
# 2048: 66 against 84 us at 48 pairs, 95 against 88 us at 72): they re-read an expert's matrices (from cache) once
# per pair and take two launches, the grouped product reads them once per 128 rows and takes four
GEMV_MAX_PAIRS = 64
# ... and where the grouped product does not apply (float32 serving, sizes it does not tile): up to here the
# matrix-vector kernels beat the per-expert library products, whose launches and host round trip cost about 1.5 ms
GEMV_FALLBACK_PAIRS = 2048


def grouped_topk_route_ref(logits, correction, top: int, group_count: int = 1, group_keep: int = 1,
                           group_top: int = 2, renorm_eps: float = 1e-20, score: str = "sigmoid", renorm: bool = True):
    N, E = logits.shape
    s = torch.softmax(logits.float(), -1) if score == "softmax" else torch.sigmoid(logits.float())
    choice = s + correction.float() if correction is not None else s
    if group_count > 1:
        per = E // group_count
        grouped = choice.view(N, group_count, per)
        worth = grouped.topk(min(group_top, per), dim=-1).values.sum(-1)
        # stable descending order: ties go to the lower group
        kept = torch.sort(worth, dim=-1, descending=True, stable=True).indices[:, :group_keep]
        allowed = torch.zeros(N, group_count, dtype=torch.bool, device=logits.device)
        allowed.scatter_(1, kept, True)
        choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(N, E)
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    w = s.gather(1, idx)
    return idx.int(), (w / (w.sum(-1, keepdim=True) + renorm_eps) if renorm else w)


SCORES = {"sigmoid": 0, "softmax": 1}


def grouped_topk_route(logits, correction, top: int, group_count: int = 1, group_keep: int = 1,
                       group_top: int = 2, renorm_eps: float = 1e-20, score: str = "sigmoid", renorm: bool = True):
    """logits [N, E] float32 (rows may be strided), correction [E] or None -> (ids [N, top] int32, weights
    [N, top] float32). ``score``: "sigmoid" or "softmax" (over all experts); ``renorm``: divide the chosen scores
    by their sum."""
    N, E = logits.shape
    assert score in SCORES
    assert E % group_count == 0 and 0 < group_keep <= group_count
    assert 0 < top <= (E // group_count) * group_keep, "fewer experts in the kept groups than are to be chosen"
    if use_hip(logits):
        return serving_kernels().grouped_topk_route(logits.float(), correction, top, group_count,
                                                    group_keep, group_top, renorm_eps, SCORES[score], renorm)
    return grouped_topk_route_ref(logits, correction, top, group_count, group_keep, group_top, renorm_eps, score,
                                  renorm)


def _act(x, activation: str):
    if activation == "relu_squared":
        return relu_squared(x)
    raise ValueError(f"unknown expert activation {activation!r}")


def routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base=None, activation: str = "relu_squared",
                          base_gate=None):
    N, top = ids.shape
    out = torch.zeros(N, w_down.shape[1], dtype=torch.float32, device=h.device) if base is None else base.float().clone()
    if base is not None and base_gate is not None:
        out = out * torch.sigmoid(base_gate.float().reshape(N, 1))
    for e in range(w_up.shape[0]):
        rows, slot = (ids == e).nonzero(as_tuple=True)
        if rows.numel():
            y = F.linear(_act(F.linear(h[rows], w_up[e]), activation), w_down[e])
            out.index_add_(0, rows, y.float() * weights[rows, slot][:, None])
    return out


def _sort_pairs(ids, E: int):
    """(order, inverse, offsets) of the (token, expert) pairs sorted by expert, all on the device: ``order[r]`` is
    the pair at sorted row ``r`` (stable: ascending pair index inside an expert), ``offsets[e] .. offsets[e + 1]``
    the rows of expert ``e``."""
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    offsets = torch.zeros(E + 1, dtype=torch.int32, device=ids.device)
    offsets[1:] = torch.cumsum(torch.bincount(flat, minlength=E), 0)
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel(), device=order.device)
    return order, inv, offsets


SORT_KERNEL_MAX_PAIRS = 8192  # the one-block sort kernel holds a step's ids in LDS


def _grouped_expert_ffn(h, w_up, w_down, ids, weights, base, base_gate=None):
    """One grouped matrix-core launch per product; the up product gathers the tokens' rows itself and squares the
    rectified accumulator. Steps of up to 8192 pairs are sorted by one kernel, larger ones by library sorts."""
    N, top = ids.shape
    K = serving_kernels()
    if ids.numel() <= SORT_KERNEL_MAX_PAIRS:
        offsets, src, inv = K.expert_sort(ids.contiguous(), w_up.shape[0])
    else:
        order, inv, offsets = _sort_pairs(ids, w_up.shape[0])
        src, inv = (order // top).int(), inv.int().view(N, top)
    hidden = K.expert_grouped_gemm(h, src, w_up, offsets, ids.numel(), True)
    y = K.expert_grouped_gemm(hidden, None, w_down, offsets, ids.numel(), False)
    return K.expert_combine(y, inv, weights, base, base_gate)


def _sorted_expert_ffn(h, w_up, w_down, ids, weights, base, activation, base_gate=None):
    """Pairs sorted by expert, one up and one down library product per expert that got rows (their row counts come
    to the host), then every token gathers its ``top`` results in slot order."""
    N, top = ids.shape
    order, inv, offsets = _sort_pairs(ids, w_up.shape[0])
    bounds = offsets.tolist()
    x = h.index_select(0, order // top)
    hidden = torch.empty(x.shape[0], w_up.shape[1], dtype=h.dtype, device=h.device)
    for e in range(w_up.shape[0]):
        lo, hi = bounds[e], bounds[e + 1]
        if hi > lo:
            torch.mm(x[lo:hi], w_up[e].t(), out=hidden[lo:hi])
    hidden = _act(hidden, activation)
    y = torch.empty(x.shape[0], w_down.shape[1], dtype=h.dtype, device=h.device)
    for e in range(w_up.shape[0]):
        lo, hi = bounds[e], bounds[e + 1]
        if hi > lo:
            torch.mm(hidden[lo:hi], w_down[e].t(), out=y[lo:hi])
    return serving_kernels().expert_combine(y, inv.int().view(N, top), weights, base, base_gate)


def _grouped_fits(h, w_up, w_down) -> bool:
    return (h.dtype == torch.bfloat16 and w_up.shape[2] % 32 == 0 and w_up.shape[1] % 32 == 0
            and w_up.shape[0] <= 1024 and w_up.is_contiguous() and w_down.is_contiguous())


def routed_expert_ffn(h, w_up, w_down, ids, weights, base: Optional[torch.Tensor] = None,
                      activation: str = "relu_squared", base_gate: Optional[torch.Tensor] = None):
    """h [N, W]; w_up [E, F, W]; w_down [E, W, F]; ids [N, top] int32; weights
    [N, top] float32; ``base`` [N, W] (any activation type) is added, e.g. a
    shared expert's output, multiplied by ``sigmoid(base_gate)`` when
    ``base_gate`` ([N] float32 logits, any stride) is given. Returns float32 [N, W]."""
    if not use_hip(h):
        return routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base, activation, base_gate)
    assert base_gate is None or (base is not None and base_gate.dtype == torch.float32 and base_gate.numel() == h.shape[0])
    if activation != "relu_squared":
        raise ValueError(f"unknown expert activation {activation!r}")
    h = h.contiguous()
    if ids.numel() <= GEMV_MAX_PAIRS:
        return serving_kernels().expert_ffn_gemv(h, w_up, w_down, ids, weights, base, base_gate)
    if _grouped_fits(h, w_up, w_down):
        return _grouped_expert_ffn(h, w_up, w_down, ids, weights, base, base_gate)
    if ids.numel() <= GEMV_FALLBACK_PAIRS:
        return serving_kernels().expert_ffn_gemv(h, w_up, w_down, ids, weights, base, base_gate)
    return _sorted_expert_ffn(h, w_up, w_down, ids, weights, base, activation, base_gate)
