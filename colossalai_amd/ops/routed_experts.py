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
experts and forms ``base + sum_j weight_j * y_j`` in float32. The activation is
``relu_squared`` or ``silu_gated`` (``up_e`` then stacks a gate and an up matrix,
``[E, 2F, W]``, and the hidden row is ``silu(gate h) * (up h)``). With
``identity=True`` an id at or above the number of expert matrices names an
*identity expert*, whose output is its input: such a pair adds ``weight * h``. On the GPU nothing
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
from .activation import relu_squared, silu_mul

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


ACTIVATIONS = ("relu_squared", "silu_gated")


def _act(x, activation: str):
    if activation == "relu_squared":
        return relu_squared(x)
    if activation == "silu_gated":
        return silu_mul(x)
    raise ValueError(f"unknown expert activation {activation!r}")


def routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base=None, activation: str = "relu_squared",
                          base_gate=None, identity: bool = False):
    N, top = ids.shape
    out = torch.zeros(N, w_down.shape[1], dtype=torch.float32, device=h.device) if base is None else base.float().clone()
    if base is not None and base_gate is not None:
        out = out * torch.sigmoid(base_gate.float().reshape(N, 1))
    if identity:
        out = out + (weights * (ids >= w_up.shape[0])).sum(-1, keepdim=True) * h.float()
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


def _grouped_expert_ffn(h, w_up, w_down, ids, weights, base, base_gate=None, activation="relu_squared", sorted_as=None):
    """One grouped matrix-core launch per product; the up product gathers the tokens' rows itself and squares the
    rectified accumulator (a gated activation runs on the packed product instead). Steps of up to 8192 pairs are
    sorted by one kernel, larger ones by library sorts. ``sorted_as`` = number of ids the sort tells apart when
    identity experts follow the real ones: their pairs sort behind every expert's rows, no product touches them and
    the combine step adds ``weight * h`` for them."""
    N, top = ids.shape
    K = serving_kernels()
    E = w_up.shape[0]
    n_ids = sorted_as or E
    if ids.numel() <= SORT_KERNEL_MAX_PAIRS:
        offsets, src, inv = K.expert_sort(ids.contiguous(), n_ids)
    else:
        order, inv, offsets = _sort_pairs(ids, n_ids)
        src, inv = (order // top).int(), inv.int().view(N, top)
    offsets = offsets[: E + 1]
    if activation == "relu_squared":
        hidden = K.expert_grouped_gemm(h, src, w_up, offsets, ids.numel(), True)
    else:
        hidden = _act(K.expert_grouped_gemm(h, src, w_up, offsets, ids.numel(), False), activation)
    y = K.expert_grouped_gemm(hidden, None, w_down, offsets, ids.numel(), False)
    if sorted_as:
        return K.expert_combine(y, inv, weights, base, base_gate, ids, E, h)
    return K.expert_combine(y, inv, weights, base, base_gate, None, 0, None)


def _sorted_expert_ffn(h, w_up, w_down, ids, weights, base, activation, base_gate=None, sorted_as=None):
    """Pairs sorted by expert, one up and one down library product per expert that got rows (their row counts come
    to the host), then every token gathers its ``top`` results in slot order."""
    N, top = ids.shape
    order, inv, offsets = _sort_pairs(ids, sorted_as or w_up.shape[0])
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
    if sorted_as:
        return serving_kernels().expert_combine(y, inv.int().view(N, top), weights, base, base_gate, ids, w_up.shape[0], h)
    return serving_kernels().expert_combine(y, inv.int().view(N, top), weights, base, base_gate, None, 0, None)


def _grouped_fits(h, w_up, w_down) -> bool:
    return (h.dtype == torch.bfloat16 and w_up.shape[2] % 32 == 0 and w_up.shape[1] % 32 == 0 and w_down.shape[2] % 32 == 0
            and w_up.shape[0] <= 1024 and w_up.is_contiguous() and w_down.is_contiguous())


def routed_expert_ffn(h, w_up, w_down, ids, weights, base: Optional[torch.Tensor] = None,
                      activation: str = "relu_squared", base_gate: Optional[torch.Tensor] = None,
                      identity: bool = False, num_ids: Optional[int] = None):
    """h [N, W]; w_up [E, F, W] (``silu_gated``: [E, 2F, W], gate rows first); w_down [E, W, F]; ids [N, top]
    int32; weights [N, top] float32; ``base`` [N, W] (any activation type) is added, e.g. a shared expert's output,
    multiplied by ``sigmoid(base_gate)`` when ``base_gate`` ([N] float32 logits, any stride) is given. With
    ``identity`` the ids from E up to ``num_ids`` (exclusive) are identity experts. Returns float32 [N, W]."""
    if not use_hip(h):
        return routed_expert_ffn_ref(h, w_up, w_down, ids, weights, base, activation, base_gate, identity)
    assert base_gate is None or (base is not None and base_gate.dtype == torch.float32 and base_gate.numel() == h.shape[0])
    if activation not in ACTIVATIONS:
        raise ValueError(f"unknown expert activation {activation!r}")
    assert not identity or (num_ids is not None and num_ids >= w_up.shape[0]), "identity experts need the id count"
    h = h.contiguous()
    gated = activation == "silu_gated"
    sorted_as = num_ids if identity else None
    if ids.numel() <= GEMV_MAX_PAIRS:
        return serving_kernels().expert_ffn_gemv(h, w_up, w_down, ids, weights, base, base_gate, gated, identity)
    if _grouped_fits(h, w_up, w_down):
        return _grouped_expert_ffn(h, w_up, w_down, ids, weights, base, base_gate, activation, sorted_as)
    if ids.numel() <= GEMV_FALLBACK_PAIRS:
        return serving_kernels().expert_ffn_gemv(h, w_up, w_down, ids, weights, base, base_gate, gated, identity)
    return _sorted_expert_ffn(h, w_up, w_down, ids, weights, base, activation, base_gate, sorted_as)
