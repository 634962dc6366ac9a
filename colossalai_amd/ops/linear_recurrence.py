"""Matrix-state linear recurrences over a ragged serving batch.

Every head keeps a float32 matrix ``S [D, Dv]`` per state slot (rows = key /
query channels, columns = value channels) that is carried from step to step.
Three update rules are provided:

* ``gated_delta_rule`` — per-channel decay plus delta-rule write
  ``S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q``
  with ``g = exp(-exp(A_log_h) * softplus(dt + dt_bias))`` per key channel,
  ``beta = sigmoid(.)``, q and k scaled to unit length per head
  (``x / sqrt(sum x^2 + unit_eps)``) and q further by ``q_scale``.
* ``tied_gate_recurrence`` (HGRN2) — the forget gate also sets the write:
  ``S <- diag(f) S + (1 - f) v^T;  o = S^T q`` with
  ``f = lower + (1 - lower) sigmoid(f_logit + f_bias)`` and ``q = silu(.)``.

* ``ssd_recurrence`` (state-space duality) — one decay per head and token:
  ``S <- a S + dt B x^T;  y = S^T C + D_skip x`` with ``dt = softplus(dt_raw +
  dt_bias)``, ``a = exp(-exp(A_log_h) dt)``; ``B`` and ``C`` are shared by the
  heads of a group (head ``h`` reads group ``h // (H / G)``).

The read-out always includes the current token's write. Gates, decays and the
state are float32 whatever the activation dtype is.
"""

import torch
import torch.nn.functional as F

from ._kernels import serving_state_kernels as serving_kernels, use_serving_hip as use_hip
from .ragged import RaggedBatch

__all__ = ["gated_delta_rule", "gated_delta_rule_ref", "tied_gate_recurrence", "tied_gate_recurrence_ref",
           "ssd_recurrence", "ssd_recurrence_ref"]


def _scan_ref(batch, state, n_out, step):
    for i in range(batch.num_seqs):
        lo, hi, slot = batch.cu_host[i], batch.cu_host[i + 1], batch.slots_host[i]
        S = state[slot].clone() if batch.start_host[i] > 0 else torch.zeros_like(state[slot])
        for t in range(lo, hi):
            S = step(S, t)
        state[slot] = S


def gated_delta_rule_ref(q, k, v, beta_logit, dt, A_log, dt_bias, state, batch: RaggedBatch,
                         unit_eps: float = 1e-6, q_scale: float = 1.0):
    N, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    rep = H // G
    qf, kf = q.float(), k.float()
    qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + unit_eps) * q_scale
    kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + unit_eps)
    qf = qf.repeat_interleave(rep, 1)
    kf = kf.repeat_interleave(rep, 1)
    vf = v.float()
    beta = torch.sigmoid(beta_logit.float())
    g = torch.exp(-torch.exp(A_log.float())[None, :, None]
                  * F.softplus(dt.float().reshape(N, H, D) + dt_bias.float().reshape(H, D)))
    out = torch.empty(N, H, Dv, dtype=torch.float32, device=q.device)

    def step(S, t):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (vf[t] - torch.einsum("hdv,hd->hv", S, kf[t]))
        S = S + kf[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        return S

    _scan_ref(batch, state, out, step)
    return out


def gated_delta_rule(q, k, v, beta_logit, dt, A_log, dt_bias, state, batch: RaggedBatch,
                     unit_eps: float = 1e-6, q_scale: float = 1.0):
    """q, k [N, G, D]; v [N, H, Dv] (H a multiple of G; head h reads q/k head
    h // (H / G)); beta_logit [N, H]; dt [N, H * D]; A_log [H]; dt_bias [H * D];
    state [slots, H, D, Dv] float32. Returns o [N, H, Dv] float32."""
    if use_hip(q):
        return serving_kernels().gated_delta_rule(q, k, v, beta_logit, dt, A_log, dt_bias, state, batch.cu,
                                                  batch.start, batch.slots, unit_eps, q_scale)
    return gated_delta_rule_ref(q, k, v, beta_logit, dt, A_log, dt_bias, state, batch, unit_eps, q_scale)


def tied_gate_recurrence_ref(q, f_logit, v, f_bias, lower, state, batch: RaggedBatch):
    N, H, D = q.shape
    Dv = v.shape[2]
    qf = F.silu(q.float())
    low = lower.float().reshape(H, D)
    f = low + (1.0 - low) * torch.sigmoid(f_logit.float().reshape(N, H, D) + f_bias.float().reshape(H, D))
    vf = v.float()
    out = torch.empty(N, H, Dv, dtype=torch.float32, device=q.device)

    def step(S, t):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * vf[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        return S

    _scan_ref(batch, state, out, step)
    return out


def tied_gate_recurrence(q, f_logit, v, f_bias, lower, state, batch: RaggedBatch):
    """q, f_logit [N, H, D] (q before its silu), v [N, H, Dv], f_bias and lower
    [H * D], state [slots, H, D, Dv] float32. Returns o [N, H, Dv] float32."""
    if use_hip(q):
        return serving_kernels().tied_gate_recurrence(q, f_logit, v, f_bias, lower, state, batch.cu, batch.start,
                                                      batch.slots)
    return tied_gate_recurrence_ref(q, f_logit, v, f_bias, lower, state, batch)


def ssd_recurrence_ref(x, B, C, dt_raw, A_log, dt_bias, D_skip, state, batch: RaggedBatch):
    N, H, Dv = x.shape
    G = B.shape[1]
    rep = H // G
    xf = x.float()
    Bf = B.float().repeat_interleave(rep, 1)   # [N, H, D]
    Cf = C.float().repeat_interleave(rep, 1)
    dt = F.softplus(dt_raw.float() + dt_bias.float(), threshold=1e30)    # [N, H], no clamp of large arguments
    a = torch.exp(-torch.exp(A_log.float())[None, :] * dt)
    skip = D_skip.float()[:, None]
    out = torch.empty(N, H, Dv, dtype=torch.float32, device=x.device)

    def step(S, t):
        S = a[t][:, None, None] * S + (dt[t][:, None] * Bf[t])[:, :, None] * xf[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, Cf[t]) + skip * xf[t]
        return S

    _scan_ref(batch, state, out, step)
    return out


def ssd_recurrence(x, B, C, dt_raw, A_log, dt_bias, D_skip, state, batch: RaggedBatch):
    """x [N, H, Dv]; B, C [N, G, D] (H a multiple of G; rows may be strided); dt_raw [N, H]; A_log, dt_bias,
    D_skip [H]; state [slots, H, D, Dv] float32. Returns y [N, H, Dv] float32."""
    if use_hip(x):
        return serving_kernels().ssd_recurrence(x, B, C, dt_raw, A_log, dt_bias, D_skip, state, batch.cu,
                                                batch.start, batch.slots)
    return ssd_recurrence_ref(x, B, C, dt_raw, A_log, dt_bias, D_skip, state, batch)
