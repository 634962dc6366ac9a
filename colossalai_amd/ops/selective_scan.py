"""Selective scan of a ragged serving batch: a diagonal state-space recurrence
whose decay depends on the token, one state row per channel.

Per channel ``c`` and state place ``n``, token after token of a sequence:

    dt_c  = softplus(dt_raw_c + dt_bias_c)
    S[c, n] <- exp(dt_c * A[c, n]) * S[c, n] + dt_c * x_c * B_n,   A = -exp(A_log)
    y_c   = sum_n S[c, n] * C_n + D_c * x_c

and the result is ``y * silu(z)``. ``B`` and ``C`` belong to the token and are
shared by all channels. The state ``S`` [channels, places] of a sequence lives
in its state slot (float32), is taken as zero for a sequence that starts at
position 0, and is written back after the portion's last token, so a result
does not depend on how a prompt was cut. The step size, both exponentials, the
state and the read-out are float32.

On the GPU a step with a long portion runs in chunks of ``CHUNK`` tokens that
are scanned in parallel: once from a zero state for each chunk's end state and
summed steps, a short sequential pass that carries the state from chunk to
chunk (the recurrence is linear in the state and a chunk's decay is
``exp(A * sum of its steps)``), and once more from each chunk's true incoming
state for the output.
"""

import torch
import torch.nn.functional as F

from ._kernels import serving_state_kernels, use_serving_hip as use_hip
from .ragged import RaggedBatch

__all__ = ["selective_scan", "selective_scan_ref", "CHUNK", "CHUNKED_FROM"]

CHUNK = 64           # tokens per chunk of the two-pass form (the kernel's own constant)
CHUNKED_FROM = 256   # a step whose longest portion has at least this many tokens runs in chunks


def _chunk_tables(batch: RaggedBatch):
    """(chunks [K, 4] int32 = (sequence, first token, end token, 0), seq_chunks [B + 1]) on the device, one copy."""
    rows, ranges = [], [0]
    for b in range(batch.num_seqs):
        lo, hi = batch.cu_host[b], batch.cu_host[b + 1]
        for t in range(lo, hi, CHUNK):
            rows += [b, t, min(t + CHUNK, hi), 0]
        ranges.append(len(rows) // 4)
    buf = torch.tensor(rows + ranges, dtype=torch.int32).to(batch.cu.device)
    return buf[: len(rows)].view(-1, 4), buf[len(rows):]


def selective_scan_ref(x, dt_raw, A_log, B, C, D_skip, dt_bias, z, state, batch: RaggedBatch, out_dtype=None):
    xf, zf = x.float(), z.float()
    dt = F.softplus(dt_raw.float() + dt_bias.float(), threshold=1e30)      # [N, C], no clamp of large arguments
    A = -torch.exp(A_log.float())                                           # [C, S]
    Bf, Cf = B.float(), C.float()
    y = torch.empty_like(xf)
    for i in range(batch.num_seqs):
        lo, hi, slot = batch.cu_host[i], batch.cu_host[i + 1], batch.slots_host[i]
        S = state[slot].clone() if batch.start_host[i] > 0 else torch.zeros_like(state[slot])
        for t in range(lo, hi):
            S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * xf[t])[:, None] * Bf[t][None, :]
            y[t] = S @ Cf[t] + D_skip.float() * xf[t]
        state[slot] = S
    return (y * F.silu(zf)).to(out_dtype or z.dtype)


def selective_scan(x, dt_raw, A_log, B, C, D_skip, dt_bias, z, state, batch: RaggedBatch, out_dtype=None):
    """x [N, C] (float32 keeps the convolution's output unrounded), dt_raw [N, C], B and C [N, S] and z [N, C]
    (rows may be strided), A_log [C, S], D_skip and dt_bias [C] float32, state [slots, C, S] float32 (slot-strided
    allowed). Returns ``y * silu(z)`` [N, C] in ``out_dtype`` (default: z's)."""
    if use_hip(x):
        chunks = seq_chunks = None
        if batch.max_new >= CHUNKED_FROM:
            if getattr(batch, "_scan_chunks", None) is None:
                batch._scan_chunks = _chunk_tables(batch)     # once per step, shared by the step's layers
            chunks, seq_chunks = batch._scan_chunks
        return serving_state_kernels().selective_scan(x, dt_raw, A_log, B, C, D_skip, dt_bias, z, state, batch.cu,
                                                      batch.start, batch.slots, out_dtype or z.dtype, chunks, seq_chunks)
    return selective_scan_ref(x, dt_raw, A_log, B, C, D_skip, dt_bias, z, state, batch, out_dtype)
