"""Short causal depthwise convolution over a ragged serving batch.

``y[t, c] = act(bias[c] + sum_d taps[c, K-1-d] * x[t-d, c])`` for ``d = 0..K-1``
(the last tap is the current token's; the bias is optional), zeros
ahead of position 0. The last ``K-1`` inputs of a sequence live in ``tail``
(one ``[K-1, C]`` block per state slot, oldest first) so a portion that starts
mid-sequence sees the inputs of earlier steps.
"""

import torch
import torch.nn.functional as F

from ._kernels import serving_state_kernels as serving_kernels, use_serving_hip as use_hip
from .ragged import RaggedBatch

__all__ = ["short_conv", "short_conv_ref"]


def short_conv_ref(x, taps, tail, batch: RaggedBatch, silu: bool = True, out_dtype=None, bias=None):
    K = taps.shape[1]
    y = torch.empty_like(x, dtype=out_dtype or x.dtype)
    tf = taps.float()
    for i in range(batch.num_seqs):
        lo, hi, slot = batch.cu_host[i], batch.cu_host[i + 1], batch.slots_host[i]
        if K == 1:
            hist = x.new_zeros(0, x.shape[1], dtype=torch.float32)
        elif batch.start_host[i] > 0:
            hist = tail[slot].float()
        else:
            hist = torch.zeros_like(tail[slot], dtype=torch.float32)
        full = torch.cat([hist, x[lo:hi].float()], 0)  # [K-1+n, C]
        acc = torch.zeros(hi - lo, x.shape[1], device=x.device)
        for j in range(K):
            acc = acc + full[j : j + hi - lo] * tf[:, j]
        if bias is not None:
            acc = acc + bias.float()
        y[lo:hi] = (F.silu(acc) if silu else acc).to(y.dtype)
        if K > 1:
            tail[slot] = full[full.shape[0] - (K - 1):]
    return y


def short_conv(x, taps, tail, batch: RaggedBatch, silu: bool = True, out_dtype=None, bias=None):
    """x [N, C], taps [C, K], bias [C] or None, tail [slots, K-1, C] float32 (slot-strided allowed).
    The sum and the activation are float32; ``out_dtype`` (default: x's) is what
    the result is stored in — float32 keeps a recurrence's inputs unrounded."""
    if use_hip(x):
        return serving_kernels().short_conv(x, taps, tail, batch.cu, batch.start, batch.slots, batch.tok_seq, silu,
                                            out_dtype or x.dtype, bias)
    return short_conv_ref(x, taps, tail, batch, silu, out_dtype, bias)
