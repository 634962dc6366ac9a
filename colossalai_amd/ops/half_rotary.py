"""Rotary positions in the *rotate-half* layout, fused with a weightless
per-head RMS norm, for the queries and keys of a ragged serving batch.

Channel ``i`` of a head is paired with channel ``i + dims / 2``, ``i`` from 0 to
``dims / 2 - 1``; the pair ``(u, v)`` of a token at position ``p`` becomes
``(u cos a - v sin a, v cos a + u sin a)`` with ``a = p * f_i`` and
``f_i = base^(-2 i / dims)`` (``ops.pair_rotary.pair_frequencies``). Only the
first ``dims`` channels turn. Afterwards (``eps`` given) the head's vector is
divided by its root mean square over all its channels,
``x / sqrt(mean(x^2) + eps)``. Either step can be left out. Positions, angles,
sine, cosine and the statistics are float32.
"""

from typing import Optional

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip

__all__ = ["rotate_halves_unit_norm", "rotate_halves_unit_norm_ref"]


def rotate_halves_unit_norm_ref(x, positions, freqs, eps, out_dtype=None):
    y = x.float().clone()
    if freqs is not None and freqs.numel():
        half = freqs.numel()
        ang = positions.to(torch.float32)[:, None] * freqs.to(torch.float32)[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        u, v = y[..., :half].clone(), y[..., half : 2 * half].clone()
        y[..., :half] = u * c - v * s
        y[..., half : 2 * half] = v * c + u * s
    if eps is not None:
        y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return y.to(out_dtype or x.dtype)


def rotate_halves_unit_norm(x, positions, freqs: Optional[torch.Tensor], eps: Optional[float], out_dtype=None):
    """x [N, H, D] (any row stride, heads D apart), positions [N] int32, freqs [dims / 2] float32 or None (no
    rotation), eps or None (no norm). Returns a contiguous [N, H, D] tensor in ``out_dtype`` (default: x's)."""
    assert x.dim() == 3 and (freqs is None or 2 * freqs.numel() <= x.shape[-1])
    if use_hip(x):
        return serving_kernels().rotate_halves_unit_norm(x, positions, freqs, -1.0 if eps is None else float(eps),
                                                         out_dtype or x.dtype)
    return rotate_halves_unit_norm_ref(x, positions, freqs, eps, out_dtype)
