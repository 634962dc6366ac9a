"""Rotary positions on neighbouring pairs of a ragged serving batch.

Dimension ``2i`` is paired with ``2i + 1`` (the interleaved layout), ``i`` from
0 to ``dims / 2 - 1``; the pair ``(u, v)`` of a token at position ``p`` becomes
``(u cos a - v sin a, v cos a + u sin a)`` with ``a = p * f_i`` and
``f_i = base^(-2 i / dims)``. Only the first ``dims`` channels of a vector turn;
the rest pass unchanged. Positions, angles, sine and cosine are float32 (the
frequencies are formed in float64 and rounded once).
"""

from typing import Optional

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip

__all__ = ["pair_frequencies", "rotate_pairs", "rotate_pairs_ref"]


def pair_frequencies(base: float, dims: int, device=None) -> torch.Tensor:
    """f_i = base^(-2 i / dims), i = 0 .. dims / 2 - 1, float32."""
    assert dims % 2 == 0, "pairs need an even number of rotated channels"
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(torch.float32).to(device)


def rotate_pairs_ref(x, positions, freqs, out: Optional[torch.Tensor] = None):
    dims = 2 * freqs.numel()
    ang = positions.to(torch.float32)[:, None] * freqs.to(torch.float32)[None, :]     # [N, dims / 2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    xf = x.float()
    u, v = xf[..., 0:dims:2], xf[..., 1:dims:2]
    y = xf.clone()
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    if out is None:
        return y.to(x.dtype)
    out.copy_(y.to(out.dtype))
    return out


def rotate_pairs(x, positions, freqs, out: Optional[torch.Tensor] = None):
    """x [N, H, R] (any row and head strides, unit channel stride), positions [N] int32, freqs [dims / 2] float32
    with ``dims <= R``. Writes to ``out`` (same shape, its own strides; may be ``x`` itself) or a new tensor."""
    assert x.dim() == 3 and 2 * freqs.numel() <= x.shape[-1]
    if use_hip(x):
        if out is None:
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        serving_kernels().rotate_pairs(x, positions, freqs, out)
        return out
    return rotate_pairs_ref(x, positions, freqs, out)
