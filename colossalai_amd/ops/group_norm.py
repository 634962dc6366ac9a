"""Grouped RMS normalisation and per-head output normalisation with a gate.

``grouped_rms_norm`` splits the feature axis into ``groups`` equal consecutive
parts, scales each part by its own ``rsqrt(mean(part^2) + eps)`` and applies an
element-wise weight; with ``residual`` it adds the result to a float32 residual
stream in place (norm on the sublayer's *output*). ``groups=1`` is plain RMS
norm. ``head_rms_norm_gate`` normalises every head vector of a ``[N, H, D]``
tensor with one shared ``[D]`` weight and optionally multiplies by
``sigmoid(gate)``. ``add_rms_norm`` serves pre-norm layers: it adds one or two
sublayer outputs to the float32 residual stream in place and hands back the
RMS-normed stream for the next layer in one pass. ``gated_grouped_rms_norm``
multiplies a row by ``silu(gate)`` *before* its grouped RMS norm (the output norm
of a state-space mixer). ``layer_norm`` is the centred norm with a weight and no
bias, ``(x - mean) / sqrt(var + eps) * w``; ``add_layer_norm`` serves layers that
norm a sublayer's output on its way into the residual stream and norm the
stream again for the next sublayer: ``residual += mult * layer_norm(y) * w_out``
in place and, when ``w_next`` is given, ``layer_norm(residual) * w_next`` in one
launch. All statistics are float32.
"""

from typing import Optional

import torch

from ._kernels import serving_kernels, use_serving_hip as use_hip

__all__ = ["grouped_rms_norm", "grouped_rms_norm_ref", "head_rms_norm_gate", "head_rms_norm_gate_ref",
           "merge_rms_norm", "merge_rms_norm_ref", "add_rms_norm", "add_rms_norm_ref",
           "gated_grouped_rms_norm", "gated_grouped_rms_norm_ref", "layer_norm", "layer_norm_ref",
           "add_layer_norm", "add_layer_norm_ref", "add_scaled_unit_norm", "add_scaled_unit_norm_ref"]


def grouped_rms_norm_ref(x, weight, groups: int, eps: float, residual=None, out_dtype=None):
    shp = x.shape
    xf = x.float().reshape(*shp[:-1], groups, shp[-1] // groups)
    y = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).reshape(shp) * weight.float()
    if residual is not None:
        residual.add_(y)
        return residual
    return y.to(out_dtype or x.dtype)


def grouped_rms_norm(x, weight, groups: int, eps: float, residual: Optional[torch.Tensor] = None, out_dtype=None):
    assert x.shape[-1] % groups == 0, "feature axis must split evenly into the norm groups"
    if use_hip(x):
        assert residual is None or residual.dtype == torch.float32
        if residual is not None or x.stride(-1) != 1:
            x = x.contiguous()  # without a residual the kernel takes strided rows
        return serving_kernels().grouped_rms_norm(x, weight, groups, eps, residual, out_dtype or x.dtype)
    return grouped_rms_norm_ref(x, weight, groups, eps, residual, out_dtype)


def head_rms_norm_gate_ref(x, weight, eps: float, gate=None, out_dtype=None):
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    if gate is not None:
        y = y * torch.sigmoid(gate.float().reshape(y.shape))
    return y.to(out_dtype or x.dtype)


def head_rms_norm_gate(x, weight, eps: float, gate=None, out_dtype=None):
    """x [N, H, D] (row-strided allowed), weight [D], gate logits [N, H * D] or None."""
    if use_hip(x):
        return serving_kernels().head_rms_norm_gate(x, weight, eps, gate, out_dtype or x.dtype)
    return head_rms_norm_gate_ref(x, weight, eps, gate, out_dtype)


def merge_rms_norm_ref(a, wa, b, wb, eps: float, out_w, groups: int, residual):
    def unit(t, w):
        tf = t.float()
        return tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps) * w.float()

    m = 0.5 * (unit(a, wa) + unit(b, wb))
    return grouped_rms_norm_ref(m, out_w, groups, eps, residual)


def merge_rms_norm(a, wa, b, wb, eps: float, out_w, groups: int, residual):
    """Two branch outputs [N, W], each RMS-normed over the full width with its
    own weight, averaged, then grouped-normed with ``out_w`` and added to the
    float32 ``residual`` in place — one pass over the row."""
    if use_hip(a):
        return serving_kernels().merge_rms_norm(a.contiguous(), wa, b.contiguous(), wb, eps, out_w, groups, residual)
    return merge_rms_norm_ref(a, wa, b, wb, eps, out_w, groups, residual)


def add_rms_norm_ref(residual, a, b, weight, eps: float, out_dtype=None):
    residual.add_(a.float() if b is None else a.float() + b.float())
    if weight is None:
        return None
    return grouped_rms_norm_ref(residual, weight, 1, eps, None, out_dtype or a.dtype)


def add_rms_norm(residual, a, b, weight, eps: float, out_dtype=None):
    """``residual += a (+ b)`` in place (float32 [N, W]; ``a``/``b`` sublayer
    outputs of any activation type, ``b`` may be None), then, when ``weight`` is
    given, returns ``rms_norm(residual) * weight`` in ``out_dtype`` — the input
    of the next pre-norm layer. With ``weight=None`` only the sum is formed."""
    if use_hip(residual):
        assert residual.dtype == torch.float32
        return serving_kernels().add_rms_norm(residual, a.contiguous(), None if b is None else b.contiguous(),
                                              weight, eps, out_dtype or a.dtype)
    return add_rms_norm_ref(residual, a, b, weight, eps, out_dtype)


def gated_grouped_rms_norm_ref(x, gate, weight, groups: int, eps: float, out_dtype=None):
    g = gate.float()
    return grouped_rms_norm_ref(x.float() * (g * torch.sigmoid(g)), weight, groups, eps, None, out_dtype or gate.dtype)


def gated_grouped_rms_norm(x, gate, weight, groups: int, eps: float, out_dtype=None):
    """x [N, W] (float32 or an activation type), gate [N, W] logits (rows may be strided): the row
    ``x * silu(gate)`` is RMS-normed in ``groups`` equal parts and weighted. The gate comes before the norm."""
    assert x.shape[-1] % groups == 0 and gate.shape == x.shape
    if use_hip(x):
        return serving_kernels().gated_grouped_rms_norm(x, gate, weight, groups, eps, out_dtype or gate.dtype)
    return gated_grouped_rms_norm_ref(x, gate, weight, groups, eps, out_dtype)


def layer_norm_ref(x, weight, eps: float, out_dtype=None):
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    d = xf - mu
    return (d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(out_dtype or x.dtype)


def layer_norm(x, weight, eps: float, out_dtype=None):
    """Centred norm of the rows of x [N, W] with a weight and no bias; the variance is the mean of the squared
    deviations (two passes over the row, float32)."""
    if use_hip(x):
        return serving_kernels().add_layer_norm(None, x.contiguous(), None, 1.0, weight, eps, out_dtype or x.dtype)
    return layer_norm_ref(x, weight, eps, out_dtype)


def add_layer_norm_ref(residual, y, w_out, mult: float, w_next, eps: float, out_dtype=None):
    residual.add_(layer_norm_ref(y, w_out, eps, torch.float32), alpha=mult)
    if w_next is None:
        return None
    return layer_norm_ref(residual, w_next, eps, out_dtype or y.dtype)


def add_layer_norm(residual, y, w_out, mult: float, w_next, eps: float, out_dtype=None):
    """``residual += mult * layer_norm(y) * w_out`` in place (float32 [N, W]; ``y`` a sublayer's output of any
    activation type), then, when ``w_next`` is given, returns ``layer_norm(residual) * w_next`` in ``out_dtype``:
    the input of the next sublayer. With ``w_next=None`` only the sum is formed."""
    if use_hip(residual):
        assert residual.dtype == torch.float32
        return serving_kernels().add_layer_norm(residual, y.contiguous(), w_out, float(mult), w_next, eps,
                                                out_dtype or y.dtype)
    return add_layer_norm_ref(residual, y, w_out, mult, w_next, eps, out_dtype)


def add_scaled_unit_norm_ref(residual, a, b, scale_a: float, scale_b: float, gain: float, eps: float, out_dtype=None):
    y = a.float() * scale_a if b is None else a.float() * scale_a + b.float() * scale_b
    residual.add_(y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * gain)
    return residual.to(out_dtype) if out_dtype is not None else None


def add_scaled_unit_norm(residual, a, b, scale_a: float, scale_b: float, gain: float, eps: float, out_dtype=None):
    """Norm on a sublayer's *output*, with one number as its weight: ``y = scale_a * a (+ scale_b * b)``,
    ``residual += gain * y / sqrt(mean(y^2) + eps)`` in place (float32 [N, W]; ``a``/``b`` sublayer outputs of any
    activation type). With ``out_dtype`` the updated rows are also handed back in that type — the next sublayer's
    input, when sublayers read the stream itself — in the same pass."""
    if use_hip(residual):
        assert residual.dtype == torch.float32 and residual.is_contiguous()
        return serving_kernels().add_scaled_unit_norm(residual, a.contiguous(), None if b is None else b.contiguous(),
                                                      float(scale_a), float(scale_b), float(gain), float(eps), out_dtype)
    return add_scaled_unit_norm_ref(residual, a, b, scale_a, scale_b, gain, eps, out_dtype)

