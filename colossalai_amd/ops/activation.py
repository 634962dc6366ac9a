"""Small element-wise activations of the serving path.

``relu_squared(x) = max(x, 0)^2`` (feed-forward activation),
``silu_mul([g | u]) = g * sigmoid(g) * u`` and ``gelu_tanh_mul([g | u]) =
gelu_tanh(g) * u`` on a packed ``[N, 2F]`` tensor (gated feed-forwards; the tanh
form of GELU is ``0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))``) and ``softcap(x, c) = c * tanh(x / c)`` (bounded logits, float32).
"""

import torch

from ._kernels import serving_kernels, use_serving_hip

__all__ = ["relu_squared", "silu_mul", "gelu_tanh_mul", "softcap"]


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    if use_serving_hip(x) and not torch.is_grad_enabled():
        return serving_kernels().relu_squared(x.contiguous())
    return torch.relu(x).square()


def silu_mul(packed: torch.Tensor) -> torch.Tensor:
    """packed [N, 2F] = [gate | up] (rows may be strided) -> [N, F]; the product
    is formed in float32 and rounded once."""
    F_ = packed.shape[-1] // 2
    if use_serving_hip(packed) and not torch.is_grad_enabled():
        return serving_kernels().silu_mul(packed)
    g, u = packed[..., :F_].float(), packed[..., F_:].float()
    return (g * torch.sigmoid(g) * u).to(packed.dtype)


def gelu_tanh_mul(packed: torch.Tensor) -> torch.Tensor:
    """packed [N, 2F] = [gate | up] (rows may be strided) -> [N, F] = gelu_tanh(gate) * up,
    formed in float32 and rounded once."""
    F_ = packed.shape[-1] // 2
    if use_serving_hip(packed) and not torch.is_grad_enabled():
        return serving_kernels().gelu_tanh_mul(packed)
    g, u = packed[..., :F_].float(), packed[..., F_:].float()
    inner = 0.7978845608028654 * (g + 0.044715 * g * g * g)
    return (0.5 * g * (1.0 + torch.tanh(inner)) * u).to(packed.dtype)


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    if use_serving_hip(x) and not torch.is_grad_enabled() and x.dtype == torch.float32:
        return serving_kernels().softcap(x.contiguous(), cap)
    return cap * torch.tanh(x / cap)
