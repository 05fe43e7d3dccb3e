"""Small element-wise activations of the serving path.

``relu_squared(x) = max(x, 0)^2`` (feed-forward activation) and
``softcap(x, c) = c * tanh(x / c)`` (bounded logits, float32).
"""

import torch

from ._kernels import serving_kernels, use_serving_hip

__all__ = ["relu_squared", "softcap"]


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    if use_serving_hip(x) and not torch.is_grad_enabled():
        return serving_kernels().relu_squared(x.contiguous())
    return torch.relu(x).square()


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    if use_serving_hip(x) and not torch.is_grad_enabled() and x.dtype == torch.float32:
        return serving_kernels().softcap(x.contiguous(), cap)
    return cap * torch.tanh(x / cap)
