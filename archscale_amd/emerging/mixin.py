"""Weight-decay flavours shared by the orthogonalized optimizers (emerging_optimizers/mixin.py:20-52)."""
from __future__ import annotations

from typing import Literal, Tuple

import torch

WeightDecayT = Literal["decoupled", "independent", "l2"]


def weight_decay_terms(method: str, lr: float, weight_decay: float) -> Tuple[float, float]:
    """(lr_wd, l2) such that the decay is  p <- p*(1 - lr_wd)  and/or  grad <- grad + l2*p.

    decoupled: p += -wd*lr*p;  independent: p += -wd*p;  l2: grad += wd*p.
    """
    if weight_decay == 0.0:
        return 0.0, 0.0
    if method == "decoupled":
        return weight_decay * lr, 0.0
    if method == "independent":
        return weight_decay, 0.0
    if method == "l2":
        return 0.0, weight_decay
    raise ValueError(f"Invalid weight decay method: {method}")


class WeightDecayMixin:
    """Eager in-place weight decay, used on the per-parameter (hook) path."""

    def _apply_weight_decay_inplace(self, p: torch.Tensor, grad: torch.Tensor, lr: float, weight_decay: float) -> None:
        lr_wd, l2 = weight_decay_terms(getattr(self, "weight_decay_method", "l2"), lr, weight_decay)
        if lr_wd != 0.0:
            p.add_(p, alpha=-lr_wd)
        if l2 != 0.0:
            grad.add_(p, alpha=l2)
