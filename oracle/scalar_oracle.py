"""CPU restatement of the reference's AdamW / hyperball-AdamW / Lion foreach updates
(lit_gpt/optim/scalar_opts.py), used to check the HIP multi-tensor kernels for the non-matrix groups.

TEST INFRASTRUCTURE ONLY, like the rest of ``oracle/``.  Pinned in tests/test_oracle.py by closed forms:
first-step AdamW is ``-lr * g / (|g| + eps)`` whatever the betas, Lion's update is ``-lr * sign``, the
hyperball variant preserves the Frobenius norm and moves along the Adam direction.
"""
from __future__ import annotations

from typing import List

import torch
from torch import Tensor


def _weight_decay_(X: List[Tensor], U: List[Tensor], lr: float, weight_decay: float, cautious_wd: bool) -> None:
    """Plain ``X *= 1 - lr*wd`` or the cautious variant that decays only where ``X*U >= 0``
    (scalar_opts.py:179-191 of the reference)."""
    if cautious_wd:
        keep = torch._foreach_mul(X, U)
        torch._foreach_sign_(keep)
        torch._foreach_add_(keep, 1)
        torch._foreach_clamp_max_(keep, 1)
        torch._foreach_mul_(keep, X)
        torch._foreach_mul_(keep, lr * weight_decay)
        torch._foreach_sub_(X, keep)
    else:
        torch._foreach_mul_(X, 1 - lr * weight_decay)


def _adam_moments_(G: List[Tensor], M: List[Tensor], V: List[Tensor], beta1: float, beta2: float) -> None:
    g_m = [g.to(dtype=m.dtype) for g, m in zip(G, M)]
    torch._foreach_lerp_(M, g_m, 1 - beta1)
    g_sq = [(g * g).to(dtype=v.dtype) for g, v in zip(g_m, V)]
    torch._foreach_lerp_(V, g_sq, 1 - beta2)


def _adam_direction(M: List[Tensor], V: List[Tensor], beta2: float, step: int, epsilon: float) -> List[Tensor]:
    """M / (sqrt(V / bias2) + eps)."""
    bias2_sqrt = (1 - beta2 ** step) ** 0.5
    denom = torch._foreach_sqrt(V)
    torch._foreach_div_(denom, bias2_sqrt)
    torch._foreach_add_(denom, epsilon)
    return torch._foreach_div(M, denom)


def adamw_update_foreach(X, G, M, V, lr, beta1, beta2, weight_decay, step, epsilon, cautious_wd=False) -> None:
    """AdamW with bias correction (scalar_opts.py:118-198 of the reference)."""
    if not X:
        return
    _adam_moments_(G, M, V, beta1, beta2)
    direction = _adam_direction(M, V, beta2, step, epsilon)
    _weight_decay_(X, direction, lr, weight_decay, cautious_wd)
    torch._foreach_mul_(direction, lr / (1 - beta1 ** step))
    torch._foreach_sub_(X, direction)


def hyperball_adamw_update_foreach(X, G, M, V, lr, beta1, beta2, weight_decay, step, epsilon,
                                   cautious_wd=False) -> None:
    """AdamW direction applied on the hypersphere: step of relative size ``lr`` along the bias-corrected
    direction, then renormalisation to the tensor's previous Frobenius norm
    (scalar_opts.py:254-377, 396-437 of the reference; the all-reduces drop out on one GPU)."""
    if not X:
        return
    _adam_moments_(G, M, V, beta1, beta2)
    U = _adam_direction(M, V, beta2, step, epsilon)
    torch._foreach_div_(U, 1 - beta1 ** step)
    _weight_decay_(X, U, lr, weight_decay, cautious_wd)
    x_norms = torch._foreach_norm(X)
    u_norms = torch._foreach_norm(U)
    scales = [xn / un.clamp_min(epsilon) for xn, un in zip(x_norms, u_norms)]
    torch._foreach_mul_(U, scales)
    torch._foreach_mul_(U, lr)
    torch._foreach_sub_(X, U)
    new_norms = torch._foreach_norm(X)
    torch._foreach_mul_(X, [xn / nn.clamp_min(epsilon) for xn, nn in zip(x_norms, new_norms)])


def lion_update_foreach(X, G, M, lr, beta1, beta2, weight_decay, cautious_wd=False) -> None:
    """Lion: sign of the beta1-interpolated momentum, then momentum EMA with beta2
    (scalar_opts.py:201-251 of the reference)."""
    if not X:
        return
    g_m = [g.to(dtype=m.dtype) for g, m in zip(G, M)]
    U = torch._foreach_lerp(M, g_m, 1 - beta1)
    torch._foreach_sign_(U)
    torch._foreach_lerp_(M, g_m, 1 - beta2)
    _weight_decay_(X, U, lr, weight_decay, cautious_wd)
    torch._foreach_mul_(U, lr)
    torch._foreach_sub_(X, U)
