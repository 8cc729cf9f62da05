"""Muon of the orthogonalized-optimizer family on MI355X
(counterpart of emerging_optimizers/orthogonalized_optimizers/muon.py:64-148)."""
from __future__ import annotations

import torch
from torch.optim.optimizer import ParamsT

from ..optim import newton_schulz_hip as ns
from .mixin import WeightDecayT
from .orthogonalized_optimizer import OrthogonalizedOptimizer
from .spectral_ball_utils import msign, msign_schedule

__all__ = ["Muon", "get_muon_scale_factor"]


def get_muon_scale_factor(size_out: int, size_in: int, mode: str = "spectral") -> float:
    """Scale of the orthogonalised update (emerging_optimizers/.../muon.py:122-148):
    shape_scaling max(1, out/in)^0.5; align_adamw_rms 0.2*max(out, in)^0.5; spectral_mup (out/in)^0.5."""
    if mode == "shape_scaling":
        return max(1, size_out / size_in) ** 0.5
    if mode == "align_adamw_rms":
        return 0.2 * max(size_out, size_in) ** 0.5
    if mode == "spectral_mup":
        return (size_out / size_in) ** 0.5
    raise ValueError(f"Invalid mode for Muon update scale factor: {mode}")


class Muon(OrthogonalizedOptimizer):
    """MomentUm Orthogonalized by Newton-schulz: update = msign(momentum) * scale * extra_scale_factor.

    Same signature as the reference.  ``coefficient_type`` and ``use_syrk`` are accepted for compatibility:
    as in the reference the matrix sign always uses the polar-express table of ``msign``, and the HIP path
    always computes symmetric products from their upper triangle.
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float = 3e-4,
        momentum_beta: float = 0.95,
        weight_decay: float = 0.01,
        *,
        use_nesterov: bool = False,
        weight_decay_method: WeightDecayT = "decoupled",
        fp32_matmul_prec: str = "medium",
        coefficient_type: str = "quintic",
        num_ns_steps: int = 5,
        scale_mode: str = "align_adamw_rms",
        extra_scale_factor: float = 1.0,
        use_syrk: bool = False,
    ) -> None:
        if num_ns_steps < 1:
            raise ValueError(f"num_ns_steps must be at least 1, got {num_ns_steps}")
        get_muon_scale_factor(1, 1, scale_mode)  # validate the mode early
        self._num_ns_steps = num_ns_steps
        self._scale_mode = scale_mode
        self._extra_scale_factor = extra_scale_factor

        def scaled_orthogonalize_fn(grad: torch.Tensor) -> torch.Tensor:
            orth = msign(grad, steps=num_ns_steps)
            return orth * get_muon_scale_factor(grad.size(-2), grad.size(-1), mode=scale_mode) * extra_scale_factor

        super().__init__(
            params, lr, momentum_beta, use_nesterov=use_nesterov, weight_decay=weight_decay,
            weight_decay_method=weight_decay_method, fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=scaled_orthogonalize_fn,
        )
        self._builtin_fn = scaled_orthogonalize_fn

    def _batched_recipe(self, group: dict):
        if self.scaled_orthogonalize_fn is not self._builtin_fn:
            return None  # someone replaced the hook: honour it per parameter
        mode, extra = self._scale_mode, self._extra_scale_factor
        return (msign_schedule(self._num_ns_steps), 1e-7, "clamp", ns.ACCURATE_PREC,
                lambda rows, cols: get_muon_scale_factor(rows, cols, mode=mode) * extra)
