"""Named-coefficient Newton-Schulz (emerging_optimizers/orthogonalized_optimizers/muon_utils.py:26-164)."""
from __future__ import annotations

import torch

from ..optim import newton_schulz_hip as ns

__all__ = ["newton_schulz", "newton_schulz_step_tsyrk"]

_COEFFICIENT_SETS = {
    "simple": [(3.4445, -4.7750, 2.0315)],
    "quintic": [
        (4.0848, -6.8946, 2.9270),
        (3.9505, -6.3029, 2.6377),
        (3.7418, -5.5913, 2.3037),
        (2.8769, -3.1427, 1.2046),
        (2.8366, -3.0525, 1.2012),
    ],
    "polar_express": [
        (7.2086, -15.5131, 9.0178),
        (3.9623, -2.5813, 0.4542),
        (3.9466, -2.5765, 0.4544),
        (3.8991, -2.5671, 0.4566),
        (3.7186, -2.5308, 0.4653),
        (3.1390, -2.3073, 0.4733),
        (2.1715, -1.5246, 0.3885),
        (1.8648, -1.2224, 0.3577),
    ],
    "aol": [
        (4.0098, -7.0585, 2.4635),
        (3.4585, -5.5479, 2.5959),
        (2.7573, -3.2939, 1.4254),
        (2.7215, -3.0494, 1.3169),
    ],
}


def newton_schulz(x: torch.Tensor, steps: int, coefficient_type: str = "polar_express",
                  custom_coefficient_sets=None, eps: float = 1e-7, transpose=None, tp_group=None,
                  use_syrk: bool = False) -> torch.Tensor:
    """fp32 in, fp32 out; the set is cycled ``i % len(set)`` and ``steps`` must be a multiple of its length.
    ``use_syrk`` is accepted and ignored (the HIP path always computes only the upper triangle).  ``transpose`` is
    accepted and has no effect: the iteration acts on the singular values only, so iterating on the matrix or on its
    transpose gives the same result, and the library always iterates with the short side first.  Tensor-parallel
    groups are not supported here."""
    if x.ndim < 2:
        raise ValueError("Input tensor x must have at least 2 dimensions since Muon is not for 1d parameters.")
    if x.dtype != torch.float32:
        raise ValueError(f"Input tensor x must be in float32, got {x.dtype}")
    if tp_group is not None:
        raise NotImplementedError("this build runs Newton-Schulz on one GPU; tp_group must be None")
    if coefficient_type in _COEFFICIENT_SETS:
        sets = _COEFFICIENT_SETS[coefficient_type]
    elif coefficient_type == "custom":
        if custom_coefficient_sets is None:
            raise ValueError("custom_coefficient_sets must be provided when coefficient_type is 'custom'.")
        sets = custom_coefficient_sets
    else:
        raise ValueError(f"Invalid coefficient type: {coefficient_type}")
    if steps % len(sets) != 0:
        raise ValueError(f"steps ({steps}) must be multiple of len(coefficient_sets) ({len(sets)}).")
    rows = [tuple(sets[i % len(sets)]) for i in range(steps)]
    out = ns.newton_schulz(x, rows, eps, eps_mode="clamp", prec=ns.ACCURATE_PREC, cast_input_first=False)
    return out.to(torch.float32)


def newton_schulz_step_tsyrk(X: torch.Tensor, a: float, b: float, c: float, tp_group=None) -> torch.Tensor:
    """One iteration ``aX + (bA + cA^2)X, A = XX^T`` on a bf16 matrix as it is, no normalisation
    (emerging_optimizers/orthogonalized_optimizers/muon_utils.py:262-287). Returns a new bf16 tensor."""
    if X.dtype != torch.bfloat16:
        raise ValueError(f"X must be bfloat16, got {X.dtype}")
    if X.ndim != 2:
        raise ValueError("X must be a 2-D matrix")
    if tp_group is not None:
        raise NotImplementedError("this build runs Newton-Schulz on one GPU; tp_group must be None")
    # one iteration in bf16 storage: one rounding of A, of B and of the result, the rounding points of the reference's
    # own kernels (measured against fp64 on inputs with singular values below 1.2: 2.6e-3)
    return ns.newton_schulz(X, [(float(a), float(b), float(c))], 0.0, prec="bf16", normalize=False)
