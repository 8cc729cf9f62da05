"""Matrix sign by Newton-Schulz with the polar-express coefficients
(emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:37-74, 142-149), on the HIP path."""
from __future__ import annotations

from typing import List, Tuple

import torch

from ..optim import newton_schulz_hip as ns

#: spectral_ball_utils.py:56-65 of the reference; iterations beyond the table repeat the last row
MSIGN_COEFFICIENTS: Tuple[Tuple[float, float, float], ...] = (
    (8.2051, -22.9019, 16.4607),
    (4.0664, -2.8612, 0.5184),
    (3.9096, -2.8234, 0.5250),
    (3.2856, -2.4153, 0.4853),
    (2.2779, -1.6198, 0.3985),
    (1.8726, -1.2307, 0.3585),
    (1.8564, -1.2132, 0.3568),
    (1.8750, -1.2500, 0.3750),
)


def msign_schedule(steps: int) -> List[Tuple[float, float, float]]:
    return [MSIGN_COEFFICIENTS[min(i, len(MSIGN_COEFFICIENTS) - 1)] for i in range(steps)]


@torch.no_grad()
def msign(G: torch.Tensor, steps: int) -> torch.Tensor:
    """fp32 in, bf16 out: normalise in fp32 with ``max(|G|, 1e-7)``, round to bf16, iterate.
    The steep first row of the table needs B = bA + cA^2 as a bf16 hi+lo pair to stay within 1e-2 of fp32."""
    if G.ndim < 2:
        raise ValueError("Input tensor must have at least 2 dimensions.")
    if G.dtype != torch.float32:
        raise ValueError("Input tensor G must be in float32")
    return ns.newton_schulz(G, msign_schedule(steps), 1e-7, eps_mode="clamp", prec="bsplit", cast_input_first=False)
