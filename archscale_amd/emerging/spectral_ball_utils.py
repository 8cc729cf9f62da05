"""Matrix sign by Newton-Schulz with the polar-express coefficients, spectral norm by power iteration, retraction,
radius and scale of the spectral-ball optimizers
(emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:37-74, 142-212, 432-466), on the HIP path."""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

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
    return ns.newton_schulz(G, msign_schedule(steps), 1e-7, eps_mode="clamp", prec=ns.ACCURATE_PREC, cast_input_first=False)


# ---------------------------------------------------------------------------
# spectral norm, retraction, radius and scale of the spectral-ball family
# ---------------------------------------------------------------------------
def spectral_norm(w: torch.Tensor, steps: int = 50) -> torch.Tensor:
    """Top singular value of every matrix of ``w`` ([..., rows, cols], bf16 or fp32) by the vector sequence of the
    reference's power iteration (spectral_ball_utils.py:151-166), on the HIP path: one Gram matrix on the matrix
    cores (squared once / twice from 6 / 16 rounds on, so that one launch stands for two / four rounds; the last
    application, whose quotient is the result, is the Gram matrix's). Returns fp32 of shape ``w.shape[:-2]``; no
    host sync."""
    import ctypes

    from .. import _lib
    if w.ndim < 2:
        raise ValueError("Input tensor must have at least 2 dimensions.")
    if steps < 1:
        raise ValueError(f"steps must be at least 1, got {steps}")
    _lib.require_cuda(w, "spectral_norm input")
    if w.dtype not in (torch.bfloat16, torch.float32):
        w = w.to(torch.float32)
    rows, cols = w.shape[-2:]
    mats = w.reshape(-1, rows, cols)
    if mats.stride(-1) != 1 or mats.stride(-2) < cols:
        mats = mats.contiguous()
    batch = mats.shape[0]
    sigma = torch.empty(batch, dtype=torch.float32, device=w.device)
    ptrs = (ctypes.c_void_p * batch)(*[mats[b].data_ptr() for b in range(batch)])
    prob = (_lib.SnProblem * 1)()
    q = prob[0]
    q.w_ptrs, q.sigma_out = ctypes.cast(ptrs, ctypes.POINTER(ctypes.c_void_p)), sigma.data_ptr()
    q.dtype, q.ld, q.batch, q.rows, q.cols = _lib.dtype_code(mats.dtype), mats.stride(-2), batch, rows, cols
    L = _lib.lib()
    ws = _lib.workspace(w.device, L.muon_spectral_norm_workspace_bytes(prob, 1), tag="sn")
    with torch.cuda.device(w.device):
        st = L.muon_spectral_norm(prob, 1, steps, ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(w.device))
    _lib.check(st, "muon_spectral_norm")
    return sigma.reshape(w.shape[:-2])


@torch.no_grad()
def power_iteration(w: torch.Tensor, steps: int = 50, eps: float = 1e-20):
    """(sigma, u, v) like spectral_ball_utils.py:151-166 of the reference: ``sigma`` fp32 of shape ``w.shape[:-2]``,
    ``u`` ``[..., rows, 1]`` and ``v`` ``[..., cols, 1]`` unit vectors in bf16, all from the HIP path
    (``muon_power_iteration``: the vector sequence runs on the Gram matrix of the short side; the short-side vector is
    its last iterate, the long-side one a single pass over the matrix). ``eps`` is unused, as in the reference."""
    import ctypes

    from .. import _lib
    if w.ndim < 2:
        raise ValueError("Input tensor must have at least 2 dimensions.")
    if steps < 1:
        raise ValueError(f"steps must be at least 1, got {steps}")
    _lib.require_cuda(w, "power_iteration input")
    if w.dtype not in (torch.bfloat16, torch.float32):
        w = w.to(torch.float32)
    rows, cols = w.shape[-2:]
    mats = w.reshape(-1, rows, cols)
    if mats.stride(-1) != 1 or mats.stride(-2) < cols:
        mats = mats.contiguous()
    batch = mats.shape[0]
    sigma = torch.empty(batch, dtype=torch.float32, device=w.device)
    u = torch.empty(batch, rows, dtype=torch.float32, device=w.device)
    v = torch.empty(batch, cols, dtype=torch.float32, device=w.device)
    ptrs = (ctypes.c_void_p * batch)(*[mats[b].data_ptr() for b in range(batch)])
    prob = (_lib.SnProblem * 1)()
    q = prob[0]
    q.w_ptrs, q.sigma_out = ctypes.cast(ptrs, ctypes.POINTER(ctypes.c_void_p)), sigma.data_ptr()
    q.dtype, q.ld, q.batch, q.rows, q.cols = _lib.dtype_code(mats.dtype), mats.stride(-2), batch, rows, cols
    L = _lib.lib()
    ws = _lib.workspace(w.device, L.muon_spectral_norm_workspace_bytes(prob, 1), tag="sn")
    with torch.cuda.device(w.device):
        st = L.muon_power_iteration(ctypes.cast(ptrs, ctypes.POINTER(ctypes.c_void_p)), q.dtype, q.ld, batch, rows, cols,
                                    steps, sigma.data_ptr(), u.data_ptr(), v.data_ptr(), ws.data_ptr(), ws.numel(),
                                    _lib.current_stream_ptr(w.device))
    _lib.check(st, "muon_power_iteration")
    lead = w.shape[:-2]
    u = torch.nn.functional.normalize(u, dim=-1).to(torch.bfloat16).reshape(*lead, rows, 1)
    v = torch.nn.functional.normalize(v, dim=-1).to(torch.bfloat16).reshape(*lead, cols, 1)
    return sigma.reshape(lead), u, v


@torch.no_grad()
def apply_retract(W: torch.Tensor, sigma: float, target_radius: float, mode: str = "hard", alpha: float = 0.05,
                  current_lr: Optional[float] = None) -> float:
    """Host-scalar retraction of one matrix, in place (spectral_ball_utils.py:168-212). MuonBall itself applies the
    same factor on the device, fused into its update kernel, without reading sigma back."""
    if mode == "hard":
        if max(sigma, 0.0) + 1e-8 != target_radius:
            W.mul_(target_radius / (max(sigma, 0.0) + 1e-8))
        return 0.0
    if mode == "dynamic":
        bias = -1.0 if sigma > target_radius else 1.0
        W.mul_(1.0 + (alpha * current_lr if current_lr is not None else alpha) * bias)
        return bias
    raise ValueError(f"Unknown retract mode: {mode}")


def compute_target_radius(shape: tuple, radius_mode: str, current_weight: Optional[torch.Tensor] = None,
                          radius_scaler: float = 1.0) -> float:
    """'spectral_mup' -> sqrt(n_out/n_in) * scaler, 'identity' -> scaler (spectral_ball_utils.py:432-440)."""
    if radius_mode == "spectral_mup":
        n_out, n_in = shape
        return radius_scaler * math.sqrt(n_out / n_in)
    if radius_mode == "identity":
        return radius_scaler * 1.0
    raise ValueError(f"Invalid radius_mode: {radius_mode}. Must be 'spectral_mup' or 'identity'.")


def get_spectral_ball_scale_factor(size_out: int, size_in: int, mode: str = "spectral") -> float:
    """spectral_ball_utils.py:442-466: align_adamw_rms 0.2*max(out,in)^0.5; shape_scaling max(1,out/in)^0.5;
    spectral_mup (out/in)^0.5."""
    if mode == "shape_scaling":
        return max(1, size_out / size_in) ** 0.5
    if mode == "align_adamw_rms":
        return 0.2 * max(size_out, size_in) ** 0.5
    if mode == "spectral_mup":
        return (size_out / size_in) ** 0.5
    raise ValueError(f"Invalid mode for SpectralBall update scale factor: {mode}")
