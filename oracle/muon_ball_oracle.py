"""CPU restatement of the reference's MuonBall arithmetic (PyTorch, eager, CPU).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``; never by the product package.

Follows emerging_optimizers/orthogonalized_optimizers/muon_ball.py (compute_muon_ball_update :60-142, the
component splits of ``orthogonalize`` :349-636) and spectral_ball_utils.py (power_iteration :151-166, apply_retract
:168-212, compute_target_radius :432-440, get_spectral_ball_scale_factor :442-466), with the rounding points of the
reference's eager execution (the power iteration runs on a bf16 copy of W with bf16 vectors).

What pins this file (tests/test_muon_ball_oracle.py):
  * power iteration: equals the top singular value from an fp64 SVD when the spectrum has a gap; for any matrix the
    k-round estimate equals the fp64 value of  |W x| / |x|,  x = (W^T W)^k 1  (the definition), and the two Gram
    forms used by the HIP path are algebraically the same number.                                   -> pinned
  * retraction: after a hard retraction the fp64 spectral norm is R; dynamic factor 1 +- alpha*lr.  -> pinned
  * radius / scale factor: scalar closed forms.                                                     -> pinned
  * splits (QKV component / group / head, FC1, MoE experts): every component of the fused tensor is updated exactly
    as the same matrix passed alone (self-consistency; the slicing itself follows the cited lines); in the QKV
    "component" mode the parameter is not retracted, because the reference retracts a reshape copy.  -> pinned
  * bf16 rounding noise of the reference's bf16 vectors (about 1e-3 on sigma) is not bit-defined across matmul
    back-ends: "parity unpinned" at the bit level, absorbed by the 2e-2 tolerance on weights.
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional, Sequence, Tuple

import torch

from . import muon_oracle as O

Tensor = torch.Tensor


def power_iteration(w: Tensor, steps: int = 50) -> Tuple[Tensor, Tensor, Tensor]:
    """(sigma, u, v) exactly as spectral_ball_utils.py:151-166: bf16 matrix, v0 = 1, `steps` bilateral rounds."""
    if w.ndim < 2:
        raise ValueError("Input tensor must have at least 2 dimensions.")
    w = w.to(torch.bfloat16)
    v = torch.ones_like(w[..., :1, :].transpose(-2, -1))
    for _ in range(steps):
        v = torch.nn.functional.normalize(w.transpose(-2, -1) @ (w @ v), dim=-2)
    u = torch.nn.functional.normalize(w @ v, dim=-2)
    s = (u.transpose(-2, -1) @ w @ v).squeeze(-1).squeeze(-1)
    return s, u, v


def power_iteration_fp64(w: Tensor, steps: int = 50) -> float:
    """The same vector sequence in fp64 on the bf16-rounded matrix: |W x| / |x| with x = (W^T W)^steps 1."""
    W = w.to(torch.bfloat16).double()
    x = torch.ones(W.shape[1], dtype=torch.float64)
    for _ in range(steps):
        x = W.T @ (W @ x)
        n = x.norm()
        if n == 0:
            return 0.0
        x = x / n
    return float((W @ x).norm())


def power_iteration_gram_fp64(w: Tensor, steps: int = 50) -> float:
    """The two Gram-matrix forms the HIP path evaluates, in fp64 (same number as power_iteration_fp64):
    rows > cols:  G = W^T W, x = G^steps 1,            sigma^2 = x^T G x / x^T x
    rows <= cols: G = W W^T, x = G^(steps-1) (W 1),    sigma^2 = |G x|^2 / x^T G x"""
    W = w.to(torch.bfloat16).double()
    rows, cols = W.shape
    if rows > cols:
        G = W.T @ W
        x = torch.ones(cols, dtype=torch.float64)
        for _ in range(steps):
            x = G @ x
            x = x / x.norm().clamp_min(1e-300)
        return float(torch.sqrt((x @ (G @ x)) / (x @ x)))
    G = W @ W.T
    x = W @ torch.ones(cols, dtype=torch.float64)
    for _ in range(steps - 1):
        x = x / x.norm().clamp_min(1e-300)
        x = G @ x
    y = G @ x
    d = x @ y
    return float(torch.sqrt((y @ y) / d)) if d > 0 else 0.0


def compute_target_radius(shape: Sequence[int], radius_mode: str, radius_scaler: float = 1.0) -> float:
    """spectral_ball_utils.py:432-440."""
    if radius_mode == "spectral_mup":
        n_out, n_in = shape
        return radius_scaler * math.sqrt(n_out / n_in)
    if radius_mode == "identity":
        return radius_scaler * 1.0
    raise ValueError(f"Invalid radius_mode: {radius_mode}. Must be 'spectral_mup' or 'identity'.")


def spectral_ball_scale_factor(size_out: int, size_in: int, mode: str) -> float:
    """spectral_ball_utils.py:442-466."""
    if mode == "shape_scaling":
        return max(1, size_out / size_in) ** 0.5
    if mode == "align_adamw_rms":
        return 0.2 * max(size_out, size_in) ** 0.5
    if mode == "spectral_mup":
        return (size_out / size_in) ** 0.5
    raise ValueError(f"Invalid mode for SpectralBall update scale factor: {mode}")


def apply_retract(W: Tensor, sigma: float, target_radius: float, mode: str = "hard", alpha: float = 0.05,
                  current_lr: Optional[float] = None) -> float:
    """In place on W; returns the bias (spectral_ball_utils.py:168-212)."""
    if mode == "hard":
        if max(sigma, 0.0) + 1e-8 != target_radius:
            W.mul_(target_radius / (max(sigma, 0.0) + 1e-8))
        return 0.0
    if mode == "dynamic":
        bias = -1.0 if sigma > target_radius else 1.0
        W.mul_(1.0 + (alpha * current_lr if current_lr is not None else alpha) * bias)
        return bias
    raise ValueError(f"Unknown retract mode: {mode}")


def component_update(W: Tensor, M: Tensor, *, radius_mode: str, scale_mode: str, power_iteration_steps: int,
                     msign_steps: int, retract_mode: str, retract_alpha: float, current_lr: Optional[float],
                     ns_storage: str = "bf16_eager", sigma_fn: Callable[[Tensor, int], float] = None) -> Tensor:
    """_compute_component_update (muon_ball.py:316-352): retracts W in place, returns scale * msign(M)."""
    R = compute_target_radius(W.shape, radius_mode)
    if sigma_fn is None:
        sigma = float(power_iteration(W, power_iteration_steps)[0])
    else:
        sigma = sigma_fn(W, power_iteration_steps)
    apply_retract(W, sigma, R, mode=retract_mode, alpha=retract_alpha, current_lr=current_lr)
    phi = O.msign(M.to(torch.float32), msign_steps, storage=ns_storage)
    return phi * spectral_ball_scale_factor(W.shape[0], W.shape[1], scale_mode)


def orthogonalize(p: Tensor, grad: Tensor, *, lr: float, split: Optional[dict] = None, **kw) -> Tensor:
    """MuonBall.orthogonalize (muon_ball.py:354-636) for one 2-D parameter. `split` selects a fused layout:
    {"kind": "qkv", "shapes": (q, k, v), "mode": "component"|"group"|"head"}            (:495-600)
    {"kind": "fc1", "shapes": (gate, up)}                                                 (:602-621)
    {"kind": "moe1", "experts": E, "gated": bool, "split_fc1": bool}                      (:407-462)
    {"kind": "moe2", "experts": E}                                                        (:464-493)
    Retracts the matching slices of p in place and returns the update of p's shape."""
    cu = lambda W, M: component_update(W, M, current_lr=lr, **kw)
    if split is None:
        return cu(p, grad)
    out_dim, in_dim = p.shape
    upd = torch.empty(p.shape, dtype=torch.float32)
    kind = split["kind"]
    if kind == "fc1":
        g, u = split["shapes"]
        assert out_dim == g + u
        upd[:g] = cu(p[:g], grad[:g])
        upd[g:] = cu(p[g:], grad[g:])
        return upd
    if kind == "qkv":
        shapes = list(split["shapes"])
        ssum = sum(shapes)
        assert out_dim % ssum == 0
        G = out_dim // ssum
        Wv, Mv, Uv = p.view(G, ssum, in_dim), grad.view(G, ssum, in_dim), upd.view(G, ssum, in_dim)
        offs = [0, shapes[0], shapes[0] + shapes[1], ssum]
        mode = split["mode"]
        if mode == "component":
            for i in range(3):
                # the rows of one component over all groups are not uniformly strided, so reshape COPIES
                # (muon_ball.py:585-586): the retraction inside the component update lands on the copy and the
                # parameter itself is NOT retracted in this mode (kept as the reference behaves)
                Wi = Wv[:, offs[i]:offs[i + 1]].reshape(-1, in_dim)
                Mi = Mv[:, offs[i]:offs[i + 1]].reshape(-1, in_dim)
                Uv[:, offs[i]:offs[i + 1]] = cu(Wi, Mi).view(G, shapes[i], in_dim)
            return upd
        for g in range(G):
            for i in range(3):
                Wi, Mi = Wv[g, offs[i]:offs[i + 1]], Mv[g, offs[i]:offs[i + 1]]
                if mode == "head" and i == 0:
                    kv = shapes[1]
                    heads = shapes[0] // kv
                    for h in range(heads):
                        Uv[g, h * kv:(h + 1) * kv] = cu(Wi[h * kv:(h + 1) * kv], Mi[h * kv:(h + 1) * kv])
                else:
                    Uv[g, offs[i]:offs[i + 1]] = cu(Wi, Mi)
        return upd
    if kind == "moe1":
        E, mult = split["experts"], (2 if split.get("gated") else 1)
        ffn = in_dim // (E * mult)
        Wr, Mr, Ur = p.view(out_dim, E, ffn * mult), grad.view(out_dim, E, ffn * mult), upd.view(out_dim, E, ffn * mult)
        for e in range(E):
            if split.get("split_fc1") and mult == 2:
                for lo in (0, ffn):
                    Ur[:, e, lo:lo + ffn] = cu(Wr[:, e, lo:lo + ffn].t(), Mr[:, e, lo:lo + ffn].t()).t()
            else:
                Ur[:, e, :] = cu(Wr[:, e, :].t(), Mr[:, e, :].t()).t()
        return upd
    if kind == "moe2":
        E = split["experts"]
        ffn = out_dim // E
        Wr, Mr, Ur = p.view(E, ffn, in_dim), grad.view(E, ffn, in_dim), upd.view(E, ffn, in_dim)
        for e in range(E):
            Ur[e] = cu(Wr[e].t(), Mr[e].t()).t()
        return upd
    raise ValueError(kind)


def muon_ball_step(p: Tensor, grad: Tensor, buf: Tensor, *, lr: float, beta: float, wd: float, nesterov: bool,
                   wd_method: str, split: Optional[dict] = None, **kw) -> None:
    """One MuonBall update of one 2-D parameter, in place on p, grad (l2 only) and buf
    (orthogonalized_optimizer.py:166-228 with MuonBall.orthogonalize)."""
    if wd != 0.0:
        if wd_method == "decoupled":
            p.add_(p, alpha=-wd * lr)
        elif wd_method == "independent":
            p.add_(p, alpha=-wd)
        elif wd_method == "l2":
            grad.add_(p, alpha=wd)
        else:
            raise ValueError(f"Invalid weight decay method: {wd_method}")
    buf.lerp_(grad, 1 - beta)
    g = grad.lerp(buf, beta) if nesterov else buf
    upd = orthogonalize(p, g, lr=lr, split=split, **kw)
    p.add_(upd, alpha=-lr)
