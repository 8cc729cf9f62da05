"""CPU restatement of the reference's Muon / MuonH arithmetic (PyTorch, eager, CPU).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py``; never by the product package.

Every function follows one piece of the reference (cited as file:line relative
to the reference checkout) and is written so that the *rounding points* of the
reference's eager CPU execution are kept: an operation the reference performs on
a bf16 tensor is performed on a bf16 tensor here too, so the result is rounded
at the same place.  ``storage="fp32"`` gives the tolerance oracle ("the
reference run in fp32 on the same bf16 inputs").

What pins this file (see tests/test_oracle.py):
  * Newton-Schulz: the fp64 closed form  U diag(p_k(..p_1(s_i/(|G|_F+eps)))) V^T
    from an SVD, transposition / orthogonal-equivariance / scale invariance,
    zero rows, batch independence.                                -> pinned
  * momentum: k-step closed form with a constant gradient.        -> pinned
  * lr adjustments / scale factors: scalar closed forms.          -> pinned
  * plain update, cautious mask: element-wise closed form and a sign truth
    table.                                                        -> pinned
  * MuonH: norm preservation, direction, U = 0 clamp path and the expansion
    |X - sU|^2 = |X|^2 - 2s<X,U> + s^2|U|^2.                      -> pinned
  * bf16 rounding ORDER inside the reference's compiled graphs (Inductor may
    fuse differently from eager) is not bit-defined by the reference itself;
    bit-level agreement with it is "parity unpinned".  The stated tolerances
    (1e-2 on NS, 2e-2 on weights) absorb it.
The reference ships no golden vector or test for this path.
"""
from __future__ import annotations

import math
from typing import Iterable, List, Optional, Sequence, Tuple

import torch

Tensor = torch.Tensor
Coeffs = Sequence[Tuple[float, float, float]]

# --------------------------------------------------------------------------
# Coefficient tables
# --------------------------------------------------------------------------

#: lit_gpt/legacy_optim.py:198 and emerging_optimizers/orthogonalized_optimizers/muon_utils.py:27-29
SIMPLE = ((3.4445, -4.7750, 2.0315),)

#: lit_gpt/optim/muon.py:875-881, lit_gpt/optim/newton_schulz_triton.py:350-356,
#: emerging_optimizers/orthogonalized_optimizers/muon_utils.py:30-38
QUINTIC = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)

#: emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:56-65 (used by msign)
POLAR_EXPRESS_MSIGN = (
    (8.2051, -22.9019, 16.4607),
    (4.0664, -2.8612, 0.5184),
    (3.9096, -2.8234, 0.5250),
    (3.2856, -2.4153, 0.4853),
    (2.2779, -1.6198, 0.3985),
    (1.8726, -1.2307, 0.3585),
    (1.8564, -1.2132, 0.3568),
    (1.8750, -1.2500, 0.3750),
)

#: emerging_optimizers/orthogonalized_optimizers/muon_utils.py:39-49
POLAR_EXPRESS = (
    (7.2086, -15.5131, 9.0178),
    (3.9623, -2.5813, 0.4542),
    (3.9466, -2.5765, 0.4544),
    (3.8991, -2.5671, 0.4566),
    (3.7186, -2.5308, 0.4653),
    (3.1390, -2.3073, 0.4733),
    (2.1715, -1.5246, 0.3885),
    (1.8648, -1.2224, 0.3577),
)

#: emerging_optimizers/orthogonalized_optimizers/muon_utils.py:50-57
AOL = (
    (4.0098, -7.0585, 2.4635),
    (3.4585, -5.5479, 2.5959),
    (2.7573, -3.2939, 1.4254),
    (2.7215, -3.0494, 1.3169),
)


def coefficient_schedule(name: str, steps: int) -> List[Tuple[float, float, float]]:
    """Expand a named table to one (a, b, c) row per iteration.

    "simple" repeats its row (legacy_optim.py:205), "quintic" is the 5-row
    production schedule (muon.py:890), "msign" indexes the 8-row table by
    iteration and repeats the last row beyond it (spectral_ball_utils.py:67-72),
    the muon_utils sets cycle ``i % len(set)`` (muon_utils.py:157-158).
    """
    if name == "simple":
        return [SIMPLE[0]] * steps
    if name == "quintic":
        return [QUINTIC[i % len(QUINTIC)] for i in range(steps)]
    if name == "msign":
        return [POLAR_EXPRESS_MSIGN[min(i, 7)] for i in range(steps)]
    if name == "polar_express":
        return [POLAR_EXPRESS[i % len(POLAR_EXPRESS)] for i in range(steps)]
    if name == "aol":
        return [AOL[i % len(AOL)] for i in range(steps)]
    raise ValueError(f"unknown coefficient table {name!r}")


# --------------------------------------------------------------------------
# Newton-Schulz
# --------------------------------------------------------------------------

def _bf16_round(t: Tensor) -> Tensor:
    return t.to(torch.bfloat16).to(torch.float32)


def newton_schulz(
    G: Tensor,
    coeffs: Coeffs,
    eps: float = 1e-7,
    *,
    eps_mode: str = "add",
    storage: str = "fp32",
    gram_tail: Optional[bool] = None,
) -> Tensor:
    """Quintic Newton-Schulz  X <- aX + (bA + cA^2)X,  A = X X^T.

    Follows lit_gpt/optim/muon.py:883-897 (== newton_schulz_triton.py:327-341,
    legacy_optim.py:199-213): cast to bf16, transpose tall matrices, divide by
    the per-matrix Frobenius norm (+eps), iterate, transpose back.

    eps_mode "add":   X / (|X| + eps)                      (muon.py:888)
             "clamp": X / max(|X|, eps) = F.normalize      (spectral_ball_utils.py:46,
                                                            muon_utils.py:125)
    storage  "fp32":        bf16 input, every later op in fp32 (tolerance oracle)
             "bf16_eager":  every op on bf16 tensors, as the reference's CPU path
             "bf16_gemm":   one bf16 rounding per GEMM epilogue, the rounding
                            points of newton_schulz_triton.py:374-378; the normalised
                            input itself is NOT rounded again (the HIP path keeps the
                            bf16 input exactly and applies the factor in fp32)
             "bf16_gemm_bsplit": as bf16_gemm but B kept as a bf16 hi+lo pair
             "f16_gemm":    a model of the HIP path's half-precision workspace (no counterpart in the reference): one
                            IEEE-half rounding per GEMM epilogue with X, A, B kept times 2^sx, 2^8, 2^6
                            (sx = floor(log2 sqrt(m n)) - 3), bf16 result; the first iteration runs on the exact input
                            with A and B in bf16
             "bf16_gemm" and "f16_gemm" also model two more choices of the HIP path (no counterpart in the
             reference): a*I inside B in the iterations after the first with |a| <= 4.2, and, with ``gram_tail`` (None:
             "bf16_gemm" only) and at least three iterations whose last two rows have |a| <= 4.2, the last two
             iterations in half storage and,
             when n >= 2m, on the Gram side: X_N = (P_N P_{N-1}) X_{N-2}, A_{N-1} = P_{N-1} A_{N-2} P_{N-1},
             P = aI + bA + cA^2.
    Returns bf16 for the bf16 / f16 modes and fp32 for "fp32", shaped like G.
    """
    if G.ndim < 2:
        raise ValueError("Newton-Schulz needs at least 2 dimensions")
    tall = G.size(-2) > G.size(-1)
    if storage in ("bf16_gemm", "f16_gemm") and G.size(-2) == G.size(-1):
        tall = True   # the models of the HIP path follow its orientation: it iterates on the transpose of a square matrix
    X = G.to(torch.bfloat16)
    if tall:
        X = X.mT

    if storage == "bf16_eager":
        nrm = X.norm(dim=(-2, -1), keepdim=True)
        X = X / (nrm + eps) if eps_mode == "add" else X / nrm.clamp_min(eps)
        for a, b, c in coeffs:
            A = X @ X.mT
            B = b * A + c * (A @ A)
            X = a * X + B @ X
    else:
        X = X.to(torch.float32)
        nrm = X.norm(dim=(-2, -1), keepdim=True)
        X = X / (nrm + eps) if eps_mode == "add" else X / nrm.clamp_min(eps)
        if storage == "fp32":
            for a, b, c in coeffs:
                A = X @ X.mT
                B = b * A + c * (A @ A)
                X = a * X + B @ X
        elif storage == "bf16_gemm_bsplit":
            for a, b, c in coeffs:
                A = _bf16_round(X @ X.mT)
                B = c * (A @ A) + b * A
                hi = _bf16_round(B)
                lo = _bf16_round(B - hi)
                X = _bf16_round(a * X + hi @ X + lo @ X)
            X = X.to(torch.bfloat16)
        elif storage in ("bf16_gemm", "f16_gemm"):
            m, n = X.shape[-2], X.shape[-1]
            N = len(coeffs)
            sx = max(int(math.floor(0.5 * math.log2(m * n))) - 3, 0)

            def half(t: Tensor, shift: int) -> Tensor:
                return (t * 2.0 ** shift).to(torch.float16).to(torch.float32) * 2.0 ** -shift

            def fold_ok(it: int) -> bool:
                return it > 0 and abs(coeffs[it][0]) <= 4.2

            wanted = (storage == "bf16_gemm") if gram_tail is None else gram_tail
            tail = wanted and N >= 3 and fold_ok(N - 2) and fold_ok(N - 1)
            first_half = 1 if storage == "f16_gemm" else (N - 2 if tail else N)
            eye = torch.eye(m, dtype=torch.float32)
            for it, (a, b, c) in enumerate(coeffs):
                last = it == N - 1
                half_ops = it >= first_half
                half_out = not last and it + 1 >= first_half
                rA = (lambda t: half(t, 8)) if half_ops else _bf16_round
                rB = (lambda t: half(t, 6)) if half_ops else _bf16_round
                A = rA(X @ X.mT)
                if tail and n >= 2 * m and it == N - 2:
                    a2, b2, c2 = coeffs[N - 1]
                    P1 = rB(c * (A @ A) + b * A + a * eye)
                    T = rB(P1 @ A)
                    A2 = rA(T @ P1)
                    P2 = rB(c2 * (A2 @ A2) + b2 * A2 + a2 * eye)
                    X = _bf16_round(rB(P2 @ P1) @ X)
                    break
                B = c * (A @ A) + b * A
                Y = rB(B + a * eye) @ X if fold_ok(it) else a * X + rB(B) @ X
                X = half(Y, sx) if half_out else _bf16_round(Y)
            X = X.to(torch.bfloat16)
        else:
            raise ValueError(f"unknown storage {storage!r}")
    if tall:
        X = X.mT
    return X.contiguous()


def newton_schulz_flatten_policy(X: Tensor, flatten: bool) -> Tuple[Tensor, torch.Size]:
    """lit_gpt/optim/muon.py:830-836: 3-D+ -> 2-D when ``flatten``; otherwise
    4-D+ -> one leading batch dimension.  Returns the view and the shape to
    restore."""
    shape = X.shape
    if flatten and X.ndim >= 3:
        X = X.flatten(start_dim=1)
    elif X.ndim >= 4:
        X = X.flatten(end_dim=-3)
    return X, shape


def msign(G: Tensor, steps: int, *, storage: str = "bf16_eager") -> Tensor:
    """emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:37-74:
    fp32 input required, F.normalize(eps=1e-7) in fp32 *before* the bf16 cast,
    8-row polar-express table, bf16 result."""
    if G.ndim < 2:
        raise ValueError("Input tensor must have at least 2 dimensions.")
    if G.dtype != torch.float32:
        raise ValueError("Input tensor G must be in float32")
    tall = G.size(-2) > G.size(-1)
    X = G.mT if tall else G
    X = X / X.norm(dim=(-2, -1), keepdim=True).clamp_min(1e-7)
    coeffs = coefficient_schedule("msign", steps)
    if storage == "bf16_eager":
        X = X.to(torch.bfloat16)
        for a, b, c in coeffs:
            A = X @ X.mT
            B = torch.addmm(A, A, A, alpha=c, beta=b) if X.ndim == 2 else b * A + c * (A @ A)
            X = torch.addmm(X, B, X, alpha=1.0, beta=a) if X.ndim == 2 else a * X + B @ X
    elif storage == "fp32":
        X = _bf16_round(X)
        for a, b, c in coeffs:
            A = X @ X.mT
            B = b * A + c * (A @ A)
            X = a * X + B @ X
    else:
        raise ValueError(storage)
    X = X.mT if tall else X
    return X.contiguous()


def emerging_newton_schulz(x: Tensor, steps: int, coefficient_type: str = "polar_express",
                           custom_coefficient_sets: Optional[Coeffs] = None, eps: float = 1e-7,
                           transpose: Optional[bool] = None, *, storage: str = "bf16_eager") -> Tensor:
    """emerging_optimizers/orthogonalized_optimizers/muon_utils.py:68-164: fp32 input required; transpose (given, or
    rows > cols); F.normalize over the last two dimensions in fp32 (X / max(|X|, eps), :125); named coefficient set or
    a custom one, ``steps`` a multiple of its length and the set cycled ``i % len(set)`` (:127-139, :157-158); the
    normalised matrix rounded to bf16 (:144) and iterated with newton_schulz_step_tsyrk (:262-287: A = XX^T,
    B = cAA + bA, X' = BX + aX, each a bf16 product); fp32 result, transposed back.

    storage "bf16_eager": every product rounds to bf16 (the reference's semantics);
            "fp32": the same rounded input iterated in fp32 (tolerance oracle)."""
    if x.ndim < 2:
        raise ValueError("Input tensor x must have at least 2 dimensions since Muon is not for 1d parameters.")
    if x.dtype != torch.float32:
        raise ValueError(f"Input tensor x must be in float32, got {x.dtype}")
    if transpose is None:
        transpose = x.size(-2) > x.size(-1)
    if transpose:
        x = x.mT
    X = x / x.norm(dim=(-2, -1), keepdim=True).clamp_min(eps)
    named = {"simple": SIMPLE, "quintic": QUINTIC, "polar_express": POLAR_EXPRESS, "aol": AOL}
    if coefficient_type in named:
        sets = named[coefficient_type]
    elif coefficient_type == "custom":
        if custom_coefficient_sets is None:
            raise ValueError("custom_coefficient_sets must be provided when coefficient_type is 'custom'.")
        sets = custom_coefficient_sets
    else:
        raise ValueError(f"Invalid coefficient type: {coefficient_type}")
    if steps % len(sets) != 0:
        raise ValueError(f"steps ({steps}) must be multiple of len(coefficient_sets) ({len(sets)}).")
    X = X.to(torch.bfloat16)
    if storage == "fp32":
        X = X.to(torch.float32)
    elif storage != "bf16_eager":
        raise ValueError(storage)
    for i in range(steps):
        a, b, c = sets[i % len(sets)]
        A = X @ X.mT
        B = c * (A @ A) + b * A
        X = B @ X + a * X
    X = X.to(torch.float32)
    if transpose:
        X = X.mT
    return X.contiguous()


def ns_singular_value_map(s: Tensor, coeffs: Coeffs) -> Tensor:
    """Scalar action of the iteration on one singular value: p(s) = a s + b s^3 + c s^5
    applied once per row of ``coeffs`` (what NS does in exact arithmetic)."""
    s = s.to(torch.float64)
    for a, b, c in coeffs:
        s2 = s * s
        s = s * (a + s2 * (b + c * s2))
    return s


# --------------------------------------------------------------------------
# lit_gpt Muon: momentum, lr adjustment, updates
# --------------------------------------------------------------------------

def muon_pre_orthogonalize(G: Tensor, M: Tensor, mu: float, nesterov: bool) -> Tensor:
    """lit_gpt/optim/muon.py:665-681.  M <- mu*M + G in M's dtype (in place);
    U = mu*M + G (nesterov) or M; U is returned in bf16."""
    g = G.to(M.dtype)
    M.mul_(mu).add_(g)
    U = M * mu + g if nesterov else M
    return U.to(torch.bfloat16)


def adjust_lr(lr: float, shape: Sequence[int], mode: Optional[str], flatten: bool = False) -> float:
    """lit_gpt/optim/muon.py:598-609, 841-866."""
    if mode is None:
        return lr
    if flatten:
        fan_out, fan_in = shape[0], math.prod(shape[1:])
    else:
        fan_out, fan_in = shape[-2], shape[-1]
    if mode == "spectral_norm":
        return lr * math.sqrt(fan_out / fan_in)
    if mode == "clip_norm":
        return lr * max(1.0, fan_out / fan_in) ** 0.5
    if mode == "rms_norm":
        return lr * 0.2 * math.sqrt(max(fan_out, fan_in))
    raise ValueError(f"Unknown adjust_lr value: {mode}")


def _weight_decay_(X: Tensor, U: Tensor, lr: float, wd: float, cautious: bool) -> None:
    """lit_gpt/optim/muon.py:703-718 (== 738-751)."""
    if cautious:
        mask = torch.clamp(torch.sign(X * U) + 1, max=1)  # {-1,0,1} -> {0,1,1}
        X.sub_(X * mask * (lr * wd))
    else:
        X.mul_(1 - lr * wd)


def muon_post_orthogonalize(X: Tensor, U: Tensor, lr: float, adjusted_lr: float, wd: float,
                            cautious: bool = False) -> None:
    """lit_gpt/optim/muon.py:703-722: weight decay, then X <- X - adjusted_lr*U
    (U*adjusted_lr is rounded in U's dtype first, as ``_foreach_mul(U, lr)`` does)."""
    _weight_decay_(X, U, lr, wd, cautious)
    X.sub_(U * adjusted_lr)


def muonh_post_orthogonalize(X: Tensor, U: Tensor, lr: float, wd: float, eps: Optional[float],
                             cautious: bool = False) -> None:
    """MuonH update of ONE tensor (one norm over the whole tensor, also for a 3-D
    stack): lit_gpt/optim/muon.py:614-639 with 725-818.  Norms are taken in the
    tensors' own dtype (bf16 norms round to bf16), U*s and *lr round separately."""
    e = 1e-10 if eps is None else eps
    _weight_decay_(X, U, lr, wd, cautious)
    x_norm = X.norm().reshape(1).square().sqrt()       # muon.py:754-758, 625
    u_norm = U.norm().reshape(1).square().sqrt()
    scale = (x_norm / u_norm.clamp_min(e)).squeeze(0)  # muon.py:780-784
    U_scaled = U * scale
    U_scaled.mul_(lr)
    X.sub_(U_scaled)                                   # muon.py:787-791
    new_norm = X.norm().reshape(1).square().sqrt()     # muon.py:794-795, 636
    X.mul_((x_norm / new_norm.clamp_min(e)).squeeze(0))  # muon.py:814-818


def muonh_post_fp64(X: Tensor, U: Tensor, lr: float, wd: float, eps: float,
                    cautious: bool = False) -> Tensor:
    """The same MuonH update in exact-ish arithmetic (fp64, no storage rounding):
    what both the reference and the HIP path approximate.  Returns new X (fp64)."""
    x = X.to(torch.float64)
    u = U.to(torch.float64)
    if cautious:
        x = x - x * torch.clamp(torch.sign(x * u) + 1, max=1) * (lr * wd)
    else:
        x = x * (1 - lr * wd)
    xn = x.norm()
    un = u.norm()
    y = x - u * (xn / un.clamp_min(eps)) * lr
    return y * (xn / y.norm().clamp_min(eps))


def lit_gpt_muon_step(
    X: Tensor, G: Tensor, M: Tensor, *, lr: float, mu: float, wd: float, eps: float,
    nesterov: bool, adjust: Optional[str], flatten: bool, cautious: bool, use_muonh: bool,
    coeffs: Coeffs = QUINTIC, ns_storage: str = "bf16_eager",
) -> None:
    """One single-GPU Muon / MuonH update of one parameter, in place on X and M:
    lit_gpt/optim/muon.py:494-499, 589-650 (the ``len(U) == 1`` branch)."""
    U = muon_pre_orthogonalize(G, M, mu, nesterov)
    Uv, shape = newton_schulz_flatten_policy(U, flatten)
    O = newton_schulz(Uv, coeffs, eps, storage=ns_storage).to(torch.bfloat16).reshape(shape)
    if use_muonh:
        muonh_post_orthogonalize(X, O, lr, wd, eps, cautious)
    else:
        muon_post_orthogonalize(X, O, lr, adjust_lr(lr, X.shape, adjust, flatten), wd, cautious)


def create_param_batches(keys: Iterable[Tuple], batch_size: int) -> List[List[int]]:
    """lit_gpt/optim/opt_utils.py:53-70 on indices: group by key in first-seen
    order, split each group into runs of ``batch_size``."""
    groups: dict = {}
    for i, k in enumerate(keys):
        groups.setdefault(k, []).append(i)
    out = []
    for g in groups.values():
        for i in range(0, len(g), batch_size):
            out.append(g[i:i + batch_size])
    return out


# --------------------------------------------------------------------------
# emerging_optimizers Muon
# --------------------------------------------------------------------------

def muon_scale_factor(size_out: int, size_in: int, mode: str) -> float:
    """emerging_optimizers/orthogonalized_optimizers/muon.py:122-148."""
    if mode == "shape_scaling":
        return max(1, size_out / size_in) ** 0.5
    if mode == "align_adamw_rms":
        return 0.2 * max(size_out, size_in) ** 0.5
    if mode == "spectral_mup":
        return (size_out / size_in) ** 0.5
    raise ValueError(f"Invalid mode for Muon update scale factor: {mode}")


def emerging_muon_step(
    p: Tensor, grad: Tensor, buf: Tensor, *, lr: float, beta: float, wd: float,
    nesterov: bool, wd_method: str, steps: int, scale_mode: str, extra_scale: float,
    ns_storage: str = "bf16_eager",
) -> None:
    """One update of one 2-D parameter, in place on p, grad (l2 only) and buf:
    emerging_optimizers/orthogonalized_optimizers/orthogonalized_optimizer.py:166-228,
    mixin.py:33-52, muon.py:97-105."""
    if p.dim() == 1:
        raise ValueError("Muon does not support 1D parameters")
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
    o = msign(g, steps, storage=ns_storage)
    o = o * muon_scale_factor(g.size(-2), g.size(-1), scale_mode) * extra_scale
    p.add_(o, alpha=-lr)
