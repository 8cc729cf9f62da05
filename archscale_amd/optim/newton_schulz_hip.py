"""Newton-Schulz orthogonalisation on MI355X: host side of ``muon_ns_batched`` / ``muon_syrk``.

Mirrors the callables of the reference that a user can install as
``Muon(newton_schulz_func=...)``:

* ``zeropower_via_newtonschulz5(G, epsilon)``  lit_gpt/optim/muon.py:869-897
* ``newton_schulz_triton(G, epsilon)``         lit_gpt/optim/newton_schulz_triton.py:344-382
  (here the same HIP path; ``newton_schulz_hip`` is the native name)
* ``zeropower_via_newtonschulz5_legacy(G, steps)``  lit_gpt/legacy_optim.py:187-213
* ``ns_line_1`` / ``ns_line_2``                lit_gpt/optim/newton_schulz_triton.py:142-178, 269-310

All of them run hand-written gfx950 kernels; there is no PyTorch fallback.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple, Union

import torch
from torch import Tensor

from .. import _lib

Coeffs = Sequence[Tuple[float, float, float]]

#: lit_gpt/optim/muon.py:875-881
QUINTIC_SCHEDULE: Coeffs = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
#: lit_gpt/legacy_optim.py:198
SIMPLE_ROW = (3.4445, -4.7750, 2.0315)

_PREC = {"bf16": _lib.PREC_BF16, "bsplit": _lib.PREC_BF16_BSPLIT, "f16": _lib.PREC_F16}
#: iterations (counted from the end) that keep B as a hi+lo pair wherever this package asks for the split itself.
#: Measured against fp32 runs on the same bf16 input (N(0,1), 256x2048 .. 2048x5632): constant-row table x5
#: 1.1-1.3e-2 without the split, 7.7-8.3e-3 with the last 2, 6.0-6.8e-3 with the last 3 and with all 5; the
#: polar-express table x5 8.1-9.2e-3 / 6.9-8.5e-3 / 5.7-7.4e-3 / 5.7-7.3e-3.
BSPLIT_TAIL = 3
#: precision mode for the coefficient tables that plain bf16 storage cannot keep within 1e-2 of an fp32 run (constant
#: coefficients, polar express): the half-precision workspace - one walk per product, a third of the error of the
#: hi+lo pair
ACCURATE_PREC = "f16"
_EPS = {"add": _lib.EPS_ADD, "clamp": _lib.EPS_CLAMP}


def _as_float(epsilon: Union[float, Tensor]) -> float:
    # the reference hands the hook a 0-d CPU tensor (muon.py:235); accept both
    return float(epsilon.item()) if isinstance(epsilon, Tensor) else float(epsilon)


def _as_batch(G: Tensor) -> Tuple[Tensor, int, int, int, int, int]:
    """View G as [batch] matrices with unit column stride: (tensor, batch, rows, cols, batch_stride, ld)."""
    if G.ndim < 2:
        raise ValueError("Newton-Schulz needs a tensor with at least 2 dimensions")
    if G.ndim > 3:
        G = G.flatten(end_dim=-3) if G.is_contiguous() else G.contiguous().flatten(end_dim=-3)
    rows, cols = G.shape[-2], G.shape[-1]
    batch = G.shape[0] if G.ndim == 3 else 1
    ok = G.stride(-1) == 1 and G.stride(-2) >= cols
    if G.ndim == 3 and batch > 1:
        ok = ok and G.stride(0) >= 0
    if not ok:
        G = G.contiguous()
    bstride = G.stride(0) if (G.ndim == 3 and batch > 1) else rows * G.stride(-2)
    return G, batch, rows, cols, bstride, G.stride(-2)


def newton_schulz(
    G: Tensor,
    coeffs: Coeffs = QUINTIC_SCHEDULE,
    epsilon: Union[float, Tensor] = 1e-7,
    *,
    eps_mode: str = "add",
    prec: str = "bf16",
    cast_input_first: bool = True,
    out: Optional[Tensor] = None,
    bsplit_tail: int = 0,
    normalize: bool = True,
    diag_fold: bool = True,
    gram_tail: Optional[bool] = None,
) -> Tensor:
    """Orthogonalise every matrix of ``G`` (``[..., rows, cols]``, bf16 or fp32) with the quintic
    Newton-Schulz iteration ``X <- aX + (bA + cA^2)X, A = XX^T``, one ``(a, b, c)`` row per iteration.

    Returns a new bf16 tensor shaped like ``G`` (``G`` itself is not modified unless ``out is G``).
    ``prec="f16"`` keeps the iterate and both Gram-side matrices in IEEE half inside the workspace (scaled by powers of
    two; 8x the mantissa of bf16 at the same matrix-core rate): what the constant-coefficient and polar-express tables
    need to stay within 1e-2 of an fp32 run.  ``prec="bsplit"`` is a diagnostic mode that nothing in the package uses
    (slower and less accurate than "f16"): it stays in bf16 and keeps ``B = bA + cA^2`` as a hi+lo
    pair (a second walk over K in ``BX``); ``bsplit_tail=t`` does so only in the
    last ``t`` iterations (0 = all), whose rounding dominates the error of the result.  ``normalize=False`` iterates on
    the input as it is (``epsilon`` is then unused).  ``diag_fold=False`` keeps ``aX`` as a separate addend in every
    iteration instead of storing ``B + aI`` in the iterations after the first with ``|a| <= 4.2``.
    ``gram_tail``: with three or more iterations the last two can be stored in half and, for matrices whose long side
    is at least twice the short one, finished on the Gram side (``X_N = P_N P_{N-1} X_{N-2}``: one ``BX`` product
    less).  ``None`` (default) does so for ``prec="bf16"`` only, ``True`` also for "f16", ``False`` never.
    """
    _lib.require_cuda(G, "Newton-Schulz input")
    if G.dtype not in (torch.bfloat16, torch.float32):
        G = G.to(torch.float32)
    if len(coeffs) < 1:
        raise ValueError("need at least one Newton-Schulz iteration")
    shape = G.shape
    Gv, batch, rows, cols, bstride, ld = _as_batch(G)
    if out is None:
        out = torch.empty(shape, dtype=torch.bfloat16, device=G.device)
    else:
        if out.shape != shape or out.dtype != torch.bfloat16 or not out.is_contiguous() or out.device != G.device:
            raise ValueError("out must be a contiguous bfloat16 tensor shaped like the input, on the same device")
    L = _lib.lib()
    pm = _PREC[prec]
    nbytes = L.muon_ns_workspace_bytes(batch, rows, cols, pm)
    ws = _lib.workspace(G.device, nbytes)
    flags = (_lib.NS_CAST_INPUT_FIRST if cast_input_first else 0) | _lib.ns_bsplit_tail(bsplit_tail)
    if not normalize:
        flags |= _lib.NS_NO_NORMALIZE
    if not diag_fold:
        flags |= _lib.NS_NO_DIAG_FOLD
    if gram_tail is not None:
        flags |= _lib.NS_GRAM_TAIL if gram_tail else _lib.NS_NO_GRAM_TAIL
    with torch.cuda.device(G.device):
        st = L.muon_ns_batched(
            Gv.data_ptr(), _lib.dtype_code(Gv.dtype), bstride, ld,
            out.data_ptr(), rows * cols, cols,
            batch, rows, cols,
            _lib.abc_array(coeffs), len(coeffs), _as_float(epsilon), _EPS[eps_mode], pm, flags,
            ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(G.device))
    _lib.check(st, "muon_ns_batched")
    return out


def newton_schulz_grouped(
    inputs: Sequence[Tensor],
    coeffs: Coeffs = QUINTIC_SCHEDULE,
    epsilon: Union[float, Tensor] = 1e-7,
    *,
    eps_mode: str = "add",
    prec: str = "bf16",
    cast_input_first: bool = True,
    outs: Optional[Sequence[Tensor]] = None,
    bsplit_tail: int = 0,
    gram_tail: Optional[bool] = None,
) -> Sequence[Tensor]:
    """Orthogonalise several batches of DIFFERENT shapes in one call: every product of the iteration is a
    single kernel launch over the tiles of all batches (15 GEMM launches in total for five iterations).
    ``inputs[i]`` is ``[..., rows_i, cols_i]`` (bf16 or fp32); ``outs[i]`` (bf16, contiguous, may be the input)
    receives the result.  All tensors must live on one device."""
    if not inputs:
        return []
    device = inputs[0].device
    views = []
    for G in inputs:
        _lib.require_cuda(G, "Newton-Schulz input")
        if G.device != device:
            raise ValueError("all inputs of a grouped call must live on one device")
        if G.dtype not in (torch.bfloat16, torch.float32):
            G = G.to(torch.float32)
        views.append((G.shape, *_as_batch(G)))
    if outs is None:
        outs = [torch.empty(shape, dtype=torch.bfloat16, device=device) for shape, *_ in views]
    probs = (_lib.NsProblem * len(views))()
    for q, (shape, Gv, batch, rows, cols, bstride, ld), out in zip(probs, views, outs):
        if out.shape != shape or out.dtype != torch.bfloat16 or not out.is_contiguous() or out.device != device:
            raise ValueError("every out must be a contiguous bfloat16 tensor shaped like its input, on the same device")
        q.in_ptr, q.out_ptr = Gv.data_ptr(), out.data_ptr()
        q.in_batch_stride, q.out_batch_stride = bstride, rows * cols
        q.in_dtype, q.in_ld, q.out_ld = _lib.dtype_code(Gv.dtype), ld, cols
        q.batch, q.rows, q.cols = batch, rows, cols
    L = _lib.lib()
    pm = _PREC[prec]
    ws = _lib.workspace(device, L.muon_ns_grouped_workspace_bytes(probs, len(views), pm))
    flags = (_lib.NS_CAST_INPUT_FIRST if cast_input_first else 0) | _lib.ns_bsplit_tail(bsplit_tail)
    if gram_tail is not None:
        flags |= _lib.NS_GRAM_TAIL if gram_tail else _lib.NS_NO_GRAM_TAIL
    with torch.cuda.device(device):
        st = L.muon_ns_grouped(probs, len(views), _lib.abc_array(coeffs), len(coeffs), _as_float(epsilon),
                               _EPS[eps_mode], pm, flags, ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(device))
    _lib.check(st, "muon_ns_grouped")
    return list(outs)


def zeropower_via_newtonschulz5(G: Tensor, epsilon: Union[float, Tensor] = 1e-7) -> Tensor:
    """Drop-in for lit_gpt/optim/muon.py:869-897 (five iterations, production coefficient schedule)."""
    return newton_schulz(G, QUINTIC_SCHEDULE, epsilon)


def newton_schulz_hip(G: Tensor, epsilon: Union[float, Tensor] = 1e-7) -> Tensor:
    """Drop-in for ``newton_schulz_triton`` (lit_gpt/optim/newton_schulz_triton.py:344-382)."""
    return newton_schulz(G, QUINTIC_SCHEDULE, epsilon)


#: name kept so that ``from ... import newton_schulz_triton`` call sites keep working
newton_schulz_triton = newton_schulz_hip


def zeropower_via_newtonschulz5_legacy(G: Tensor, steps: int = 5) -> Tensor:
    """Drop-in for lit_gpt/legacy_optim.py:187-213: constant (3.4445, -4.7750, 2.0315) row, eps 1e-7."""
    assert G.ndim >= 2
    return newton_schulz(G, [SIMPLE_ROW] * steps, 1e-7, prec=ACCURATE_PREC)


# ---------------------------------------------------------------------------
# single products
# ---------------------------------------------------------------------------

def _syrk(A: Tensor, C: Optional[Tensor], alpha: float, beta: float, out: Optional[Tensor]) -> Tensor:
    _lib.require_cuda(A, "syrk input")
    if A.ndim > 3 or A.ndim < 2:
        raise ValueError(f"Input tensor must be 2D or 3D, but got {A.ndim}D tensor.")
    if A.dtype != torch.bfloat16:
        raise TypeError("Input tensor must be bfloat16")
    Av, batch, n, k, a_bs, lda = _as_batch(A)
    if out is None:
        out = torch.empty((*A.shape[:-1], n), device=A.device, dtype=A.dtype)
    assert out.size(-2) == n and out.size(-1) == n, "Output matrix has incorrect shape"
    if out.dtype != torch.bfloat16 or out.stride(-1) != 1:
        raise ValueError("out must be bfloat16 with unit column stride")
    d_bs = out.stride(0) if (out.ndim == 3 and batch > 1) else n * out.stride(-2)
    c_ptr, c_bs, ldc = 0, 0, 0
    if C is not None:
        if C.shape[-2:] != (n, n) or C.dtype != torch.bfloat16:
            raise RuntimeError("if c is provided, c must be bfloat16 of shape (N, N)")
        Cv, cb, _, _, c_bs, ldc = _as_batch(C)
        if cb != batch:
            raise RuntimeError("c must have the batch size of a")
        c_ptr = Cv.data_ptr()
    L = _lib.lib()
    ws = _lib.workspace(A.device, L.muon_syrk_workspace_bytes(batch, n, k), tag="syrk")
    with torch.cuda.device(A.device):
        st = L.muon_syrk(Av.data_ptr(), a_bs, lda, c_ptr, c_bs, ldc, out.data_ptr(), d_bs, out.stride(-2),
                         batch, n, k, float(alpha), float(beta), ws.data_ptr(), ws.numel(),
                         _lib.current_stream_ptr(A.device))
    _lib.check(st, "muon_syrk")
    return out


def ns_line_1(A: Tensor, *, out: Optional[Tensor] = None) -> Tensor:
    """C = A @ A.T for A of shape ([b,] M, K) (newton_schulz_triton.py:142-178)."""
    return _syrk(A, None, 1.0, 0.0, out)


def ns_line_2(A: Tensor, alpha: float, beta: float, *, out: Optional[Tensor] = None) -> Tensor:
    """C = alpha * A @ A.T + beta * A for symmetric A ([b,] M, M) (newton_schulz_triton.py:269-310)."""
    if A.shape[-2] != A.shape[-1]:
        raise ValueError(f"Input must be symmetric square matrix, but got shape {A.shape}")
    return _syrk(A, A, alpha, beta, out)


def tsyrk_ex(a: Tensor, c: Optional[Tensor] = None, alpha: float = 1.0, beta: float = 0.0) -> Tensor:
    """D = alpha * a @ a.T + beta * c with c symmetric (emerging_optimizers/triton_kernels/syrk.py:188-261);
    both triangles of D are written."""
    if a.dtype != torch.bfloat16:
        raise TypeError("Input tensor must be bfloat16")
    if a.dim() != 2:
        raise TypeError("Input tensor must be 2D")
    n = a.shape[0]
    if not ((c is None and beta == 0.0) or (c is not None and c.shape == (n, n))):
        raise RuntimeError("if c is provided, c must be of shape (N, N)")
    return _syrk(a, c if beta != 0.0 else None, alpha, beta, None)
