"""The default Newton-Schulz path (half-storage tail, Gram-side finish) on the spectra where storage precision and
range matter: log-spaced singular values, low rank plus noise, a near-rank-deficient matrix, gradients whose norm is
below the epsilon.  Every case runs through the HIP kernels (C ABI) and is compared with the oracle iterated in fp32
on the same bf16 input (lit_gpt/optim/muon.py:883-896).

Bars, stated per case: with the half-precision workspace every spectrum here but "low rank plus noise" holds the
contract's 1e-2 (that one: 2e-2); all-bf16 storage does not hold 1e-2 on any of them - neither does the reference's own
bf16 arithmetic, which is 1.6 to 2.3 times further from the fp32 run - so for bf16 the assertions are (i) no further
from the fp32 run than the reference's eager bf16 path, (ii) the tail no worse than the plain last iterations
(err_tail <= 1.1 err_plain + 2e-4, on the HIP results), (iii) a ceiling per spectrum.  In every case the output is
finite and each singular direction with sigma / |G|_F >= 1e-2 carries the value the scalar map of the coefficient
table assigns to it (u_i^T O v_i = p(sigma_i) within 1e-2).
"""
import math

import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu

NS_TOL = 1e-2


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm()).item()


def _from_svd(m, n, s, seed):
    g = torch.Generator().manual_seed(seed)
    U, _ = torch.linalg.qr(torch.randn(m, m, generator=g, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(n, m, generator=g, dtype=torch.float64))
    return ((U * s) @ V.T).float()


def _spectrum(kind, m, n, seed):
    if kind == "log":            # singular values log-spaced over three decades
        return _from_svd(m, n, torch.logspace(0, -3, m, dtype=torch.float64), seed)
    if kind == "lowrank":        # rank 16 plus 1e-2 Gaussian noise
        g = torch.Generator().manual_seed(seed + 1)
        return (torch.randn(m, 16, generator=g) @ torch.randn(16, n, generator=g) / 4.0
                + 1e-2 * torch.randn(m, n, generator=g))
    if kind == "deficient":      # half of the singular values at 1, half at 1e-4
        s = torch.ones(m, dtype=torch.float64)
        s[m // 2:] = 1e-4
        return _from_svd(m, n, s, seed + 2)
    raise ValueError(kind)


# ceiling of the relative Frobenius error against the fp32 run: (half workspace, bf16 storage)
CEIL = {"log": (NS_TOL, 4.5e-2), "lowrank": (2e-2, 1.6e-1), "deficient": (NS_TOL, 6.5e-2)}


@pytest.mark.parametrize("shape", [(512, 1408), (512, 512), (1408, 512)])
@pytest.mark.parametrize("kind", ["log", "lowrank", "deficient"])
def test_hard_spectra_through_the_kernels(gpu_device, kind, shape):
    import archscale_amd.optim.newton_schulz_hip as H
    print("case", kind, shape, flush=True)
    m, n = min(shape), max(shape)
    G = (_spectrum(kind, m, n, 7) * 1e-3)
    if shape[0] > shape[1]:
        G = G.mT.contiguous()
    G = G.to(torch.bfloat16)
    want = O.newton_schulz(G, O.QUINTIC, 1e-7, storage="fp32")
    eager = _rel(O.newton_schulz(G, O.QUINTIC, 1e-7, storage="bf16_eager"), want)
    Gd = G.double() if shape[0] <= shape[1] else G.double().mT
    U, S, Vh = torch.linalg.svd(Gd, full_matrices=False)
    s_in = S / Gd.norm()
    keep = s_in >= 1e-2
    p = O.ns_singular_value_map(s_in, O.QUINTIC)
    for prec in ("bf16", "f16"):
        res = {}
        for tail in (None, False):
            got = H.newton_schulz(G.to(gpu_device), O.QUINTIC, 1e-7, prec=prec, gram_tail=tail)
            torch.cuda.synchronize()
            assert torch.isfinite(got.float()).all()
            res[tail] = _rel(got, want)
            Od = got.double().cpu() if shape[0] <= shape[1] else got.double().cpu().mT
            d = torch.einsum("ij,ij->j", U, Od @ Vh.T)
            dev = (d - p)[keep].abs().max().item()
            print(kind, shape, prec, "tail" if tail is None else "plain", "err", res[tail], "sv dev", dev, flush=True)
            assert dev <= 1e-2
            assert (d - p).abs().max().item() <= 3e-2
        ceil = CEIL[kind][0 if prec == "f16" else 1]
        assert res[None] <= ceil and res[False] <= ceil
        if prec == "bf16":
            # the default takes the half-storage tail (and the Gram side for n >= 2m): no worse than plain iterations
            assert res[None] <= 1.1 * res[False] + 2e-4
            assert res[None] <= eager      # and closer to the fp32 run than the reference's own bf16 arithmetic
        else:
            assert res[None] == res[False]   # half workspace: the tail is off unless asked for


@pytest.mark.parametrize("prec", ["bf16", "f16"])
def test_norm_below_epsilon_and_zero(gpu_device, prec):
    """|G|_F far below eps (the additive epsilon dominates the normalisation: X0 = G / eps is tiny, every product of the
    iteration is tinier) and an all-zero input, with and without the tail: finite output, exact zeros stay zeros, and
    the result follows the oracle, whose fp32 iteration has no range problem.  In exact arithmetic a tiny X0 is only
    scaled: X5 = (prod a_k) X0 up to O(|X0|^3)."""
    import archscale_amd.optim.newton_schulz_hip as H
    g = torch.Generator().manual_seed(3)
    base = torch.randn(256, 640, generator=g)
    base = base / base.norm()
    a_prod = math.prod(a for a, _, _ in O.QUINTIC)
    errs = {}
    for norm in (1e-9, 1e-12):
        G = (base * norm).to(torch.bfloat16)
        want = O.newton_schulz(G, O.QUINTIC, 1e-7, storage="fp32")
        if norm <= 1e-11:
            lin = G.double() / (G.double().norm() + 1e-7) * a_prod
            assert _rel(want, lin) < 1e-2      # the oracle itself is in the linear regime
        for tail in (None, False, True):
            got = H.newton_schulz(G.to(gpu_device), O.QUINTIC, 1e-7, prec=prec, gram_tail=tail)
            torch.cuda.synchronize()
            assert torch.isfinite(got.float()).all()
            errs[(norm, tail)] = _rel(got, want)
            print("norm", norm, prec, tail, "err", errs[(norm, tail)], flush=True)
    for key, err in errs.items():
        assert err <= NS_TOL, key
    z = torch.zeros(3, 192, 448, dtype=torch.bfloat16, device=gpu_device)
    for tail in (None, False, True):
        assert torch.all(H.newton_schulz(z, O.QUINTIC, 1e-7, prec=prec, gram_tail=tail) == 0)


def test_custom_table_beyond_the_half_range_keeps_bf16_storage(gpu_device):
    """The half-storage tail assumes |B + aI| <= 1000 (it is stored times 2^6); every table of the reference is under 25.
    A custom table whose last rows are beyond that (1.5 |b| + 2.25 |c| + |a| > 500) must not take the tail: the default
    call equals the call with plain last iterations bit for bit, and stays finite where bf16 storage does."""
    import archscale_amd.optim.newton_schulz_hip as H
    g = torch.Generator().manual_seed(9)
    G = torch.randn(64, 96, generator=g).to(torch.bfloat16).to(gpu_device)
    mild = [(3.0, -3.2, 1.2)] * 3
    for last in [(2.0, -400.0, 0.0), (1.0, 0.0, 300.0)]:
        coeffs = mild + [last, last]
        got = H.newton_schulz(G, coeffs, 1e-7)
        plain = H.newton_schulz(G, coeffs, 1e-7, gram_tail=False)
        torch.cuda.synchronize()
        assert torch.equal(got, plain)
        assert torch.isfinite(got.float()).all()
    # a table inside the range still takes the tail by default (the two calls differ)
    coeffs = mild + [(2.0, -1.5, 0.5)] * 2
    assert not torch.equal(H.newton_schulz(G, coeffs, 1e-7), H.newton_schulz(G, coeffs, 1e-7, gram_tail=False))
