"""Pins the CPU oracle against what the mathematics fixes (no reference import).

The reference has no golden vector or test for the Muon path, so each oracle
function is checked against an independent closed form: an fp64 SVD for
Newton-Schulz, geometric sums for momentum, element-wise formulas for the
updates and the defining invariants of MuonH.
"""
import math

import pytest
import torch

from oracle import muon_oracle as O

torch.manual_seed(0)


def _svd_closed_form(G, coeffs, eps):
    """U diag(p(s/(|G|_F+eps))) V^T in fp64 from an SVD: independent of the iteration."""
    G64 = G.to(torch.bfloat16).to(torch.float64)
    U, S, Vh = torch.linalg.svd(G64, full_matrices=False)
    s = S / (G64.norm() + eps)
    return U @ torch.diag_embed(O.ns_singular_value_map(s, coeffs)) @ Vh


@pytest.mark.parametrize("shape", [(24, 64), (64, 24), (32, 32)])
@pytest.mark.parametrize("table", ["simple", "quintic", "msign"])
def test_ns_fp32_matches_svd_closed_form(shape, table):
    g = torch.Generator().manual_seed(sum(shape) * 7 + len(table))
    G = torch.randn(*shape, generator=g)
    coeffs = O.coefficient_schedule(table, 5)
    want = _svd_closed_form(G, coeffs, 1e-7)
    got = O.newton_schulz(G, coeffs, 1e-7, storage="fp32").to(torch.float64)
    # fp32 iteration vs exact: only fp32 round-off, amplified by the slope (~5e2) at zero
    assert (got - want).norm() / want.norm() < 2e-4


@pytest.mark.parametrize("kind,steps", [("simple", 3), ("quintic", 5), ("polar_express", 8), ("aol", 4), ("aol", 8),
                                        ("custom", 4)])
@pytest.mark.parametrize("shape", [(20, 48), (48, 20)])
def test_emerging_newton_schulz_matches_svd_closed_form(kind, steps, shape):
    """fp32 in / fp32 out, clamp eps, the named set cycled: against U diag(p(s / max(|X|, eps))) V^T from an fp64 SVD of
    the bf16-rounded normalised input (a wrong table row, a set indexed without the modulo or eps added instead of
    clamped fails this)."""
    g = torch.Generator().manual_seed(sum(shape) + steps)
    x = torch.randn(*shape, generator=g)
    custom = [(3.0, -3.2, 1.2), (2.0, -1.5, 0.5)] if kind == "custom" else None
    sets = {"simple": O.SIMPLE, "quintic": O.QUINTIC, "polar_express": O.POLAR_EXPRESS, "aol": O.AOL, "custom": custom}[kind]
    rows = [sets[i % len(sets)] for i in range(steps)]
    xn = (x / x.norm().clamp_min(1e-7)).to(torch.bfloat16).to(torch.float64)
    U, S, Vh = torch.linalg.svd(xn, full_matrices=False)
    want = U @ torch.diag_embed(O.ns_singular_value_map(S, rows)) @ Vh
    got = O.emerging_newton_schulz(x, steps, kind, custom, storage="fp32")
    assert got.dtype == torch.float32 and got.shape == x.shape
    assert (got.double() - want).norm() / want.norm() < 5e-4
    # the reference's own (all-bf16) semantics stay close to it; an explicit transpose flag changes nothing mathematically
    eager = O.emerging_newton_schulz(x, steps, kind, custom)
    assert (eager.double() - want).norm() / want.norm() < 6e-2
    flipped = O.emerging_newton_schulz(x, steps, kind, custom, transpose=shape[0] <= shape[1], storage="fp32")
    assert (flipped.double() - want).norm() / want.norm() < 5e-4
    # eps is a clamp, not an addend: a huge eps divides by eps exactly
    big = O.emerging_newton_schulz(x, 1, "custom", [(1.0, 0.0, 0.0)], eps=1e3, storage="fp32")
    assert torch.allclose(big, (x / 1e3).to(torch.bfloat16).float(), rtol=1e-6, atol=0)


def test_emerging_newton_schulz_errors():
    x = torch.randn(4, 8)
    with pytest.raises(ValueError):
        O.emerging_newton_schulz(x, 5, "aol")                 # 5 is no multiple of 4
    with pytest.raises(ValueError):
        O.emerging_newton_schulz(x.double(), 5, "quintic")
    with pytest.raises(ValueError):
        O.emerging_newton_schulz(x, 5, "custom")
    with pytest.raises(ValueError):
        O.emerging_newton_schulz(x, 5, "nope")
    with pytest.raises(ValueError):
        O.emerging_newton_schulz(torch.randn(8), 5, "quintic")


def test_ns_singular_map_is_polynomial():
    # a plausible slip (dropping the s^5 term, or using s^2) must fail this
    s = torch.tensor([0.0, 0.1, 0.5, 1.0], dtype=torch.float64)
    a, b, c = 3.4445, -4.7750, 2.0315
    want = a * s + b * s ** 3 + c * s ** 5
    assert torch.allclose(O.ns_singular_value_map(s, [(a, b, c)]), want, atol=1e-14)
    assert O.ns_singular_value_map(torch.tensor([1.0]), [(a, b, c)]).item() == pytest.approx(a + b + c)


def test_ns_singular_value_band():
    # bands of the five-step maps for inputs s in [0.01, 1], computed in exact scalar arithmetic
    s = torch.linspace(0.01, 1.0, 20001, dtype=torch.float64)
    for table, lo, hi in [("simple", 0.6818, 1.1344), ("quintic", 0.9778, 1.0318)]:
        out = O.ns_singular_value_map(s, O.coefficient_schedule(table, 5))
        assert out.min().item() == pytest.approx(lo, abs=2e-3)
        assert out.max().item() == pytest.approx(hi, abs=2e-3)


def test_ns_transpose_and_scale_invariance_and_batch():
    G = torch.randn(3, 16, 40)
    c = O.coefficient_schedule("quintic", 5)
    out = O.newton_schulz(G, c, 1e-7, storage="fp32")
    # tall input = transpose of the wide result
    outT = O.newton_schulz(G.mT.contiguous(), c, 1e-7, storage="fp32")
    assert torch.allclose(outT, out.mT, atol=1e-5)
    # positive scaling by a power of two does not change the result (up to eps)
    out2 = O.newton_schulz(G * 8.0, c, 1e-7, storage="fp32")
    assert torch.allclose(out2, out, atol=1e-5)
    # each matrix of a batch equals its own 2-D result (per-matrix norm)
    for i in range(3):
        assert torch.allclose(O.newton_schulz(G[i], c, 1e-7, storage="fp32"), out[i], atol=1e-5)


def test_ns_equivariance_and_zero_rows():
    G = torch.randn(12, 20)
    G[3] = 0
    c = O.coefficient_schedule("simple", 5)
    out = O.newton_schulz(G, c, 1e-7, storage="fp32")
    assert torch.all(out[3] == 0)
    perm = torch.randperm(12)
    outp = O.newton_schulz(G[perm], c, 1e-7, storage="fp32")
    assert torch.allclose(outp, out[perm], atol=1e-5)
    assert torch.all(O.newton_schulz(torch.zeros(4, 8), c, 1e-7, storage="fp32") == 0)


def test_ns_eps_modes():
    G = torch.randn(8, 16)
    c = O.coefficient_schedule("simple", 1)
    big = 10.0  # eps much larger than the norm: the two modes differ by a known factor
    n = G.to(torch.bfloat16).float().norm().item()
    add = O.newton_schulz(G, [(1.0, 0.0, 0.0)], big, eps_mode="add", storage="fp32")
    clamp = O.newton_schulz(G, [(1.0, 0.0, 0.0)], big, eps_mode="clamp", storage="fp32")
    assert torch.allclose(add, G.to(torch.bfloat16).float() / (n + big), rtol=1e-6)
    assert torch.allclose(clamp, G.to(torch.bfloat16).float() / max(n, big), rtol=1e-6)
    del c


@pytest.mark.parametrize("table,storage,bar", [
    ("quintic", "bf16_gemm", 1e-2), ("simple", "bf16_gemm_bsplit", 1e-2),
    ("quintic", "bf16_eager", 2e-2), ("simple", "bf16_eager", 4e-2),
    ("quintic", "f16_gemm", 4e-3), ("simple", "f16_gemm", 4e-3), ("msign", "f16_gemm", 4e-3),
])
def test_ns_bf16_modes_close_to_fp32(table, storage, bar):
    g = torch.Generator().manual_seed(5)
    G = torch.randn(128, 512, generator=g)
    c = O.coefficient_schedule(table, 5)
    ref = O.newton_schulz(G, c, 1e-7, storage="fp32")
    got = O.newton_schulz(G, c, 1e-7, storage=storage).float()
    assert got.dtype == torch.float32 and (got - ref).norm() / ref.norm() < bar


def test_gram_tail_is_the_same_map():
    """The last two iterations on the Gram side, X_N = (P_N P_{N-1}) X_{N-2} with A_{N-1} = P_{N-1} A_{N-2} P_{N-1} and
    P = aI + bA + cA^2, against two plain iterations in fp64 (a transposed factor, a wrong power of P or the wrong
    coefficient row in P_N fails this), and the storage models with and without it against the fp32 run."""
    g = torch.Generator().manual_seed(21)
    X = torch.randn(12, 40, generator=g, dtype=torch.float64)
    X = X / X.norm()
    (a1, b1, c1), (a2, b2, c2) = O.QUINTIC[3], O.QUINTIC[4]
    plain = X
    for a, b, c in ((a1, b1, c1), (a2, b2, c2)):
        A = plain @ plain.mT
        plain = a * plain + (b * A + c * (A @ A)) @ plain
    eye = torch.eye(12, dtype=torch.float64)
    A = X @ X.mT
    P1 = a1 * eye + b1 * A + c1 * (A @ A)
    A2 = (P1 @ A) @ P1
    P2 = a2 * eye + b2 * A2 + c2 * (A2 @ A2)
    assert torch.allclose((P2 @ P1) @ X, plain, rtol=1e-12, atol=1e-14)
    G = torch.randn(96, 320, generator=g)          # n >= 2m: the models take the Gram-side tail
    for table, storage, bar in (("quintic", "bf16_gemm", 6e-3), ("simple", "f16_gemm", 4e-3), ("quintic", "f16_gemm", 4e-3)):
        c = O.coefficient_schedule(table, 5)
        ref = O.newton_schulz(G, c, 1e-7, storage="fp32")
        with_tail = O.newton_schulz(G, c, 1e-7, storage=storage, gram_tail=True).float()
        without = O.newton_schulz(G, c, 1e-7, storage=storage, gram_tail=False).float()
        e1 = ((with_tail - ref).norm() / ref.norm()).item()
        e0 = ((without - ref).norm() / ref.norm()).item()
        assert e1 < bar and e1 < 1.15 * e0 + 2e-4, (table, storage, e1, e0)
        assert not torch.equal(with_tail, without)
    # a large `a` in the last rows (no a*I inside B there) or fewer than three iterations: no tail
    big = [(3.0, -3.2, 1.2), (2.0, -1.5, 0.5), (5.0, -3.0, 0.5)]
    assert torch.equal(O.newton_schulz(G, big, 1e-7, storage="bf16_gemm"),
                       O.newton_schulz(G, big, 1e-7, storage="bf16_gemm", gram_tail=False))
    two = O.coefficient_schedule("quintic", 2)
    assert torch.equal(O.newton_schulz(G, two, 1e-7, storage="f16_gemm", gram_tail=True),
                       O.newton_schulz(G, two, 1e-7, storage="f16_gemm", gram_tail=False))
    # default: the bfloat16 model takes it, the half model does not
    c = O.coefficient_schedule("quintic", 5)
    assert torch.equal(O.newton_schulz(G, c, 1e-7, storage="bf16_gemm"), O.newton_schulz(G, c, 1e-7, storage="bf16_gemm", gram_tail=True))
    assert torch.equal(O.newton_schulz(G, c, 1e-7, storage="f16_gemm"), O.newton_schulz(G, c, 1e-7, storage="f16_gemm", gram_tail=False))


def test_msign_contract():
    G = torch.randn(16, 48)
    with pytest.raises(ValueError):
        O.msign(G.to(torch.bfloat16), 5)
    with pytest.raises(ValueError):
        O.msign(torch.randn(4), 5)
    out = O.msign(G, 5)
    assert out.dtype == torch.bfloat16 and out.shape == G.shape
    # normalisation happens in fp32 BEFORE the bf16 cast, with clamp semantics
    Gn = G / G.norm().clamp_min(1e-7)
    want = _svd_closed_form(Gn, O.coefficient_schedule("msign", 5), 0.0)
    # |Gn|_F after bf16 rounding is 1 up to 2^-9, which the closed form renormalises; allow it
    got = O.msign(G, 5, storage="fp32").double()
    assert (got - want).norm() / want.norm() < 5e-3
    assert O.coefficient_schedule("msign", 10)[9] == O.POLAR_EXPRESS_MSIGN[7]


def test_coefficient_tables():
    assert O.coefficient_schedule("simple", 3) == [(3.4445, -4.7750, 2.0315)] * 3
    assert O.coefficient_schedule("quintic", 5)[0] == (4.0848, -6.8946, 2.9270)
    assert O.coefficient_schedule("quintic", 5)[4] == (2.8366, -3.0525, 1.2012)
    assert O.coefficient_schedule("polar_express", 9)[8] == O.POLAR_EXPRESS[0]
    # slope at zero = product of the a's
    assert math.prod(r[0] for r in O.coefficient_schedule("simple", 5)) == pytest.approx(484.9, rel=1e-3)
    assert math.prod(r[0] for r in O.coefficient_schedule("quintic", 5)) == pytest.approx(492.7, rel=1e-3)
    with pytest.raises(ValueError):
        O.coefficient_schedule("nope", 5)


def test_momentum_closed_form():
    G = torch.randn(6, 10)
    mu = 0.9
    M = torch.zeros_like(G)
    for k in range(1, 6):
        U = O.muon_pre_orthogonalize(G, M, mu, nesterov=True)
        geo = (1 - mu ** k) / (1 - mu)
        assert torch.allclose(M, G * geo, rtol=1e-5)
        assert torch.allclose(U.float(), (G * (mu * geo + 1)).to(torch.bfloat16).float(), rtol=1e-2)
        assert U.dtype == torch.bfloat16
    M = torch.zeros_like(G)
    U = O.muon_pre_orthogonalize(G, M, mu, nesterov=False)
    assert torch.equal(U, M.to(torch.bfloat16))
    # first nesterov step from zero state is (1+mu) G
    M = torch.zeros_like(G)
    U = O.muon_pre_orthogonalize(G, M, mu, nesterov=True)
    assert torch.allclose(U.float(), ((1 + mu) * G).to(torch.bfloat16).float())


def test_adjust_lr_and_scale_factors():
    assert O.adjust_lr(0.02, (5632, 2048), "spectral_norm") == pytest.approx(0.02 * math.sqrt(2.75))
    assert O.adjust_lr(0.02, (2048, 5632), "clip_norm") == pytest.approx(0.02)
    assert O.adjust_lr(0.02, (5632, 2048), "clip_norm") == pytest.approx(0.02 * math.sqrt(2.75))
    assert O.adjust_lr(0.02, (64, 512, 2048), "rms_norm") == pytest.approx(0.02 * 0.2 * math.sqrt(2048))
    assert O.adjust_lr(0.02, (64, 8, 4), "spectral_norm", flatten=True) == pytest.approx(0.02 * math.sqrt(2.0))
    assert O.adjust_lr(0.02, (3, 3), None) == 0.02
    with pytest.raises(ValueError):
        O.adjust_lr(0.02, (3, 3), "bad")
    assert O.muon_scale_factor(8, 2, "shape_scaling") == 2.0
    assert O.muon_scale_factor(2, 8, "shape_scaling") == 1.0
    assert O.muon_scale_factor(100, 400, "align_adamw_rms") == pytest.approx(4.0)
    assert O.muon_scale_factor(8, 2, "spectral_mup") == 2.0
    with pytest.raises(ValueError):
        O.muon_scale_factor(1, 1, "bad")


def test_plain_update_and_cautious_truth_table():
    X = torch.tensor([[1.0, -1.0, 2.0, 0.0, -3.0]])
    U = torch.tensor([[1.0, 1.0, -1.0, 5.0, 0.0]])
    lr, alr, wd = 0.1, 0.3, 0.5
    Y = X.clone()
    O.muon_post_orthogonalize(Y, U, lr, alr, wd, cautious=False)
    assert torch.allclose(Y, X * (1 - lr * wd) - alr * U)
    Y = X.clone()
    O.muon_post_orthogonalize(Y, U, lr, alr, wd, cautious=True)
    mask = torch.tensor([[1.0, 0.0, 0.0, 1.0, 1.0]])  # sign(x*u) >= 0 decays, zeros included
    assert torch.allclose(Y, X - lr * wd * X * mask - alr * U)


@pytest.mark.parametrize("wd,cautious", [(0.0, False), (0.1, False), (0.1, True)])
def test_muonh_invariants(wd, cautious):
    X = torch.randn(24, 40) * 0.02
    U = torch.randn(24, 40)
    lr, eps = 0.02, 1e-8
    Y = X.clone()
    O.muonh_post_orthogonalize(Y, U, lr, wd, eps, cautious)
    Xd = X.clone()
    O._weight_decay_(Xd, U, lr, wd, cautious)
    # norm preserved (norm after weight decay)
    assert Y.norm().item() == pytest.approx(Xd.norm().item(), rel=1e-5)
    # direction: Y parallel to Xd - lr*(|Xd|/|U|) U
    D = Xd - lr * (Xd.norm() / U.norm()) * U
    cos = (Y * D).sum() / (Y.norm() * D.norm())
    assert cos.item() == pytest.approx(1.0, abs=1e-6)
    # expansion of the intermediate norm
    s = lr * Xd.norm() / U.norm()
    want_sq = Xd.norm() ** 2 - 2 * s * (Xd * U).sum() + s ** 2 * U.norm() ** 2
    assert (D.norm() ** 2).item() == pytest.approx(want_sq.item(), rel=1e-5)
    # fp64 restatement agrees
    Y64 = O.muonh_post_fp64(X, U, lr, wd, eps, cautious)
    assert torch.allclose(Y.double(), Y64, rtol=1e-4, atol=1e-7)


def test_muonh_zero_update_and_whole_tensor_norm():
    X = torch.randn(4, 6, 8)
    Y = X.clone()
    O.muonh_post_orthogonalize(Y, torch.zeros_like(X), 0.02, 0.0, 1e-8)
    assert torch.allclose(Y, X, rtol=1e-6)
    # a 3-D tensor is renormalised as ONE tensor, not per matrix
    U = torch.randn(4, 6, 8)
    Y = X.clone()
    O.muonh_post_orthogonalize(Y, U, 0.5, 0.0, 1e-8)
    assert Y.norm().item() == pytest.approx(X.norm().item(), rel=1e-5)
    per = [abs(Y[i].norm().item() / X[i].norm().item() - 1) for i in range(4)]
    assert max(per) > 1e-3


def test_muonh_bf16_reference_semantics_close_to_fp64():
    X = (torch.randn(256, 64) * 0.02).to(torch.bfloat16)
    U = torch.randn(256, 64).to(torch.bfloat16)
    Y = X.clone()
    O.muonh_post_orthogonalize(Y, U, 0.02, 0.0, 1e-8)
    Y64 = O.muonh_post_fp64(X, U, 0.02, 0.0, 1e-8)
    rel = (Y.double() - Y64).norm() / Y64.norm()
    assert rel < 5e-3
    # and a no-op "update" sits at ~lr: W parity alone cannot see a missing step
    assert ((X.double() - Y64).norm() / Y64.norm()).item() == pytest.approx(0.02, rel=0.1)


def test_flatten_policy_and_batches():
    X = torch.randn(2, 3, 4, 5)
    v, shape = O.newton_schulz_flatten_policy(X, flatten=True)
    assert v.shape == (2, 60) and shape == X.shape
    v, _ = O.newton_schulz_flatten_policy(X, flatten=False)
    assert v.shape == (6, 4, 5)
    v, _ = O.newton_schulz_flatten_policy(X[0], flatten=False)
    assert v.shape == (3, 4, 5)
    keys = ["a", "b", "a", "a", "b"]
    assert O.create_param_batches(keys, 2) == [[0, 2], [3], [1, 4]]
    assert O.create_param_batches(keys, 1) == [[0], [2], [3], [1], [4]]


def test_lit_gpt_step_first_step_equals_ns_of_grad():
    # from a zero momentum state U = (1+mu) G and NS is scale invariant
    X = torch.randn(16, 32) * 0.02
    G = torch.randn(16, 32) * 1e-3
    M = torch.zeros_like(X)
    Y = X.clone()
    O.lit_gpt_muon_step(Y, G, M, lr=0.02, mu=0.95, wd=0.0, eps=1e-8, nesterov=True,
                        adjust="spectral_norm", flatten=False, cautious=False, use_muonh=False,
                        ns_storage="fp32")
    ns = O.newton_schulz(G * 1.95, O.QUINTIC, 1e-8, storage="fp32").to(torch.bfloat16).float()
    # bf16(0.95 G + G) and bf16(1.95 G) may differ by one bf16 ulp per element: update is ~3e-3 per element
    assert torch.allclose(Y, X - 0.02 * math.sqrt(0.5) * ns, atol=3e-4)
    assert not torch.allclose(Y, X, atol=3e-4)
    assert torch.allclose(M, G)


@pytest.mark.parametrize("method", ["decoupled", "independent", "l2"])
def test_emerging_step(method):
    p = torch.randn(12, 20)
    g = torch.randn(12, 20)
    buf = torch.zeros_like(g)
    p0, g0 = p.clone(), g.clone()
    O.emerging_muon_step(p, g, buf, lr=0.1, beta=0.9, wd=0.5, nesterov=True, wd_method=method,
                         steps=5, scale_mode="spectral_mup", extra_scale=2.0, ns_storage="fp32")
    if method == "decoupled":
        pd, gd = p0 * (1 - 0.05), g0
    elif method == "independent":
        pd, gd = p0 * 0.5, g0
    else:
        pd, gd = p0, g0 + 0.5 * p0
    assert torch.allclose(buf, 0.1 * gd, rtol=1e-5, atol=1e-7)           # EMA from zero
    u = 0.1 * gd + 0.9 * buf                                           # lerp nesterov
    o = O.msign(u, 5, storage="fp32") * math.sqrt(12 / 20) * 2.0
    assert torch.allclose(p, pd - 0.1 * o, atol=1e-5)
    with pytest.raises(ValueError):
        O.emerging_muon_step(torch.randn(4), torch.randn(4), torch.zeros(4), lr=0.1, beta=0.9, wd=0.0,
                             nesterov=False, wd_method=method, steps=5, scale_mode="spectral_mup",
                             extra_scale=1.0)


# ---------------------------------------------------------------------------
# scalar optimizers of the non-matrix groups (oracle/scalar_oracle.py)
# ---------------------------------------------------------------------------
def test_scalar_oracle_closed_forms():
    from oracle import scalar_oracle as S
    g = torch.randn(7, 5)
    x0 = torch.randn(7, 5)
    # AdamW, first step from zero moments: M/bias1 = g, sqrt(V/bias2) = |g|  =>  x <- x(1-lr wd) - lr g/(|g|+eps)
    x, m, v = x0.clone(), torch.zeros(7, 5), torch.zeros(7, 5)
    S.adamw_update_foreach([x], [g], [m], [v], 0.1, 0.9, 0.95, 0.5, 1, 1e-8)
    assert torch.allclose(x, x0 * (1 - 0.05) - 0.1 * g / (g.abs() + 1e-8), atol=1e-6)
    assert torch.allclose(m, 0.1 * g) and torch.allclose(v, 0.05 * g * g)
    # Lion: update is -lr*sign(lerp), momentum is the beta2 EMA
    x, m = x0.clone(), torch.full((7, 5), 0.3)
    S.lion_update_foreach([x], [g], [m], 0.1, 0.9, 0.99, 0.0)
    assert torch.allclose(x, x0 - 0.1 * torch.sign(0.9 * 0.3 + 0.1 * g), atol=1e-7)
    assert torch.allclose(m, 0.99 * 0.3 + 0.01 * g, atol=1e-7)
    # cautious decay only where x*u >= 0
    x, m = torch.tensor([[1.0, -1.0]]), torch.zeros(1, 2)
    S.lion_update_foreach([x], [torch.tensor([[1.0, 1.0]])], [m], 0.1, 0.9, 0.99, 0.5, cautious_wd=True)
    assert torch.allclose(x, torch.tensor([[1.0 - 0.05 - 0.1, -1.0 - 0.1]]))
    # hyperball AdamW: norm preserved, moves along -direction
    x, m, v = x0.clone(), torch.zeros(7, 5), torch.zeros(7, 5)
    S.hyperball_adamw_update_foreach([x], [g], [m], [v], 0.1, 0.9, 0.95, 0.0, 1, 1e-8)
    assert x.norm().item() == pytest.approx(x0.norm().item(), rel=1e-5)
    d = g / (g.abs() + 1e-8)
    want = x0 - 0.1 * x0.norm() / d.norm() * d
    want = want * x0.norm() / want.norm()
    assert torch.allclose(x, want, atol=1e-5)
