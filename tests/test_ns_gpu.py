"""Parity of the HIP Newton-Schulz path (through the C ABI) against the CPU oracle.

Bar: relative Frobenius error <= 1e-2 against the oracle run in fp32 on the same bf16 inputs
(the tolerance the path's contract states), and singular values inside the band of the
coefficient table.
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


def _randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


@pytest.fixture(scope="module")
def ns(gpu_device):
    import archscale_amd.optim.newton_schulz_hip as H
    return H


@pytest.mark.parametrize("shape", [(128, 256), (256, 128), (512, 2048), (2048, 256), (768, 1024), (2, 256, 512),
                                   (3, 384, 128)])
@pytest.mark.parametrize("table", ["quintic", "simple"])
def test_ns_matches_fp32_oracle(ns, gpu_device, shape, table):
    print("case", shape, table, flush=True)
    G = _randn(shape, 11 + sum(shape))
    coeffs = O.coefficient_schedule(table, 5)
    prec = "bsplit" if table == "simple" else "bf16"
    got = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, prec=prec)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and got.shape == G.shape
    want = O.newton_schulz(G, coeffs, 1e-7, storage="fp32")
    err = _rel(got, want)
    print("rel err", err, flush=True)
    assert err <= NS_TOL
    # the modelled rounding points (one per GEMM epilogue) explain the error: same order of magnitude
    model = O.newton_schulz(G, coeffs, 1e-7, storage="bf16_gemm_bsplit" if prec == "bsplit" else "bf16_gemm")
    assert _rel(got, model.float()) <= NS_TOL


def test_config1_single_matrix(ns, gpu_device):
    """One 512x2048 gradient, N(0,1) from seed, constant (3.4445,-4.7750,2.0315) row, eps 1e-7."""
    G = _randn((512, 2048), 1235)
    got = ns.zeropower_via_newtonschulz5_legacy(G.to(gpu_device), steps=5)
    want = O.newton_schulz(G, O.coefficient_schedule("simple", 5), 1e-7, storage="fp32")
    assert _rel(got, want) <= NS_TOL
    # singular values land in the band of the five-step map for this spectrum
    s_in = torch.linalg.svdvals(G.double()) / G.double().norm()
    band = O.ns_singular_value_map(s_in, O.coefficient_schedule("simple", 5))
    s_out = torch.linalg.svdvals(got.double().cpu())
    assert s_out.min() >= band.min() - 0.02 and s_out.max() <= band.max() + 0.02
    # and what the reference's own CPU path (bf16 eager) produces is no closer to fp32 than we are
    eager = O.newton_schulz(G, O.coefficient_schedule("simple", 5), 1e-7, storage="bf16_eager")
    assert _rel(got, want) <= _rel(eager.float(), want)


def test_production_hook_names(ns, gpu_device):
    G = _randn((256, 512), 3).to(gpu_device)
    a = ns.zeropower_via_newtonschulz5(G, epsilon=torch.tensor(1e-8))
    b = ns.newton_schulz_triton(G, epsilon=1e-8)
    assert torch.equal(a, b)
    want = O.newton_schulz(G.cpu(), O.QUINTIC, 1e-8, storage="fp32")
    assert _rel(a, want) <= NS_TOL


def test_transpose_batch_and_zero(ns, gpu_device):
    G = _randn((3, 128, 320), 5)
    out = ns.newton_schulz(G.to(gpu_device))
    outT = ns.newton_schulz(G.mT.contiguous().to(gpu_device))
    # the tall problem iterates the same X: results are exact transposes
    assert torch.equal(outT, out.mT)
    for i in range(3):
        assert torch.equal(ns.newton_schulz(G[i].to(gpu_device)), out[i])
    z = ns.newton_schulz(torch.zeros(64, 192, dtype=torch.bfloat16, device=gpu_device))
    assert torch.all(z == 0)
    # zeroed rows stay exactly zero
    G2 = _randn((256, 512), 6)
    G2[7] = 0
    G2[200] = 0
    o2 = ns.newton_schulz(G2.to(gpu_device))
    assert torch.all(o2[7] == 0) and torch.all(o2[200] == 0)


@pytest.mark.parametrize("shape", [(100, 200), (130, 77), (2, 65, 300), (257, 1000)])
def test_ragged_shapes(ns, gpu_device, shape):
    """Extents that are no multiple of any tile: padding must not leak into the result."""
    G = _randn(shape, 17 + sum(shape))
    got = ns.newton_schulz(G.to(gpu_device))
    want = O.newton_schulz(G, O.QUINTIC, 1e-7, storage="fp32")
    assert _rel(got, want) <= NS_TOL


def test_fp32_input_and_clamp_mode(ns, gpu_device):
    g = torch.Generator().manual_seed(9)
    G = torch.randn(192, 448, generator=g)
    coeffs = O.coefficient_schedule("msign", 5)
    # the polar-express table starts with a steep row (8.2, -22.9, 16.5): it needs the B split to stay under 1e-2
    got = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, eps_mode="clamp", cast_input_first=False, prec="bsplit")
    want = O.msign(G, 5, storage="fp32")
    assert _rel(got, want) <= NS_TOL
    assert _rel(got, want) <= _rel(O.msign(G, 5).float(), want)  # and beats the reference's own bf16 path
    # strided input (a column slice) is read in place through its leading dimension
    big = _randn((128, 512), 10).to(gpu_device)
    view = big[:, :256]
    assert torch.equal(ns.newton_schulz(view), ns.newton_schulz(view.contiguous()))


def test_in_place_out(ns, gpu_device):
    G = _randn((4, 256, 384), 12).to(gpu_device)
    ref = ns.newton_schulz(G)
    buf = G.clone()
    ns.newton_schulz(buf, out=buf)
    assert torch.equal(buf, ref)


def test_grouped_equals_separate(ns, gpu_device):
    """All shape classes in one grouped call (one launch per product over every class) give bit-identical
    results to one call per class; mixes both tile configurations, tall and wide, 2-D and 3-D, fp32 input."""
    ins = [_randn((3, 256, 768), 31), _randn((640, 128), 32), _randn((2, 128, 1024), 33), _randn((1024, 1024), 34),
           torch.randn(100, 200, generator=torch.Generator().manual_seed(35))]
    ins = [t.to(gpu_device) for t in ins]
    for prec, coeffs in (("bf16", O.QUINTIC), ("bsplit", O.coefficient_schedule("simple", 5))):
        sep = [ns.newton_schulz(t, coeffs, 1e-7, prec=prec) for t in ins]
        grp = ns.newton_schulz_grouped(ins, coeffs, 1e-7, prec=prec)
        for a, b in zip(sep, grp):
            assert torch.equal(a, b)
    # in place, and more problems than fit one launch (9 > 8)
    many = [_randn((128, 128 * (i + 1)), 40 + i).to(gpu_device) for i in range(9)]
    want = [ns.newton_schulz(t) for t in many]
    ns.newton_schulz_grouped(many, outs=many)
    for a, b in zip(want, many):
        assert torch.equal(a, b)
    assert ns.newton_schulz_grouped([]) == []


def test_syrk_products(ns, gpu_device):
    X = _randn((2, 192, 320), 21, 0.05).to(gpu_device)
    A = ns.ns_line_1(X)
    want = (X.float() @ X.float().mT)
    assert _rel(A, want) < 4e-3 and torch.equal(A, A.mT)
    B = ns.ns_line_2(A, alpha=2.0315, beta=-4.775)
    wantB = 2.0315 * (A.float() @ A.float()) - 4.775 * A.float()
    assert _rel(B, wantB) < 4e-3 and torch.equal(B, B.mT)
    with pytest.raises(ValueError):
        ns.ns_line_2(X, 1.0, 1.0)
    D = ns.tsyrk_ex(X[0], A[1], alpha=0.5, beta=2.0)
    assert _rel(D, 0.5 * (X[0].float() @ X[0].float().T) + 2.0 * A[1].float()) < 4e-3


def test_errors(ns, gpu_device):
    with pytest.raises(ValueError):
        ns.newton_schulz(torch.zeros(8, device=gpu_device))
    from archscale_amd._lib import MuonLibraryError
    with pytest.raises(MuonLibraryError):
        ns.newton_schulz(torch.zeros(8, 8))
    assert math.isfinite(1.0)


def test_bsplit_tail(gpu_device):
    """Keeping B as a hi+lo pair only in the last t iterations: t = iters is the full split bit for bit, t = 3 stays at
    the accuracy of the full split for the constant-row table, and unknown flag bits are rejected."""
    import archscale_amd.optim.newton_schulz_hip as H
    from archscale_amd import _lib
    g = torch.Generator().manual_seed(31)
    G = torch.randn(3, 384, 1024, generator=g).to(torch.bfloat16)
    Gd = G.to(gpu_device)
    coeffs = O.coefficient_schedule("simple", 5)
    full = H.newton_schulz(Gd, coeffs, 1e-7, prec="bsplit")
    assert torch.equal(H.newton_schulz(Gd, coeffs, 1e-7, prec="bsplit", bsplit_tail=5), full)
    assert torch.equal(H.newton_schulz(Gd, coeffs, 1e-7, prec="bsplit", bsplit_tail=9), full)
    want = O.newton_schulz(G, coeffs, 1e-7, storage="fp32")
    e_full, e3, e0 = (_rel(x, want) for x in (full, H.newton_schulz(Gd, coeffs, 1e-7, prec="bsplit", bsplit_tail=3),
                                              H.newton_schulz(Gd, coeffs, 1e-7, prec="bf16")))
    assert e3 <= 1e-2 and e3 <= 1.1 * e_full and e0 > e3
    assert torch.equal(H.newton_schulz(Gd, coeffs, 1e-7, prec="bf16", bsplit_tail=3), H.newton_schulz(Gd, coeffs, 1e-7, prec="bf16"))
    assert H.BSPLIT_TAIL == 3
    with pytest.raises(ValueError):
        _lib.ns_bsplit_tail(256)
    ws = _lib.workspace(gpu_device, 1 << 20)
    abc = _lib.abc_array(coeffs)
    st = _lib.lib().muon_ns_batched(Gd.data_ptr(), 0, 384 * 1024, 1024, full.data_ptr(), 384 * 1024, 1024, 3, 384, 1024, abc, 5,
                                    1e-7, 0, 1, 1 << 20, ws.data_ptr(), ws.numel(), 0)
    assert st < 0


@pytest.mark.parametrize("shape", [(256, 512), (384, 200), (100, 36)])
def test_single_step_without_normalisation(gpu_device, shape):
    """newton_schulz_step_tsyrk: one iteration on the matrix as it is (wide and tall inputs; the tall one is iterated
    transposed inside, which is the same polynomial)."""
    from archscale_amd.emerging.muon_utils import newton_schulz_step_tsyrk
    a, b, c = 3.4445, -4.7750, 2.0315
    X = (_randn(shape, 5).float() / max(shape) ** 0.5 * 0.6).to(torch.bfloat16)   # singular values below ~1.2
    got = newton_schulz_step_tsyrk(X.to(gpu_device), a, b, c)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and got.shape == X.shape
    Xd = X.double()
    A = Xd @ Xd.T
    want = a * Xd + (b * A + c * A @ A) @ Xd
    assert _rel(got, want) <= 4e-3          # one bf16 rounding of A, of B and of the result
    with pytest.raises(ValueError):
        newton_schulz_step_tsyrk(X.float().to(gpu_device), a, b, c)


@pytest.mark.parametrize("shape", [(2304, 2560), (3328, 2816), (3584, 5632), (2560, 2560)])
def test_wide_grids_whose_sides_are_not_multiples_of_four_tiles(gpu_device, shape):
    """The product X' = (B + aI) X walks a grid of more than 8 tile rows (short side above 2048) in blocks of 4 x 4 tiles;
    the last block row and the last block of a row are narrower when a side is no multiple of four tiles (grids of
    9 x 10, 11 x 13, 14 x 22 and 10 x 10 tiles here; the symmetric products of the same step walk triangles of side 9,
    11, 14 and 10).
    A tile left out or written twice shows as an error of order one against the fp64 iteration."""
    from archscale_amd.emerging.muon_utils import newton_schulz_step_tsyrk
    print("case", shape, flush=True)
    a, b, c = 3.4445, -4.7750, 2.0315
    X = (_randn(shape, 15).float() / max(shape) ** 0.5 * 0.6).to(torch.bfloat16).to(gpu_device)
    got = newton_schulz_step_tsyrk(X, a, b, c)
    torch.cuda.synchronize()
    Xd = X.double()
    A = Xd @ Xd.T
    want = a * Xd + (b * A + c * A @ A) @ Xd
    assert _rel(got, want) <= 4e-3
    err = (got.double() - want).abs()
    assert err.max().item() <= 0.05 * want.abs().max().item()   # no tile missing: every entry is close, not just the norm


def test_quartered_tail_matches_other_grids(ns, gpu_device):
    """A launch whose last round holds few tiles hands them to the 128x128 configuration as quadrants. Which tiles
    those are depends on the batch, the arithmetic of a tile does not: the same matrix gives the same bits alone
    (small-call path), in a batch of 8 (tail of 32 tiles) and in a batch of 16 (tail of 64 tiles)."""
    G = _randn((16, 2048, 2048), 91).to(gpu_device)
    all16 = ns.newton_schulz(G)
    first8 = ns.newton_schulz(G[:8])
    alone = ns.newton_schulz(G[3])
    torch.cuda.synchronize()
    assert torch.equal(all16[:8], first8)
    assert torch.equal(all16[3], alone)
    from oracle import muon_oracle as O
    want = O.newton_schulz(G[3].cpu(), O.coefficient_schedule("quintic", 5), 1e-7, storage="fp32")
    assert _rel(alone, want) <= NS_TOL


@pytest.mark.parametrize("table,prec", [("quintic", "bf16"), ("simple", "bsplit"), ("msign", "bsplit")])
def test_diagonal_fold_and_addend_agree(ns, gpu_device, table, prec):
    """By default an iteration after the first with |a| <= 4.2 stores B + aI and computes X' = (B + aI) X; diag_fold=False keeps aX as
    an addend. Both stay within the bar of the fp32 run (their rounding errors are independent of each other)."""
    G = _randn((2, 512, 1280), 23)
    coeffs = O.coefficient_schedule(table, 5)
    kw = dict(prec=prec, bsplit_tail=3 if prec == "bsplit" else 0, eps_mode="clamp" if table == "msign" else "add")
    folded = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, **kw)
    addend = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, diag_fold=False, **kw)
    torch.cuda.synchronize()
    for b in range(2):
        want = O.newton_schulz(G[b], coeffs, 1e-7, storage="fp32", eps_mode=kw["eps_mode"])
        assert _rel(folded[b], want) <= NS_TOL
        assert _rel(addend[b], want) <= NS_TOL
        assert _rel(folded[b], addend[b]) <= NS_TOL
    assert not torch.equal(folded, addend)      # the flag reaches the kernels


def test_dominant_singular_value(ns, gpu_device):
    """A matrix with one dominant singular value (a 30x rank-one spike on Gaussian noise): after the normalisation the
    rest of the spectrum, and with it A = XX^T, is tiny in the first iteration, and rounding the NORMALISED input to
    bf16 alone would move the result by 5e-2 (the reference's eager bf16 path is 8.5e-2 away from the fp32 run). The
    library keeps a bf16 input exactly and applies the factor in the first iteration's epilogues, so the result is
    checked against the fp32 run itself, and against an fp64 iteration from the same input."""
    g = torch.Generator().manual_seed(31)
    G = torch.randn(512, 2048, generator=g) + 30.0 * torch.randn(512, 1, generator=g) @ torch.randn(1, 2048, generator=g)
    coeffs = O.coefficient_schedule("quintic", 5)

    def fp64_iteration(X):
        for a, b, c in coeffs:
            A = X @ X.T
            X = a * X + (b * A + c * A @ A) @ X
        return X

    Gb = G.to(torch.bfloat16)
    exact = fp64_iteration(Gb.double() / (Gb.double().norm() + 1e-7))
    want = O.newton_schulz(Gb, coeffs, 1e-7, storage="fp32")
    for prec, bar in (("bf16", 0.75 * NS_TOL), ("f16", 4e-3)):
        for kw in (dict(), dict(diag_fold=False)):
            got = ns.newton_schulz(Gb.to(gpu_device), coeffs, 1e-7, prec=prec, **kw)
            torch.cuda.synchronize()
            print("rel err", prec, kw, _rel(got, exact), _rel(got, want), flush=True)
            assert _rel(got, exact) <= bar and _rel(got, want) <= bar
    # fp32 input, normalised in fp32 and rounded once (the order of msign): which way an entry rounds depends on the last
    # bit of the norm, and this input amplifies the rounding of the normalised copy tenfold, so only the order of
    # magnitude is fixed here
    rounded = fp64_iteration((G / (G.norm() + 1e-7)).to(torch.bfloat16).double())
    got = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, cast_input_first=False)
    assert _rel(got, rounded) <= 3e-2


@pytest.mark.parametrize("prec", ["bf16", "f16"])
def test_power_of_two_scaling_is_exact(ns, gpu_device, prec):
    """A bf16 input goes into the workspace times a power of two and the rest of 1/|X| is applied in fp32, so a matrix
    times 2^k (exact in bf16) must give the same bits as the matrix itself when eps is zero, for tiny and huge k."""
    G = _randn((200, 330), 77).to(torch.bfloat16)
    coeffs = O.coefficient_schedule("quintic", 5)
    base = ns.newton_schulz(G.to(gpu_device), coeffs, 0.0, prec=prec)
    assert _rel(base, O.newton_schulz(G, coeffs, 0.0, storage="fp32")) <= (4e-3 if prec == "f16" else NS_TOL)
    for k in (-40, -13, 9, 30):
        got = ns.newton_schulz((G.float() * 2.0 ** k).to(torch.bfloat16).to(gpu_device), coeffs, 0.0, prec=prec)
        assert torch.equal(got, base), k


def test_grouped_call_with_mixed_input_kinds(ns, gpu_device):
    """One grouped call over a bf16 tensor (kept exactly, factor deferred) and an fp32 tensor that is normalised before
    it is rounded (not deferrable): in bf16 storage each problem takes its own route, with the half workspace the whole
    call takes the common one; every result stays within its bar of the fp32 run."""
    coeffs = O.coefficient_schedule("quintic", 5)
    a = _randn((2, 128, 320), 5).to(torch.bfloat16)
    b = _randn((192, 96), 6)
    want_a = O.newton_schulz(a, coeffs, 1e-7, storage="fp32")
    want_b = O.newton_schulz(b, coeffs, 1e-7, storage="fp32")   # the oracle rounds first; the difference is one rounding
    for prec, bar in (("bf16", NS_TOL), ("f16", 4e-3)):
        got_a, got_b = ns.newton_schulz_grouped([a.to(gpu_device), b.to(gpu_device)], coeffs, 1e-7, prec=prec,
                                                cast_input_first=False)
        torch.cuda.synchronize()
        print(prec, _rel(got_a, want_a), _rel(got_b, want_b), flush=True)
        assert _rel(got_a, want_a) <= bar and _rel(got_b, want_b) <= NS_TOL


def test_random_shapes_strides_and_modes(ns, gpu_device):
    """Seeded sweep over shapes that are no multiple of anything, strided inputs, both input dtypes, all coefficient
    tables, split tails, the no-fold flag and grouped calls of mixed size: every result within the bar of the fp32 run,
    grouped results identical to single calls."""
    import random
    rng = random.Random(20251)
    # the constant and polar-express tables run in the half-precision workspace, which is what the package itself uses for
    # them; "simple_bsplit" keeps the bf16 hi+lo pair (a diagnostic mode) in the sweep for its code paths
    tables = {"quintic": ("bf16", 0), "simple": ("f16", 0), "msign": ("f16", 0), "simple_bsplit": ("bsplit", 3)}
    singles = []
    for case in range(14):
        rows, cols = rng.choice([1, 3, 17, 64, 100, 129, 255, 300, 513]), rng.choice([2, 31, 64, 96, 200, 257, 640, 1025])
        if rows * cols < 64:
            cols = 96
        batch = rng.choice([1, 1, 2, 3])
        table = rng.choice(list(tables))
        prec, tail = tables[table]
        dtype = rng.choice([torch.bfloat16, torch.float32])
        pad = rng.choice([0, 0, 8, 5])
        fold = rng.random() < 0.7
        print("case", case, (batch, rows, cols), table, dtype, "pad", pad, "fold", fold, flush=True)
        g = torch.Generator().manual_seed(1000 + case)
        full = torch.randn(batch, rows, cols + pad, generator=g).to(dtype)
        G = full[..., :cols]
        coeffs = O.coefficient_schedule("simple" if table == "simple_bsplit" else table, 5)
        em = "clamp" if table == "msign" else "add"
        got = ns.newton_schulz(G.to(gpu_device) if pad == 0 else full.to(gpu_device)[..., :cols], coeffs, 1e-7, eps_mode=em,
                               prec=prec, bsplit_tail=tail, diag_fold=fold)
        torch.cuda.synchronize()
        assert got.shape == G.shape and torch.isfinite(got.float()).all()
        for b in range(batch):
            want = O.newton_schulz(G[b].to(torch.bfloat16), coeffs, 1e-7, storage="fp32", eps_mode=em)
            # the contract's 1e-2 from 16 rows up; a matrix with a handful of singular values has no averaging at all
            # (emulated 3x64 with the polar-express table: 2.2e-2 in half storage, 3.9e-2 in bf16), so below that the bar is
            # 3e-2.  The hi+lo pair
            # in bf16 storage holds 1e-2 only from 256 rows up (emulated 64x64: 8.5e-3 .. 1.4e-2) and is not what the
            # package runs anywhere: below that it is checked for its code paths only, against a loose ceiling.
            small = min(rows, cols)
            if prec == "bsplit":
                bar = NS_TOL if small >= 256 else 2 * NS_TOL if small >= 64 else 0.15
            else:
                bar = NS_TOL if small >= 16 else 3 * NS_TOL
            assert _rel(got[b], want) <= bar, (case, b)
        if table == "quintic" and dtype == torch.bfloat16 and fold:
            singles.append((G.contiguous().to(gpu_device), got))
    # the quintic bf16 cases once more in ONE grouped call
    if len(singles) > 1:
        outs = ns.newton_schulz_grouped([t for t, _ in singles], O.coefficient_schedule("quintic", 5), 1e-7)
        torch.cuda.synchronize()
        for o, (_, ref) in zip(outs, singles):
            assert torch.equal(o, ref)


@pytest.mark.parametrize("shape", [(512, 2048), (2048, 512), (300, 700), (2, 129, 64), (1024, 1024)])
@pytest.mark.parametrize("table", ["quintic", "simple", "msign"])
def test_half_precision_workspace(ns, gpu_device, shape, table):
    """prec="f16": iterate, A and B in IEEE half inside the workspace, each times a power of two (input and result stay
    bfloat16). One walk per product, no hi+lo pair, and within 4e-3 of the fp32 run for every coefficient table: less
    than half the error of plain bfloat16 storage."""
    G = _randn(shape, 7 + sum(shape))
    coeffs = O.coefficient_schedule(table, 5)
    em = "clamp" if table == "msign" else "add"
    got = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, eps_mode=em, prec="f16")
    plain = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, eps_mode=em, prec="bf16", gram_tail=False)   # bf16 storage throughout
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and got.shape == G.shape
    mats = G if G.ndim == 3 else G[None]
    want = torch.stack([O.newton_schulz(x, coeffs, 1e-7, storage="fp32", eps_mode=em) for x in mats]).reshape(G.shape)
    err = _rel(got, want)
    print("rel err", err, flush=True)
    assert err <= 4e-3
    assert err <= 0.5 * _rel(plain, want)
    # the CPU model of the same rounding points (half storage, the same power-of-two factors, a*I inside B): what is
    # left between the two is the order of the fp32 sums, which flips some of the final bf16 roundings
    model = torch.stack([O.newton_schulz(x, coeffs, 1e-7, storage="f16_gemm", eps_mode=em) for x in mats]).reshape(G.shape)
    assert _rel(got, model) <= 2.5e-3


def test_half_precision_workspace_scales(ns, gpu_device):
    """The power-of-two factors keep the half-precision workspace in range for gradients of any magnitude (the input is
    normalised first) and for a large matrix, whose normalised entries (1e-4) sit at the bottom of the format."""
    coeffs = O.coefficient_schedule("simple", 5)
    base = _randn((256, 640), 3).float()
    ref = None
    for mag in (1e-12, 1.0, 1e12):
        got = ns.newton_schulz((base * mag).to(torch.bfloat16).to(gpu_device), coeffs, 1e-30, prec="f16").float().cpu()
        assert torch.isfinite(got).all()
        ref = got if ref is None else ref
        assert _rel(got, ref) <= 4e-3          # bf16(base * mag) differs from bf16(base) * mag by rounding only
    big = _randn((4096, 8192), 4).to(gpu_device)
    got = ns.newton_schulz(big, O.QUINTIC, 1e-7, prec="f16")
    torch.cuda.synchronize()
    sv = torch.linalg.svdvals(got[:, :4096].float().cpu() @ got[:, :4096].float().cpu().T + got[:, 4096:].float().cpu() @ got[:, 4096:].float().cpu().T)
    # singular values of the result squared: the production schedule lands every one of them in (0.4, 1.3)^2
    assert sv.min().item() > 0.16 and sv.max().item() < 1.7


@pytest.mark.parametrize("kind,steps", [("simple", 5), ("quintic", 5), ("quintic", 10), ("polar_express", 8),
                                        ("polar_express", 16), ("aol", 4), ("aol", 8), ("custom", 4)])
@pytest.mark.parametrize("shape", [(320, 1100), (1100, 320), (257, 257), (3, 200, 136)])
def test_emerging_newton_schulz_named_sets(gpu_device, kind, steps, shape):
    """emerging_optimizers' newton_schulz (fp32 in, fp32 out, clamp eps, named sets cycled) through the HIP path against
    the oracle's restatement iterated in fp32 on the same rounded input."""
    from archscale_amd.emerging.muon_utils import newton_schulz
    print("case", kind, steps, shape, flush=True)
    g = torch.Generator().manual_seed(17 + steps + sum(shape))
    x = torch.randn(*shape, generator=g) * 3e-2
    custom = [(3.0, -3.2, 1.2), (2.0, -1.5, 0.5)] if kind == "custom" else None
    got = newton_schulz(x.to(gpu_device), steps, kind, custom)
    torch.cuda.synchronize()
    assert got.dtype == torch.float32 and got.shape == x.shape
    want = O.emerging_newton_schulz(x, steps, kind, custom, storage="fp32")
    err = _rel(got, want)
    print("rel err", err, flush=True)
    assert err <= NS_TOL
    # no further from the fp32 run than the reference's own all-bf16 arithmetic is
    eager = O.emerging_newton_schulz(x, steps, kind, custom)
    assert err <= max(_rel(eager, want), 4e-3)
    # an explicit transpose flag (either value) changes nothing
    flipped = newton_schulz(x.to(gpu_device), steps, kind, custom, transpose=shape[-2] <= shape[-1])
    assert torch.equal(flipped, got)


@pytest.mark.parametrize("shape", [(512, 2048), (2048, 256), (320, 1100), (3, 136, 400), (256, 512), (300, 599)])
@pytest.mark.parametrize("prec,table", [("bf16", "quintic"), ("f16", "quintic"), ("f16", "simple")])
def test_gram_side_tail(ns, gpu_device, shape, prec, table):
    """The last two iterations in half storage and, for n >= 2m, on the Gram side (the default) against the same call
    with plain last iterations and against the fp32 oracle: no further from the oracle than the plain path."""
    print("case", shape, prec, table, flush=True)
    G = _randn(shape, 31 + sum(shape))
    coeffs = O.coefficient_schedule(table, 5)
    want = O.newton_schulz(G, coeffs, 1e-7, storage="fp32")
    got = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, prec=prec, gram_tail=True)
    plain = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, prec=prec, gram_tail=False)
    auto = ns.newton_schulz(G.to(gpu_device), coeffs, 1e-7, prec=prec)
    torch.cuda.synchronize()
    assert torch.equal(auto, got if prec == "bf16" else plain)      # the default: on for bf16 storage, off for half
    e1, e0 = _rel(got, want), _rel(plain, want)
    print("rel err with / without the tail", e1, e0, flush=True)
    assert e1 <= NS_TOL and e1 <= 1.1 * e0 + 2e-4
    m, n = min(shape[-2:]), max(shape[-2:])
    if n >= 2 * m or prec == "bf16":
        assert not torch.equal(got, plain)       # the default really took the other path
    else:
        assert torch.equal(got, plain)           # half workspace, n < 2m: nothing changes
    model = O.newton_schulz(G, coeffs, 1e-7, storage="f16_gemm" if prec == "f16" else "bf16_gemm", gram_tail=True)
    assert _rel(got, model.float()) <= (2.5e-3 if prec == "f16" else 6e-3)


def test_gram_side_tail_spiked_and_grouped(ns, gpu_device):
    """A gradient with a dominant direction (Gaussian plus a 30x rank-one spike), and a grouped call that mixes classes
    that take the Gram-side tail with classes that do not: every problem equals its own single call bit for bit."""
    g = torch.Generator().manual_seed(5)
    spike = (torch.randn(512, 2048, generator=g) + 30 * torch.randn(512, 1, generator=g) @ torch.randn(1, 2048, generator=g))
    spike = spike.to(torch.bfloat16)
    want = O.newton_schulz(spike, O.QUINTIC, 1e-7, storage="fp32")
    for prec, bar in (("bf16", 8e-3), ("f16", 3e-3)):
        got = ns.newton_schulz(spike.to(gpu_device), O.QUINTIC, 1e-7, prec=prec, gram_tail=True)
        plain = ns.newton_schulz(spike.to(gpu_device), O.QUINTIC, 1e-7, prec=prec, gram_tail=False)
        e1, e0 = _rel(got, want), _rel(plain, want)
        print("spike", prec, e1, e0, flush=True)
        assert e1 <= bar and e1 <= 1.1 * e0 + 2e-4
    shapes = [(2, 256, 1024), (384, 384), (640, 256), (3, 300, 700), (512, 600)]
    ins = [_randn(s, 100 + i).to(gpu_device) for i, s in enumerate(shapes)]
    for prec in ("bf16", "f16"):
        outs = ns.newton_schulz_grouped(ins, O.QUINTIC, 1e-7, prec=prec, gram_tail=True)
        torch.cuda.synchronize()
        for x, o in zip(ins, outs):
            single = ns.newton_schulz(x, O.QUINTIC, 1e-7, prec=prec, gram_tail=True)
            assert torch.equal(o, single), (prec, tuple(x.shape))
            assert _rel(o, O.newton_schulz(x.cpu(), O.QUINTIC, 1e-7, storage="fp32")) <= NS_TOL


@pytest.mark.parametrize("shape", [(1536, 8192), (8192, 1536)])
def test_k_split_of_long_reductions(ns, gpu_device, shape):
    """A matrix with few upper-triangle tiles (21 of 256 x 256) and a long reduction (K = 8192) has its A = X X^T product
    cut along K: four blocks per 128 x 128 quadrant leave fp32 partial results, the last one to arrive adds them in the
    order of the parts.  The cut is a function of the matrix's own shape, so the matrix gives the same bits alone (the
    small-call path), in a batch, in a grouped call next to other shapes, and on every repetition (which block arrives
    last changes from run to run; the sum does not); and the result is within the bar of the fp32 oracle."""
    G = _randn(shape, 77)
    Gd = G.to(gpu_device)
    want = O.newton_schulz(G, O.QUINTIC, 1e-7, storage="fp32")
    for prec, bar in (("bf16", NS_TOL), ("f16", 4e-3)):
        alone = ns.newton_schulz(Gd, O.QUINTIC, 1e-7, prec=prec)
        torch.cuda.synchronize()
        err = _rel(alone, want)
        print("k-split", shape, prec, "rel err", err, flush=True)
        assert err <= bar
        for _ in range(3):
            assert torch.equal(ns.newton_schulz(Gd, O.QUINTIC, 1e-7, prec=prec), alone)
        batch = torch.stack([Gd, _randn(shape, 78).to(gpu_device), Gd])
        out = ns.newton_schulz(batch, O.QUINTIC, 1e-7, prec=prec)
        assert torch.equal(out[0], alone) and torch.equal(out[2], alone)
        other = _randn((2, 256, 640), 79).to(gpu_device)
        a, b = ns.newton_schulz_grouped([other, Gd], O.QUINTIC, 1e-7, prec=prec)
        assert torch.equal(b, alone)
        assert torch.equal(a, ns.newton_schulz(other, O.QUINTIC, 1e-7, prec=prec))


def test_odd_number_of_small_tiles_in_a_batch(ns, gpu_device):
    """Short sides of 384 or 640 (three or five 128-tiles, the expert width of the depth-24 MoE set) and a ragged one, in
    a batch large enough for the usual tile choice, in both orientations of the final store: within the bar of the fp32
    oracle in either orientation (the two orientations sum the squares for the norm in different orders, so they agree
    to the last bits only), and the same bits as a single call, which takes the small configuration throughout."""
    for shape in [(384, 1024), (640, 768), (300, 1000)]:
        G = _randn((24,) + shape, 41 + sum(shape))
        out = ns.newton_schulz(G.to(gpu_device))
        outT = ns.newton_schulz(G.mT.contiguous().to(gpu_device))
        torch.cuda.synchronize()
        assert _rel(outT.mT, out) <= 1e-3
        for i in (0, 11, 23):
            want = O.newton_schulz(G[i], O.QUINTIC, 1e-7, storage="fp32")
            assert _rel(out[i], want) <= NS_TOL and _rel(outT[i].mT, want) <= NS_TOL, (shape, i)
            assert torch.equal(ns.newton_schulz(G[i].to(gpu_device)), out[i])
            assert torch.equal(ns.newton_schulz(G[i].mT.contiguous().to(gpu_device)), outT[i])
        f16 = ns.newton_schulz(G.to(gpu_device), O.QUINTIC, 1e-7, prec="f16")
        assert _rel(f16[5], O.newton_schulz(G[5], O.QUINTIC, 1e-7, storage="fp32")) <= 4e-3


@pytest.mark.parametrize("n", [3072, 2560, 4096, 2304, 2816, 3584])
def test_large_triangles_are_covered_tile_by_tile(ns, gpu_device, n):
    """The stand-alone symmetric products on matrices with more than eight tiles of 256 along a side (12, 10, 16, 9, 11
    and 14): large upper triangles are walked in blocks of 4 x 4 tiles; when the side is no multiple of four tiles the
    last block column is 2, 1 or 3 tiles wide and the last diagonal block a triangle of that side.  Every tile must be
    written exactly once.  The result is checked against an fp32 product element by element (an unwritten tile holds
    whatever the workspace held, a misplaced one the wrong block of the product) and it is bit-symmetric."""
    print("case", n, flush=True)
    X = _randn((n, 320), 51 + n, 0.05).to(gpu_device)
    A = ns.ns_line_1(X)
    want = X.float() @ X.float().T
    torch.cuda.synchronize()
    assert torch.equal(A, A.mT)
    assert (A.float() - want).abs().max().item() <= 4e-3 * want.abs().max().item()
    B = ns.ns_line_2(A, alpha=2.0315 / 64, beta=-4.775)
    wantB = (2.0315 / 64) * (A.float() @ A.float()) - 4.775 * A.float()
    assert torch.equal(B, B.mT)
    assert (B.float() - wantB).abs().max().item() <= 6e-3 * wantB.abs().max().item()
