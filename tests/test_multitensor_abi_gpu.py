"""The multi-tensor entry points called DIRECTLY through the C ABI (device item tables filled by hand), over every
storage-dtype combination and over sizes that straddle the 8192-element chunk and the 16-byte vector width.
Expected values: the same arithmetic in fp64 on the host with the reference's rounding points (M <- c_mm M + c_mg (G + l2 W),
U = c_um M' + c_ug G; plain and MuonH updates in their closed forms)."""
import itertools

import numpy as np
import pytest
import torch

from archscale_amd import _lib

pytestmark = pytest.mark.gpu

NUMELS = [1, 7, 8, 9, 8191, 8192, 8193, 3 * 8192 + 5, 100_003]
BF, F32 = torch.bfloat16, torch.float32


def _table(rows, numels, device):
    prefix = np.zeros(len(numels) + 1, dtype=np.int32)
    for i, n in enumerate(numels):
        prefix[i + 1] = prefix[i] + (n + _lib.CHUNK_ELEMS - 1) // _lib.CHUNK_ELEMS
    dev = torch.from_numpy(rows.view(np.uint8).copy()).to(device)
    return dev, torch.from_numpy(prefix).to(device), int(prefix[-1])


def _rand(n, dtype, gen, scale):
    # 8-byte misaligned starts would break the vector path: torch allocations are 256-byte aligned, as the ABI asks
    return (torch.randn(n, generator=gen) * scale).to(dtype)


@pytest.mark.parametrize("g_dt,m_dt,u_dt", list(itertools.product((BF, F32), (BF, F32), (BF, F32))))
@pytest.mark.parametrize("l2", [0.0, 0.01])
def test_momentum_all_dtype_combinations(gpu_device, g_dt, m_dt, u_dt, l2):
    gen = torch.Generator().manual_seed(11)
    G = [_rand(n, g_dt, gen, 1e-2) for n in NUMELS]
    M = [_rand(n, m_dt, gen, 1e-2) for n in NUMELS]
    W = [_rand(n, F32, gen, 0.02) for n in NUMELS]
    Gd, Md, Wd = ([t.to(gpu_device) for t in L] for L in (G, M, W))
    Ud = [torch.full((n,), float("nan"), dtype=u_dt, device=gpu_device) for n in NUMELS]
    rows = np.zeros(len(NUMELS), dtype=_lib.PRE_ITEM)
    for r, g, m, u, w in zip(rows, Gd, Md, Ud, Wd):
        r["g"], r["m"], r["u"], r["w"] = g.data_ptr(), m.data_ptr(), u.data_ptr(), w.data_ptr() if l2 else 0
        r["numel"] = g.numel()
        r["g_dtype"], r["m_dtype"], r["u_dtype"], r["w_dtype"] = (_lib.dtype_code(t.dtype) for t in (g, m, u, w))
    tab, prefix, chunks = _table(rows, NUMELS, gpu_device)
    c_mm, c_mg, c_um, c_ug = 0.95, 1.0, 0.95, 1.0
    _lib.check(_lib.lib().muon_momentum(tab.data_ptr(), prefix.data_ptr(), len(NUMELS), chunks, c_mm, c_mg, c_um, c_ug,
                                        l2, _lib.current_stream_ptr(gpu_device)), "muon_momentum")
    torch.cuda.synchronize()
    for g, m, w, gd, md, ud in zip(G, M, W, Gd, Md, Ud):
        # reference order (muon.py:665-679, mixin.py:48-49): G += l2 W in G's dtype and in place; G cast to M's dtype;
        # M updated and rounded to its storage type; U formed from the ROUNDED momentum
        gg = (g.double() + l2 * w.double()).to(g_dt) if l2 else g
        gm = gg.to(m_dt).double()
        m_want = (c_mm * m.double() + c_mg * gm).to(m_dt)
        u_want = c_um * m_want.double() + c_ug * gm
        ulp = lambda dt: 2 ** -7 if dt == BF else 2e-7      # one unit in the last place of the stored value
        assert torch.allclose(gd.double().cpu(), gg.double(), rtol=ulp(g_dt), atol=5e-9)
        assert torch.allclose(md.double().cpu(), m_want.double(), rtol=ulp(m_dt), atol=5e-9)
        assert torch.allclose(ud.double().cpu(), u_want, rtol=ulp(u_dt), atol=5e-9)


@pytest.mark.parametrize("w_dt", [BF, F32])
@pytest.mark.parametrize("cautious", [0, 1])
def test_plain_and_muonh_updates_ragged(gpu_device, w_dt, cautious):
    gen = torch.Generator().manual_seed(12)
    lr, lr_wd, eps = 0.02, 0.02 * 0.1, 1e-8
    for muonh in (False, True):
        W = [_rand(n, w_dt, gen, 0.02) for n in NUMELS]
        U = [_rand(n, BF, gen, 0.05) for n in NUMELS]
        Wd, Ud = [t.to(gpu_device) for t in W], [t.to(gpu_device) for t in U]
        rows = np.zeros(len(NUMELS), dtype=_lib.POST_ITEM)
        ratios = np.linspace(0.5, 2.0, len(NUMELS)).astype(np.float32)
        for r, w, u, k in zip(rows, Wd, Ud, ratios):
            r["w"], r["u"], r["numel"], r["lr_ratio"], r["w_dtype"] = w.data_ptr(), u.data_ptr(), w.numel(), k, _lib.dtype_code(w.dtype)
        tab, prefix, chunks = _table(rows, NUMELS, gpu_device)
        L = _lib.lib()
        if muonh:
            scratch = torch.empty(L.muon_muonh_scratch_floats(len(NUMELS), chunks), dtype=F32, device=gpu_device)
            _lib.check(L.muon_update_muonh(tab.data_ptr(), prefix.data_ptr(), len(NUMELS), chunks, lr, lr_wd, eps, cautious,
                                           scratch.data_ptr(), _lib.current_stream_ptr(gpu_device)), "muon_update_muonh")
        else:
            _lib.check(L.muon_update_plain(tab.data_ptr(), prefix.data_ptr(), len(NUMELS), chunks, lr, lr_wd, cautious,
                                           _lib.current_stream_ptr(gpu_device)), "muon_update_plain")
        torch.cuda.synchronize()
        for w, u, k, got in zip(W, U, ratios, Wd):
            x, uu = w.double(), u.double()
            xd = torch.where(x * uu >= 0, x - lr_wd * x, x) if cautious else x * (1 - lr_wd)
            if muonh:
                s = xd.norm() / uu.norm().clamp_min(eps)
                y = xd - lr * s * uu
                want = y * xd.norm() / y.norm().clamp_min(eps)
            else:
                want = xd - lr * float(k) * uu
            tol = 2 ** -7 if w_dt == BF else 2e-6
            assert torch.allclose(got.double().cpu(), want, rtol=tol, atol=1e-9), (muonh, w.numel())


def test_argument_errors_do_not_launch(gpu_device):
    L = _lib.lib()
    assert L.muon_momentum(0, 0, 1, 1, 0.9, 1.0, 0.9, 1.0, 0.0, 0) < 0
    assert L.muon_update_plain(0, 0, 1, 1, 0.1, 0.0, 0, 0) < 0
    assert L.muon_update_muonh(0, 0, 1, 1, 0.1, 0.0, 1e-8, 0, 0, 0) < 0
    assert L.muon_momentum(0, 0, 0, 0, 0.9, 1.0, 0.9, 1.0, 0.0, 0) == 0      # nothing to do
    torch.cuda.synchronize()


def test_streaming_yardsticks(gpu_device):
    """muon_calibration_stream: the copy, the read-only pass and the two-read / two-write mix do what the header says
    (word-wise, on sizes that are and are not a multiple of a block's piece)."""
    import numpy as np
    from archscale_amd import _lib
    L = _lib.lib()
    stream = _lib.current_stream_ptr(gpu_device)
    for n_words in (4, 4 * 1024 * 4, 4 * (3 * 1024 + 17)):
        rng = np.random.default_rng(n_words)
        a = torch.from_numpy(rng.integers(0, 2 ** 31, n_words, dtype=np.int64).astype(np.int32)).to(gpu_device)
        b = torch.from_numpy(rng.integers(0, 2 ** 31, n_words, dtype=np.int64).astype(np.int32)).to(gpu_device)
        c = torch.zeros_like(a)
        a0, b0 = a.clone(), b.clone()
        nbytes = 4 * n_words
        assert L.muon_calibration_stream(_lib.STREAM_READ, a.data_ptr(), b.data_ptr(), 0, nbytes, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(a, a0) and torch.equal(b, b0)
        assert L.muon_calibration_stream(_lib.STREAM_MIX, a.data_ptr(), b.data_ptr(), c.data_ptr(), nbytes, stream) == 0
        torch.cuda.synchronize()
        total = a0 + b0                     # int32 wrap-around = the kernel's unsigned 32-bit sum
        assert torch.equal(b, total) and torch.equal(c, total ^ a0) and torch.equal(a, a0)
        assert L.muon_calibration_stream(_lib.STREAM_COPY, a.data_ptr(), c.data_ptr(), 0, nbytes, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(c, a0)
    assert L.muon_calibration_stream(7, a.data_ptr(), b.data_ptr(), c.data_ptr(), 16, stream) == -1
    assert L.muon_calibration_stream(_lib.STREAM_MIX, a.data_ptr(), b.data_ptr(), 0, 16, stream) == -1
    assert L.muon_calibration_stream(_lib.STREAM_READ, a.data_ptr(), b.data_ptr(), 0, 12, stream) == -1
