"""MuonBall on the GPU (through the C ABI) against the CPU oracle: spectral norm by power iteration, the fused
retraction + update kernel, and whole optimizer steps with and without fused-parameter splits."""
import math

import numpy as np
import pytest
import torch

from oracle import muon_ball_oracle as B
from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu

SIGMA_TOL = 3e-3     # vs the same vector sequence in fp64 (the HIP path keeps fp32 vectors and a bf16 Gram matrix)
SIGMA_REF_TOL = 1.5e-2   # vs the reference's bf16 execution, whose result is itself a bf16 number
W_TOL = 2e-2


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


@pytest.mark.parametrize("shape", [(48, 160), (160, 48), (64, 64), (300, 700), (700, 300), (512, 2048), (2048, 512), (1, 40), (40, 1)])
@pytest.mark.parametrize("steps", [1, 2, 6, 7, 16, 19, 50])
def test_spectral_norm_matches_the_definition(gpu_device, shape, steps):
    from archscale_amd.emerging.spectral_ball_utils import spectral_norm
    g = torch.Generator().manual_seed(shape[0] * 7 + shape[1] + steps)
    W = (torch.randn(*shape, generator=g) * 0.02).to(torch.bfloat16)
    got = spectral_norm(W.to(gpu_device), steps).item()
    want = B.power_iteration_fp64(W, steps)
    assert abs(got - want) / want < SIGMA_TOL, (got, want)
    ref = float(B.power_iteration(W, steps)[0])
    assert abs(got - ref) / ref < SIGMA_REF_TOL


@pytest.mark.parametrize("shape", [(96, 200), (200, 96), (256, 256)])
def test_spectral_norm_scales_with_the_matrix(gpu_device, shape):
    """The grouped rounds run on powers of the Gram matrix that the library rescales by its trace: a matrix times a
    power of two (exact in bf16) must give exactly that multiple of sigma, up to fp32 rounding, from 2^-30 to 2^20."""
    from archscale_amd.emerging.spectral_ball_utils import spectral_norm
    g = torch.Generator().manual_seed(shape[0] + 3 * shape[1])
    W = (torch.randn(*shape, generator=g) * 0.02).to(torch.bfloat16)
    base = spectral_norm(W.to(gpu_device), 50).item()
    assert abs(base - B.power_iteration_fp64(W, 50)) < SIGMA_TOL * base
    for e in (-30, -12, 9, 20):
        got = spectral_norm((W.float() * 2.0 ** e).to(torch.bfloat16).to(gpu_device), 50).item()
        assert abs(got / 2.0 ** e - base) <= 1e-4 * base, (e, got / 2.0 ** e, base)


def test_spectral_norm_batches_dtypes_strides_and_zero(gpu_device):
    from archscale_amd.emerging.spectral_ball_utils import spectral_norm, power_iteration
    g = torch.Generator().manual_seed(5)
    W = torch.randn(3, 2, 96, 200, generator=g) * 0.05
    W[1, 1] = 0
    got = spectral_norm(W.to(gpu_device), 30).cpu()
    assert got.shape == (3, 2) and got[1, 1].item() == 0.0
    for i in range(3):
        for j in range(2):
            want = B.power_iteration_fp64(W[i, j], 30)
            assert abs(got[i, j].item() - want) <= SIGMA_TOL * want
    # a strided view (rows of a wider matrix)
    big = (torch.randn(64, 256, generator=g) * 0.02).to(torch.bfloat16).to(gpu_device)
    view = big[:, 64:192]
    assert abs(spectral_norm(view, 20).item() - B.power_iteration_fp64(view.cpu(), 20)) < SIGMA_TOL * 0.5
    s, u, v = power_iteration(W[0, 0].to(gpu_device), 10)
    assert u.shape == (96, 1) and v.shape == (200, 1) and abs(s.item() - B.power_iteration_fp64(W[0, 0], 10)) < 1e-2
    with pytest.raises(ValueError):
        spectral_norm(torch.zeros(4, device=gpu_device), 3)
    with pytest.raises(ValueError):
        spectral_norm(W.to(gpu_device), 0)


# ---------------------------------------------------------------------------------------------------------------
# fused retraction + update kernel, called directly through the C ABI
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("w_dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["hard", "dynamic"])
def test_ball_apply_strided_blocks(gpu_device, w_dt, mode):
    from archscale_amd import _lib
    g = torch.Generator().manual_seed(3)
    # blocks of two "parameters": whole matrix, a column block (ld > cols), a row block, an odd-sized block (scalar path)
    P1 = (torch.randn(96, 160, generator=g) * 0.05).to(w_dt)
    P2 = (torch.randn(37, 53, generator=g) * 0.05).to(w_dt)
    F1 = torch.randn(96, 160, generator=g).to(torch.bfloat16)
    F2 = torch.randn(37, 53, generator=g).to(torch.bfloat16)
    blocks = [  # (param, phi, off, rows, cols, ld, radius, ratio, sigma or None)
        (0, 0, 96, 64, 160, 0.7, 1.5, 0.9),
        (0, 64, 96, 96, 160, 1.1, 0.5, 2.0),
        (1, 0, 20, 53, 53, 0.8, 1.0, 0.3),
        (1, 20 * 53, 17, 53, 53, 0.9, 2.0, None),
    ]
    Pd = [P1.to(gpu_device), P2.to(gpu_device)]
    Fd = [F1.to(gpu_device), F2.to(gpu_device)]
    sig = torch.tensor([b[7] if b[7] is not None else 0.0 for b in blocks], dtype=torch.float32, device=gpu_device)
    items = np.zeros(len(blocks), dtype=_lib.BALL_ITEM)
    prefix = np.zeros(len(blocks) + 1, dtype=np.int32)
    for r, (pi, off, rows, cols, ld, radius, ratio, s) in enumerate(blocks):
        it = items[r]
        it["w"] = Pd[pi].data_ptr() + off * Pd[pi].element_size()
        it["phi"] = Fd[pi].data_ptr() + off * 2
        it["sigma"] = sig.data_ptr() + 4 * r if s is not None else 0
        it["ld_w"] = it["ld_phi"] = ld
        it["rows"], it["cols"], it["radius"], it["lr_ratio"], it["w_dtype"] = rows, cols, radius, ratio, _lib.dtype_code(w_dt)
        prefix[r + 1] = prefix[r] + (rows * cols + _lib.CHUNK_ELEMS - 1) // _lib.CHUNK_ELEMS
    tab = torch.from_numpy(items.view(np.uint8).copy()).to(gpu_device)
    pre = torch.from_numpy(prefix).to(gpu_device)
    log = torch.full((2 * len(blocks),), float("nan"), device=gpu_device)
    lr, decay, alpha_lr = 0.02, 0.998, 0.05 * 0.02
    _lib.check(_lib.lib().muon_ball_apply(tab.data_ptr(), pre.data_ptr(), len(blocks), int(prefix[-1]), lr, decay,
                                          _lib.RETRACT_DYNAMIC if mode == "dynamic" else _lib.RETRACT_HARD, alpha_lr,
                                          log.data_ptr(), _lib.current_stream_ptr(gpu_device)), "muon_ball_apply")
    torch.cuda.synchronize()
    want = [P1.double().clone(), P2.double().clone()]
    src = [P1.double(), P2.double()]
    phi = [F1.double(), F2.double()]
    for r, (pi, off, rows, cols, ld, radius, ratio, s) in enumerate(blocks):
        r0, c0 = divmod(off, ld)
        if s is None:
            f, bias, sd = 1.0, 0.0, 0.0
        else:
            sd = float(np.float32(decay) * np.float32(s))
            if mode == "hard":
                f, bias = radius / (max(sd, 0.0) + 1e-8), 0.0
            else:
                bias = -1.0 if sd > radius else 1.0
                f = 1.0 + alpha_lr * bias
        blk = (slice(r0, r0 + rows), slice(c0, c0 + cols))
        want[pi][blk] = f * decay * src[pi][blk] - lr * ratio * phi[pi][blk]
        assert log[2 * r].item() == pytest.approx(sd, rel=1e-6) and log[2 * r + 1].item() == bias
    tol = 2 ** -7 if w_dt == torch.bfloat16 else 3e-6
    for got, w in zip(Pd, want):
        assert torch.allclose(got.double().cpu(), w, rtol=tol, atol=1e-7)
    # untouched region of P1 (columns 160.. do not exist; rows/cols outside every block: none here) and argument errors
    L = _lib.lib()
    assert L.muon_ball_apply(0, 0, 1, 1, 0.1, 1.0, 0, 0.0, 0, 0) < 0
    assert L.muon_ball_apply(tab.data_ptr(), pre.data_ptr(), len(blocks), int(prefix[-1]), 0.1, 1.0, 7, 0.0, 0, 0) < 0


# ---------------------------------------------------------------------------------------------------------------
# whole optimizer steps
# ---------------------------------------------------------------------------------------------------------------
def _named(t, name, **attrs):
    p = torch.nn.Parameter(t)
    p.param_name = name
    for k, v in attrs.items():
        setattr(p, k, v)
    return p


def _run_pair(gpu_device, shapes, wdtype, opt_kw, splits=None, attrs=None, steps=2, seed=0, ns_storage="fp32", sigma_fn=None):
    """Runs `steps` MuonBall steps on the GPU and the oracle on the CPU from the same state; returns both weight lists."""
    from archscale_amd.emerging import MuonBall
    g = torch.Generator().manual_seed(seed)
    W0 = [(torch.randn(*s, generator=g) * 0.05).to(wdtype) for s in shapes]
    grads = [[(torch.randn(*s, generator=g) * 1e-2).to(wdtype) for s in shapes] for _ in range(steps)]
    params = [_named(w.clone().to(gpu_device), f"layer{i}.weight", **((attrs or {}).get(i, {}))) for i, w in enumerate(W0)]
    opt = MuonBall(params, **opt_kw)
    for gs in grads:
        for p, gr in zip(params, gs):
            p.grad = gr.clone().to(gpu_device)
        opt.step()
    torch.cuda.synchronize()
    kw = dict(radius_mode=opt_kw.get("radius_mode", "spectral_mup"), scale_mode=opt_kw.get("scale_mode", "align_adamw_rms"),
              power_iteration_steps=opt_kw.get("power_iteration_steps", 10), msign_steps=opt_kw.get("msign_steps", 5),
              retract_mode=opt_kw.get("retract_mode", "hard"), retract_alpha=opt_kw.get("retract_alpha", 0.05),
              ns_storage=ns_storage, sigma_fn=sigma_fn)
    X = [w.clone() for w in W0]
    M = [torch.zeros_like(w) for w in W0]
    for gs in grads:
        for i, (x, gr, m) in enumerate(zip(X, gs, M)):
            B.muon_ball_step(x, gr.clone(), m, lr=opt_kw.get("lr", 3e-4), beta=opt_kw.get("momentum_beta", 0.9),
                             wd=opt_kw.get("weight_decay", 0.01), nesterov=opt_kw.get("use_nesterov", True),
                             wd_method=opt_kw.get("weight_decay_method", "decoupled"),
                             split=(splits or {}).get(i), **kw)
    return [p.detach().cpu() for p in params], X, W0, opt, params


SHAPES = [(128, 256), (256, 128), (128, 256), (64, 64)]


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("retract_mode", ["hard", "dynamic"])
@pytest.mark.parametrize("wd_method,wd", [("decoupled", 0.1), ("independent", 0.01), ("l2", 0.1), ("decoupled", 0.0)])
def test_step_matches_oracle(gpu_device, wdtype, retract_mode, wd_method, wd):
    kw = dict(lr=0.02, momentum_beta=0.9, weight_decay=wd, weight_decay_method=wd_method, use_nesterov=True,
              power_iteration_steps=10, msign_steps=5, retract_mode=retract_mode)
    # tolerance oracle: fp32 msign and the exact (fp64) value of the same power-iteration sequence; the reference's own
    # sigma is a bf16 number (up to 0.8 % off), which test_step_reference_semantics_bf16 covers at the weight tolerance
    got, want, W0, opt, _ = _run_pair(gpu_device, SHAPES, wdtype, kw, seed=1, sigma_fn=B.power_iteration_fp64)
    for gw, ww, w0 in zip(got, want, W0):
        assert _rel(gw, ww) <= W_TOL
        if wdtype == torch.float32:
            # the hard retraction alone rescales W by R/sigma (a large change); the step direction is checked on top of it
            assert _rel(gw - w0, ww - w0) <= 3e-2
    if retract_mode == "hard":
        # two steps from W0: after the last retraction + update the spectral norm is R up to the update (lr * scale)
        for gw, s in zip(got, SHAPES):
            R = math.sqrt(s[0] / s[1])
            top = torch.linalg.svdvals(gw.double())[0].item()
            assert abs(top - R) / R < 0.3


def test_step_reference_semantics_bf16(gpu_device):
    """Against the reference's own (eager bf16) msign and bf16 power iteration, bf16 weights, 50 rounds."""
    kw = dict(lr=0.02, momentum_beta=0.9, weight_decay=0.01, use_nesterov=True, power_iteration_steps=50, msign_steps=5)
    got, want, _, _, _ = _run_pair(gpu_device, SHAPES, torch.bfloat16, kw, seed=2, ns_storage="bf16_eager", steps=1)
    for gw, ww in zip(got, want):
        assert _rel(gw, ww) <= W_TOL


@pytest.mark.parametrize("case", ["fc1", "qkv_group", "qkv_head", "qkv_component", "moe1_split", "moe1", "moe2"])
@pytest.mark.parametrize("retract_mode", ["hard", "dynamic"])
def test_fused_parameter_splits(gpu_device, case, retract_mode):
    kw = dict(lr=0.02, momentum_beta=0.9, weight_decay=0.1, use_nesterov=True, power_iteration_steps=8, msign_steps=5,
              retract_mode=retract_mode)
    attrs, splits = {}, {}
    if case == "fc1":
        shapes = [(96, 80), (96, 80), (64, 80)]
        kw.update(split_fc1=True, is_fc1_fn=lambda p: p.shape[0] == 96, fc1_split_shapes=(48, 48))
        splits = {0: {"kind": "fc1", "shapes": (48, 48)}, 1: {"kind": "fc1", "shapes": (48, 48)}}
    elif case.startswith("qkv"):
        shapes = [(128, 80), (128, 80), (48, 80)]
        mode = case.split("_")[1]
        kw.update(split_qkv=True, is_qkv_fn=lambda p: p.shape[0] == 128, qkv_split_shapes=(32, 16, 16), qkv_split_mode=mode)
        splits = {i: {"kind": "qkv", "shapes": (32, 16, 16), "mode": mode} for i in (0, 1)}
    elif case.startswith("moe1"):
        shapes = [(80, 192), (64, 64)]
        sf = case == "moe1_split"
        kw.update(split_moe_experts=True, is_grouped_moe_fn=lambda p: getattr(p, "num_local_experts", 0) > 1, split_fc1=sf)
        attrs = {0: dict(num_local_experts=3, is_gated=True)}
        splits = {0: {"kind": "moe1", "experts": 3, "gated": True, "split_fc1": sf}}
    else:
        shapes = [(192, 80), (64, 64)]
        kw.update(split_moe_experts=True, is_grouped_moe_fn=lambda p: getattr(p, "num_local_experts", 0) > 1)
        attrs = {0: dict(num_local_experts=4)}
        splits = {0: {"kind": "moe2", "experts": 4}}
    # parameter names carry weight1 / weight2 for the MoE cases, as the reference keys on them
    from archscale_amd.emerging import MuonBall
    g = torch.Generator().manual_seed(17)
    W0 = [torch.randn(*s, generator=g) * 0.05 for s in shapes]
    G0 = [torch.randn(*s, generator=g) * 1e-2 for s in shapes]
    names = {"moe1": "mlp.experts.weight1", "moe1_split": "mlp.experts.weight1", "moe2": "mlp.experts.weight2"}
    params = [_named(w.clone().to(gpu_device), names.get(case, "attn.w") if i == 0 else f"other{i}.weight",
                     **attrs.get(i, {})) for i, w in enumerate(W0)]
    opt = MuonBall(params, **kw)
    for p, gr in zip(params, G0):
        p.grad = gr.clone().to(gpu_device)
    opt.step()
    torch.cuda.synchronize()
    okw = dict(radius_mode="spectral_mup", scale_mode="align_adamw_rms", power_iteration_steps=8, msign_steps=5,
               retract_mode=retract_mode, retract_alpha=0.05, ns_storage="fp32", sigma_fn=B.power_iteration_fp64)
    for i, (w0, g0, p) in enumerate(zip(W0, G0, params)):
        x, m = w0.clone(), torch.zeros_like(w0)
        B.muon_ball_step(x, g0.clone(), m, lr=0.02, beta=0.9, wd=0.1, nesterov=True, wd_method="decoupled",
                         split=splits.get(i), **okw)
        assert _rel(p.detach(), x) <= W_TOL, (case, i)
        assert _rel(p.detach().cpu() - w0, x - w0) <= 3e-2, (case, i)
    if retract_mode == "dynamic":
        bias, sn = opt.get_retract_bias_dict(), opt.get_spectral_norm_dict()
        assert bias and sn and set(bias) == set(sn)
        assert all(v in (-1.0, 1.0) for v in bias.values())
        n_pieces = {"fc1": 2 + 2 + 1, "qkv_group": 2 * 6 + 1, "qkv_head": 2 * 8 + 1, "qkv_component": 2 * 3 + 1,
                    "moe1_split": 6 + 1, "moe1": 3 + 1, "moe2": 4 + 1}[case]
        assert len(bias) == n_pieces
        # a piece's reported spectral norm is that of the decayed slice
        i = len(shapes) - 1                                   # the last parameter is never split
        assert sn[f"other{i}.weight"] == pytest.approx(0.998 * B.power_iteration_fp64(W0[i], 8), rel=5e-3)
    else:
        assert opt.get_retract_bias_dict() is None


def test_state_groups_and_errors(gpu_device):
    from archscale_amd.emerging import MuonBall
    g = torch.Generator().manual_seed(4)
    a = torch.nn.Parameter((torch.randn(64, 96, generator=g) * 0.05).to(gpu_device))
    b = torch.nn.Parameter((torch.randn(96, 64, generator=g) * 0.05).to(gpu_device))
    c = torch.nn.Parameter((torch.randn(64, 96, generator=g) * 0.05).to(gpu_device))   # never gets a gradient
    opt = MuonBall([{"params": [a, c]}, {"params": [b], "lr": 0.01, "wd_mult": 0.0}], lr=0.02, weight_decay=0.1)
    c0 = c.detach().clone()
    for _ in range(2):
        a.grad = torch.randn_like(a) * 1e-2
        b.grad = torch.randn_like(b) * 1e-2
        opt.step()
    assert torch.equal(c, c0) and c not in opt.state
    assert opt.state[a]["momentum_buffer"].shape == a.shape
    sd = opt.state_dict()
    opt2 = MuonBall([{"params": [a, c]}, {"params": [b], "lr": 0.01, "wd_mult": 0.0}], lr=0.02, weight_decay=0.1)
    opt2.load_state_dict(sd)
    assert torch.equal(opt2.state[a]["momentum_buffer"], opt.state[a]["momentum_buffer"])
    assert opt.step(lambda: 1.25) == 1.25
    with pytest.raises(ValueError):
        _step_1d(gpu_device)
    with pytest.raises(ValueError):
        bad = MuonBall([a], lr=0.1, radius_mode="initialize")
        a.grad = torch.randn_like(a)
        bad.step()


def _step_1d(gpu_device):
    from archscale_amd.emerging import MuonBall
    p = torch.nn.Parameter(torch.zeros(8, device=gpu_device))
    p.grad = torch.ones_like(p)
    MuonBall([p], lr=0.1).step()


def test_spectral_norm_of_the_transpose(gpu_device):
    """Before convergence the estimate depends on which side the all-ones start vector lives on; MoE expert slices are
    handed over transposed (muon_ball.py:441-485)."""
    import ctypes
    from archscale_amd import _lib
    g = torch.Generator().manual_seed(8)
    for shape in [(80, 32), (32, 80), (64, 64)]:
        W = (torch.randn(*shape, generator=g) * 0.05).to(torch.bfloat16)
        Wd = W.to(gpu_device)
        sigma = torch.empty(1, dtype=torch.float32, device=gpu_device)
        ptrs = (ctypes.c_void_p * 1)(Wd.data_ptr())
        prob = (_lib.SnProblem * 1)()
        q = prob[0]
        q.w_ptrs, q.sigma_out = ctypes.cast(ptrs, ctypes.POINTER(ctypes.c_void_p)), sigma.data_ptr()
        q.dtype, q.ld, q.batch, q.rows, q.cols, q.flags = _lib.DTYPE_BF16, shape[1], 1, shape[0], shape[1], _lib.SN_TRANSPOSED
        L = _lib.lib()
        ws = _lib.workspace(gpu_device, L.muon_spectral_norm_workspace_bytes(prob, 1), tag="sn")
        _lib.check(L.muon_spectral_norm(prob, 1, 4, ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(gpu_device)), "sn")
        want_t, want = B.power_iteration_fp64(W.t().contiguous(), 4), B.power_iteration_fp64(W, 4)
        assert abs(sigma.item() - want_t) / want_t < SIGMA_TOL
        assert abs(want_t - want) / want > 2 * SIGMA_TOL          # the two orientations really differ here
    q.flags = 2
    assert L.muon_spectral_norm(prob, 1, 4, ws.data_ptr(), ws.numel(), 0) < 0


def test_fused_momentum_matches_separate_calls(gpu_device):
    """Unsplit parameters take the fused momentum + msign call; same buffers and (up to where the update is rounded to
    bf16) the same weights as the separate momentum launch."""
    from archscale_amd.emerging import MuonBall
    shapes = [(256, 512), (512, 256), (256, 512), (192, 320)]
    outs = []
    for fuse in (True, False):
        g = torch.Generator().manual_seed(77)
        params = [torch.nn.Parameter((torch.randn(*s, generator=g) * 0.05).to(gpu_device)) for s in shapes]
        opt = MuonBall(params, lr=0.02, momentum_beta=0.9, weight_decay=0.1, use_nesterov=True, weight_decay_method="l2",
                       power_iteration_steps=20, msign_steps=5)
        opt.fuse_momentum = fuse
        w0 = [p.detach().clone() for p in params]
        for k in range(2):
            gg = torch.Generator().manual_seed(90 + k)
            for p, s in zip(params, shapes):
                p.grad = (torch.randn(*s, generator=gg) * 1e-2).to(gpu_device)
            opt.step()
        torch.cuda.synchronize()
        plan = next(iter(opt._ball_plans.values()))[1]
        assert plan.base.fused == fuse
        outs.append(([p.detach().clone() for p in params], [opt.state[p]["momentum_buffer"].clone() for p in params], w0))
    (wf, mf, w0), (ws, ms, _) = outs
    rel = lambda a, b: ((a.double() - b.double()).norm() / b.double().norm()).item()
    for a, b, m1, m2, w in zip(wf, ws, mf, ms, w0):
        assert rel(m1, m2) <= 2e-3
        assert rel(a - w, b - w) <= 1e-2


@pytest.mark.parametrize("case", ["plain", "fc1", "qkv_group", "qkv_component", "moe1_split", "moe2"])
@pytest.mark.parametrize("retract_mode", ["hard", "dynamic"])
def test_orthogonalize_per_tensor(gpu_device, case, retract_mode):
    """MuonBall.orthogonalize(p, grad, lr=...): the reference's per-tensor entry (muon_ball.py:354-636) retracts the
    parameter (piece by piece) in place and returns the update; against the oracle's restatement of the same method."""
    from archscale_amd.emerging import MuonBall
    kw = dict(lr=0.02, momentum_beta=0.9, weight_decay=0.0, power_iteration_steps=8, msign_steps=5, retract_mode=retract_mode)
    attrs, split, shape, name = {}, None, (96, 80), "attn.w"
    if case == "fc1":
        kw.update(split_fc1=True, is_fc1_fn=lambda p: True, fc1_split_shapes=(48, 48))
        split = {"kind": "fc1", "shapes": (48, 48)}
    elif case.startswith("qkv"):
        shape, mode = (128, 80), case.split("_")[1]
        kw.update(split_qkv=True, is_qkv_fn=lambda p: True, qkv_split_shapes=(32, 16, 16), qkv_split_mode=mode)
        split = {"kind": "qkv", "shapes": (32, 16, 16), "mode": mode}
    elif case == "moe1_split":
        shape, name = (80, 192), "mlp.experts.weight1"
        kw.update(split_moe_experts=True, is_grouped_moe_fn=lambda p: True, split_fc1=True)
        attrs = dict(num_local_experts=3, is_gated=True)
        split = {"kind": "moe1", "experts": 3, "gated": True, "split_fc1": True}
    elif case == "moe2":
        shape, name = (192, 80), "mlp.experts.weight2"
        kw.update(split_moe_experts=True, is_grouped_moe_fn=lambda p: True)
        attrs = dict(num_local_experts=4)
        split = {"kind": "moe2", "experts": 4}
    g = torch.Generator().manual_seed(23)
    W0 = torch.randn(*shape, generator=g) * 0.05
    M0 = torch.randn(*shape, generator=g) * 1e-2
    p = _named(W0.clone().to(gpu_device), name, **attrs)
    opt = MuonBall([p], **kw)
    upd = opt.orthogonalize(p, M0.clone().to(gpu_device), lr=0.02)
    torch.cuda.synchronize()
    assert upd.shape == p.shape and upd.dtype == torch.bfloat16
    x = W0.clone()
    want = B.orthogonalize(x, M0.clone(), lr=0.02, split=split, radius_mode="spectral_mup", scale_mode="align_adamw_rms",
                           power_iteration_steps=8, msign_steps=5, retract_mode=retract_mode, retract_alpha=0.05,
                           ns_storage="fp32", sigma_fn=B.power_iteration_fp64)
    assert _rel(upd, want) <= 1e-2, case
    assert _rel(p.detach(), x) <= 5e-3, case                      # the retraction reached the parameter (fp32 weights)
    if case != "qkv_component":
        assert not torch.equal(p.detach().cpu(), W0)
    else:
        assert torch.equal(p.detach().cpu(), W0)                 # gathered copies: the parameter is not retracted, as in the reference
    if retract_mode == "dynamic":
        assert (len(opt.retract_bias_dict) > 0) == (case != "plain")   # logged per labelled component, like the reference
    # applying it the way the base class does is one step of the optimizer
    with torch.no_grad():
        p.add_(upd.to(p.dtype), alpha=-0.02)
    x.add_(want, alpha=-0.02)
    assert _rel(p.detach(), x) <= W_TOL


@pytest.mark.parametrize("retract_mode", ["hard", "dynamic"])
def test_orthogonalize_bf16_weights_keep_the_factor_in_fp32(gpu_device, retract_mode):
    """bf16 parameters through the per-tensor entry: the retraction factor (R / sigma, or 1 +- alpha * lr) multiplies the
    weights in fp32 and the product is rounded once, as the reference's ``W.mul_(python_float)`` does
    (muon_ball.py:301-352); the result is what the same factor gives on the host.  A factor rounded to bf16 first would
    be off by up to 0.4 %."""
    from archscale_amd.emerging import MuonBall
    from archscale_amd.emerging.spectral_ball_utils import spectral_norm, compute_target_radius
    g = torch.Generator().manual_seed(29)
    W0 = (torch.randn(96, 80, generator=g) * 0.05).to(torch.bfloat16)
    M0 = (torch.randn(96, 80, generator=g) * 1e-2).to(torch.bfloat16)
    lr = 0.2      # dynamic mode: factor 1 +- 0.01, which bf16 would round to 1.0078 / 0.9922
    p = _named(W0.clone().to(gpu_device), "attn.w")
    opt = MuonBall([p], lr=lr, momentum_beta=0.9, weight_decay=0.0, power_iteration_steps=8, msign_steps=5,
                   retract_mode=retract_mode)
    sigma = spectral_norm(W0.to(gpu_device), 8).item()
    R = compute_target_radius((96, 80), "spectral_mup")
    opt.orthogonalize(p, M0.clone().to(gpu_device), lr=lr)
    torch.cuda.synchronize()
    factor = R / (sigma + 1e-8) if retract_mode == "hard" else 1.0 + 0.05 * lr * (-1.0 if sigma > R else 1.0)
    want = (W0.float() * torch.tensor(factor, dtype=torch.float32)).to(torch.bfloat16)
    got = p.detach().cpu()
    assert (got.float() - want.float()).abs().max().item() <= 2.0 ** -8 * want.float().abs().max().item()   # one bf16 ulp
    assert _rel(got, W0.double() * factor) <= 2.5e-3      # bf16 rounding of the product only (measured 1.9e-3)


@pytest.mark.parametrize("shape", [(48, 160), (160, 48), (64, 64), (3, 100, 260), (2, 2, 300, 72), (1, 40), (40, 1)])
@pytest.mark.parametrize("steps", [1, 7, 50])
def test_power_iteration_vectors(gpu_device, shape, steps):
    """(sigma, u, v) of the reference's power_iteration (spectral_ball_utils.py:151-166) from the library: against the same
    vector sequence in fp64, v_k = normalize(W^T W v_{k-1}) from the all-ones vector, u = normalize(W v), sigma = |W v|."""
    from archscale_amd.emerging.spectral_ball_utils import power_iteration, spectral_norm
    g = torch.Generator().manual_seed(sum(shape) + steps)
    W = (torch.randn(*shape, generator=g) * 0.02).to(torch.bfloat16)
    sigma, u, v = power_iteration(W.to(gpu_device), steps)
    torch.cuda.synchronize()
    rows, cols = shape[-2:]
    assert sigma.shape == shape[:-2] and u.shape == (*shape[:-2], rows, 1) and v.shape == (*shape[:-2], cols, 1)
    assert u.dtype == torch.bfloat16 and v.dtype == torch.bfloat16
    assert torch.equal(sigma, spectral_norm(W.to(gpu_device), steps))          # the same sigma as the norm-only entry
    Wd = W.double().reshape(-1, rows, cols)
    for b in range(Wd.shape[0]):
        vv = torch.ones(cols, 1, dtype=torch.float64)
        for _ in range(steps):
            vv = Wd[b].T @ (Wd[b] @ vv)
            vv = vv / vv.norm()
        uu = Wd[b] @ vv
        s_ref = uu.norm().item()
        uu = uu / uu.norm()
        ub = u.reshape(-1, rows, 1)[b].double().cpu()
        vb = v.reshape(-1, cols, 1)[b].double().cpu()
        assert abs(sigma.reshape(-1)[b].item() - s_ref) <= 1e-2 * s_ref      # (sigma itself: the tests above)
        assert abs(ub.norm().item() - 1) < 1e-2 and abs(vb.norm().item() - 1) < 1e-2
        # the pair realises the estimate: u^T W v = sigma (second-order in the direction error of either vector)
        assert (ub.T @ Wd[b] @ vb).item() == pytest.approx(s_ref, rel=1.5e-2)
        if steps <= 7:
            # far from convergence the sequence itself is the definition: same direction and sign as in fp64, to the three
            # digits of a bf16 unit vector (after many rounds the direction inside a cluster of close singular values
            # depends on the rounding of the Gram matrix, in the reference's bf16 arithmetic as much as here)
            assert (ub - uu).norm().item() <= 1.5e-2 and (vb - vv).norm().item() <= 1.5e-2, (b, (ub - uu).norm(), (vb - vv).norm())
