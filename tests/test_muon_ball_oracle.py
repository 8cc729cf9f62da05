"""Pins of oracle/muon_ball_oracle.py: closed forms and invariants that do not restate its formulas."""
import math

import pytest
import torch

from oracle import muon_ball_oracle as B
from oracle import muon_oracle as O


def _gapped(rows, cols, sigma1, seed):
    """Matrix with a known, well separated top singular value."""
    g = torch.Generator().manual_seed(seed)
    U, _ = torch.linalg.qr(torch.randn(rows, min(rows, cols), generator=g, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(cols, min(rows, cols), generator=g, dtype=torch.float64))
    s = torch.linspace(0.3, 0.05, min(rows, cols), dtype=torch.float64)
    s[0] = sigma1
    return (U * s) @ V.T


@pytest.mark.parametrize("shape", [(48, 96), (96, 48), (64, 64)])
def test_power_iteration_finds_top_singular_value(shape):
    W = _gapped(*shape, 2.5, 3).float()
    want = torch.linalg.svdvals(W.to(torch.bfloat16).double())[0].item()
    s, u, v = B.power_iteration(W, steps=50)
    assert abs(float(s) - want) / want < 1e-2            # the reference's result is a bf16 number (ulp 2^-8 .. 2^-7)
    assert abs(B.power_iteration_fp64(W, 50) - want) / want < 1e-9
    assert abs(B.power_iteration_gram_fp64(W, 50) - want) / want < 1e-9
    assert u.shape == (shape[0], 1) and v.shape == (shape[1], 1)
    # u, v are unit vectors aligned with the top singular pair
    assert abs(float(u.float().norm()) - 1) < 1e-2 and abs(float(v.float().norm()) - 1) < 1e-2


@pytest.mark.parametrize("shape", [(40, 72), (72, 40), (56, 56)])
@pytest.mark.parametrize("steps", [1, 2, 7, 50])
def test_gram_forms_equal_the_definition_before_convergence(shape, steps):
    """No spectral gap (Gaussian matrix): the k-round value is NOT the top singular value yet, and the Gram forms
    must reproduce exactly that unconverged number."""
    g = torch.Generator().manual_seed(11)
    W = torch.randn(*shape, generator=g) * 0.02
    a, b = B.power_iteration_fp64(W, steps), B.power_iteration_gram_fp64(W, steps)
    assert abs(a - b) / a < 1e-10
    top = torch.linalg.svdvals(W.to(torch.bfloat16).double())[0].item()
    assert a <= top * (1 + 1e-12)
    if steps <= 2:
        assert a < 0.999 * top                            # really unconverged: the test has teeth
    # the bf16 restatement follows the same sequence up to rounding noise
    assert abs(float(B.power_iteration(W, steps)[0]) - a) / a < 1.5e-2


def test_power_iteration_zero_matrix_and_batch():
    assert float(B.power_iteration(torch.zeros(8, 16), 5)[0]) == 0.0
    assert B.power_iteration_gram_fp64(torch.zeros(8, 16), 5) == 0.0
    W = torch.stack([_gapped(24, 40, 1.5, 1).float(), _gapped(24, 40, 0.7, 2).float()])
    s = B.power_iteration(W, 30)[0]
    assert s.shape == (2,) and abs(float(s[0]) - 1.5) < 2e-2 and abs(float(s[1]) - 0.7) < 1e-2
    with pytest.raises(ValueError):
        B.power_iteration(torch.zeros(4), 3)


def test_retraction():
    W = _gapped(32, 64, 3.0, 5).float()
    R = B.compute_target_radius(W.shape, "spectral_mup")
    assert R == pytest.approx(math.sqrt(32 / 64))
    assert B.compute_target_radius((5, 7), "identity") == 1.0
    with pytest.raises(ValueError):
        B.compute_target_radius((5, 7), "initialize")
    X = W.clone()
    assert B.apply_retract(X, 3.0, R, mode="hard") == 0.0
    assert torch.linalg.svdvals(X.double())[0].item() == pytest.approx(R, rel=1e-5)
    X = W.clone()
    assert B.apply_retract(X, 3.0, R, mode="dynamic", alpha=0.05, current_lr=0.1) == -1.0
    assert torch.allclose(X, W * (1 - 0.005))
    X = W.clone()
    assert B.apply_retract(X, 0.1, R, mode="dynamic", alpha=0.05) == 1.0
    assert torch.allclose(X, W * 1.05)
    with pytest.raises(ValueError):
        B.apply_retract(X, 1.0, R, mode="soft")


def test_scale_factors():
    assert B.spectral_ball_scale_factor(64, 16, "shape_scaling") == 2.0
    assert B.spectral_ball_scale_factor(16, 64, "shape_scaling") == 1.0
    assert B.spectral_ball_scale_factor(16, 64, "align_adamw_rms") == pytest.approx(0.2 * 8)
    assert B.spectral_ball_scale_factor(16, 64, "spectral_mup") == 0.5
    with pytest.raises(ValueError):
        B.spectral_ball_scale_factor(1, 1, "x")


KW = dict(radius_mode="spectral_mup", scale_mode="align_adamw_rms", power_iteration_steps=20, msign_steps=5,
          retract_mode="hard", retract_alpha=0.05, ns_storage="fp32")


def test_step_lands_on_the_spectral_sphere_and_moves_along_msign():
    g = torch.Generator().manual_seed(7)
    p = _gapped(48, 80, 2.0, 9).float()
    grad = torch.randn(48, 80, generator=g) * 1e-2
    buf = torch.zeros_like(p)
    p0 = p.clone()
    B.muon_ball_step(p, grad.clone(), buf, lr=0.01, beta=0.9, wd=0.0, nesterov=True, wd_method="decoupled", **KW)
    assert torch.allclose(buf, 0.1 * grad)
    R = math.sqrt(48 / 80)
    retracted = p0 * (R / (B.power_iteration(p0, 20)[0].item() + 1e-8))
    delta = (retracted - p) / 0.01 / (0.2 * math.sqrt(80))
    # delta = msign(nesterov blend): singular values ~1, same singular vectors as the blend (0.19 * grad)
    sv = torch.linalg.svdvals(delta.double())
    assert sv.max() < 1.2 and sv.min() > 0.6
    want = O.msign(0.19 * grad, 5, storage="fp32")
    assert ((delta - want.float()).norm() / want.float().norm()).item() < 2e-3


@pytest.mark.parametrize("split", [
    {"kind": "fc1", "shapes": (24, 24)},
    {"kind": "qkv", "shapes": (16, 8, 8), "mode": "group"},
    {"kind": "qkv", "shapes": (16, 8, 8), "mode": "head"},
    {"kind": "qkv", "shapes": (16, 8, 8), "mode": "component"},
    {"kind": "moe1", "experts": 3, "gated": True, "split_fc1": True},
    {"kind": "moe1", "experts": 3, "gated": True, "split_fc1": False},
    {"kind": "moe2", "experts": 4},
])
def test_split_components_equal_the_same_matrix_alone(split):
    g = torch.Generator().manual_seed(21)
    shape = {"fc1": (48, 40), "qkv": (64, 40), "moe1": (40, 96), "moe2": (96, 40)}[split["kind"]]
    p = torch.randn(*shape, generator=g) * 0.05
    m = torch.randn(*shape, generator=g) * 1e-2
    p_in = p.clone()
    upd = B.orthogonalize(p, m, lr=0.01, split=split, **KW)
    assert upd.shape == p.shape
    # pick one component by hand and run it alone
    if split["kind"] == "fc1":
        W, M, got_u, got_w = p_in[24:].clone(), m[24:], upd[24:], p[24:]
    elif split["kind"] == "qkv" and split["mode"] == "group":
        W, M, got_u, got_w = p_in[32 + 16:32 + 24].clone(), m[32 + 16:32 + 24], upd[32 + 16:32 + 24], p[32 + 16:32 + 24]   # K of group 1
    elif split["kind"] == "qkv" and split["mode"] == "head":
        W, M, got_u, got_w = p_in[8:16].clone(), m[8:16], upd[8:16], p[8:16]                                           # Q head 1 of group 0
    elif split["kind"] == "qkv":
        rows = list(range(16, 24)) + list(range(48, 56))                                                              # K of both groups
        W, M, got_u, got_w = p_in[rows].clone(), m[rows], upd[rows], None
        assert torch.equal(p, p_in)                                                                                   # no retraction in this mode
    elif split["kind"] == "moe1" and split["split_fc1"]:
        W, M = p_in[:, 32 + 16:64].t().clone(), m[:, 32 + 16:64].t()                                                   # "up" of expert 1
        got_u, got_w = upd[:, 32 + 16:64].t(), p[:, 32 + 16:64].t()
    elif split["kind"] == "moe1":
        W, M, got_u, got_w = p_in[:, 32:64].t().clone(), m[:, 32:64].t(), upd[:, 32:64].t(), p[:, 32:64].t()
    else:
        W, M, got_u, got_w = p_in[48:72].t().clone(), m[48:72].t(), upd[48:72].t(), p[48:72].t()
    want_u = B.component_update(W, M, current_lr=0.01, **KW)
    assert torch.allclose(got_u.float(), want_u.float(), rtol=1e-6, atol=1e-8)
    if got_w is not None:
        assert torch.allclose(got_w, W, rtol=1e-6, atol=1e-9)
