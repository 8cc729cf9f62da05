"""Host logic of MuonBall that needs no GPU: constructor validation and the slicing of fused parameters into pieces
(checked against explicit tensor views of the layouts in muon_ball.py:407-621 of the reference)."""
import pytest
import torch

from archscale_amd.emerging import MuonBall
from archscale_amd.emerging.spectral_ball_utils import (apply_retract, compute_target_radius,
                                                        get_spectral_ball_scale_factor)


def _p(shape, name="w", **attrs):
    p = torch.nn.Parameter(torch.arange(shape[0] * shape[1], dtype=torch.float32).view(*shape))
    p.param_name = name
    for k, v in attrs.items():
        setattr(p, k, v)
    return p


def test_constructor_validation_and_defaults():
    p = _p((4, 6))
    opt = MuonBall([p])
    d = opt.defaults
    assert (d["lr"], d["momentum_beta"], d["weight_decay"]) == (3e-4, 0.9, 0.01)
    assert opt.use_nesterov and opt.weight_decay_method == "decoupled" and opt.power_iteration_steps == 10
    assert opt.msign_steps == 5 and opt.radius_mode == "spectral_mup" and opt.scale_mode == "align_adamw_rms"
    assert opt.retract_mode == "hard" and opt.retract_alpha == 0.05 and opt.qkv_split_mode == "component"
    assert opt.get_retract_bias_dict() is None and opt.get_spectral_norm_dict() is None
    for kw in (dict(power_iteration_steps=0), dict(msign_steps=0), dict(radius_mode="x"), dict(retract_mode="soft"),
               dict(qkv_split_mode="rows")):
        with pytest.raises(ValueError):
            MuonBall([p], **kw)
    MuonBall([p], radius_mode="initialize")      # accepted by the constructor, rejected when the radius is computed
    with pytest.raises(NotImplementedError):
        opt.scaled_orthogonalize_fn(p)

    class _G:
        def size(self):
            return 2
    class _PG:
        tp = _G()
    with pytest.raises(NotImplementedError):
        MuonBall([p], pg_collection=_PG())


def test_cpu_tensors_fail_loudly():
    from archscale_amd._lib import MuonLibraryError
    p = _p((4, 6))
    p.grad = torch.ones_like(p)
    with pytest.raises(MuonLibraryError):
        MuonBall([p]).step()


def _view(p, pc):
    return torch.as_strided(p.data, (pc.rows, pc.cols), (pc.ld, 1), pc.off)


def test_pieces_standard_fc1_qkv():
    opt = MuonBall([_p((4, 6))], split_fc1=True, is_fc1_fn=lambda p: p.shape[0] == 10, fc1_split_shapes=(6, 4),
                   split_qkv=True, is_qkv_fn=lambda p: p.shape[0] == 16, qkv_split_shapes=(4, 2, 2), qkv_split_mode="group")
    p = _p((5, 7))
    (pc,) = opt._pieces_of(0, p, p)
    assert (pc.off, pc.rows, pc.cols, pc.ld, pc.shape, pc.label) == (0, 5, 7, 7, (5, 7), None)
    p = _p((10, 3))
    gate, up = opt._pieces_of(0, p, p)
    assert torch.equal(_view(p, gate), p.data[:6]) and torch.equal(_view(p, up), p.data[6:])
    assert (gate.label, up.label, gate.shape, up.shape) == ("gate", "up", (6, 3), (4, 3))
    p = _p((16, 3))
    pieces = opt._pieces_of(0, p, p)
    assert [pc.label for pc in pieces] == ["g0.q", "g0.k", "g0.v", "g1.q", "g1.k", "g1.v"]
    v = p.data.view(2, 8, 3)
    assert torch.equal(_view(p, pieces[4]), v[1, 4:6]) and torch.equal(_view(p, pieces[0]), v[0, 0:4])
    opt.qkv_split_mode = "head"
    pieces = opt._pieces_of(0, p, p)
    assert [pc.label for pc in pieces] == ["g0.Q.h0", "g0.Q.h1", "g0.K", "g0.V", "g1.Q.h0", "g1.Q.h1", "g1.K", "g1.V"]
    assert torch.equal(_view(p, pieces[5]), v[1, 2:4]) and pieces[5].shape == (2, 3)
    opt.qkv_split_mode = "component"
    q, k, vv = opt._pieces_of(0, p, p)
    assert (q.gather, k.gather, vv.gather) == ((2, 8, 0, 4), (2, 8, 4, 2), (2, 8, 6, 2))
    assert (q.shape, k.shape, q.label) == ((8, 3), (4, 3), "q")
    opt.qkv_split_shapes = (5, 2, 2)
    with pytest.raises(AssertionError):
        opt._pieces_of(0, p, p)


def test_pieces_moe():
    opt = MuonBall([_p((4, 6))], split_moe_experts=True, is_grouped_moe_fn=lambda p: hasattr(p, "num_local_experts"))
    p = _p((5, 12), "experts.weight1", num_local_experts=3, is_gated=True)
    pieces = opt._pieces_of(0, p, p)
    r = p.data.view(5, 3, 4)
    assert [pc.label for pc in pieces] == ["expert0", "expert1", "expert2"]
    assert all(torch.equal(_view(p, pc), r[:, e, :]) and pc.shape == (4, 5) for e, pc in enumerate(pieces))
    opt.split_fc1 = True
    pieces = opt._pieces_of(0, p, p)
    assert [pc.label for pc in pieces] == ["expert0.gate", "expert0.up", "expert1.gate", "expert1.up", "expert2.gate", "expert2.up"]
    assert torch.equal(_view(p, pieces[3]), r[:, 1, 2:4]) and pieces[3].shape == (2, 5)
    p = _p((12, 5), "experts.weight2", num_local_experts=4)
    pieces = opt._pieces_of(0, p, p)
    r = p.data.view(4, 3, 5)
    assert all(torch.equal(_view(p, pc), r[e]) and pc.shape == (5, 3) for e, pc in enumerate(pieces))
    # one expert, or a name without weight1/weight2: the whole matrix
    p = _p((12, 5), "experts.weight2", num_local_experts=1)
    assert len(opt._pieces_of(0, p, p)) == 1
    p = _p((12, 5), "experts.other", num_local_experts=4)
    assert len(opt._pieces_of(0, p, p)) == 1
    with pytest.raises(ValueError):
        t = torch.nn.Parameter(torch.zeros(2, 3, 4))
        opt._pieces_of(0, t, t)


def test_scalar_helpers():
    assert compute_target_radius((64, 16), "spectral_mup") == 2.0 and compute_target_radius((3, 5), "identity", radius_scaler=0.5) == 0.5
    with pytest.raises(ValueError):
        compute_target_radius((3, 5), "initialize")
    assert get_spectral_ball_scale_factor(16, 64, "align_adamw_rms") == pytest.approx(1.6)
    assert get_spectral_ball_scale_factor(64, 16, "shape_scaling") == 2.0 and get_spectral_ball_scale_factor(16, 64, "spectral_mup") == 0.5
    with pytest.raises(ValueError):
        get_spectral_ball_scale_factor(1, 1)
    W = torch.ones(2, 2)
    assert apply_retract(W, 2.0, 1.0, mode="hard") == 0.0 and torch.allclose(W, torch.full((2, 2), 0.5))
    assert apply_retract(W, 2.0, 1.0, mode="dynamic", alpha=0.1, current_lr=0.5) == -1.0 and torch.allclose(W, torch.full((2, 2), 0.475))
    with pytest.raises(ValueError):
        apply_retract(W, 1.0, 1.0, mode="x")
