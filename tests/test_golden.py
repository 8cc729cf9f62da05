"""Committed known-answer vectors (tests/golden/muon_golden.npz, written by tests/golden/make_golden.py from
fp64 closed forms): the CPU oracle is checked against them here, the HIP path in the gpu-marked tests."""
import os

import numpy as np
import pytest
import torch

from oracle import muon_oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "muon_golden.npz"))


def _rel(a, b):
    a, b = torch.as_tensor(a).double().cpu(), torch.as_tensor(b).double()
    return ((a - b).norm() / b.norm()).item()


@pytest.mark.parametrize("name", ["wide", "tall", "square"])
@pytest.mark.parametrize("table", ["simple", "quintic"])
def test_oracle_ns_matches_golden(name, table):
    G = torch.from_numpy(GOLD[f"ns_in_{name}"])
    want = GOLD[f"ns_out_{name}_{table}"]
    got = O.newton_schulz(G, O.coefficient_schedule(table, 5), 1e-7, storage="fp32")
    assert _rel(got, want) < 5e-4
    # the reference's eager bf16 semantics stay within its known distance of the exact answer
    eager = O.newton_schulz(G, O.coefficient_schedule(table, 5), 1e-7, storage="bf16_eager")
    assert _rel(eager.float(), want) < 6e-2


def test_oracle_updates_match_golden():
    lr, wd, eps = GOLD["upd_hyper"]
    X = torch.from_numpy(GOLD["upd_x"]).float()
    U = torch.from_numpy(GOLD["upd_u"]).to(torch.bfloat16)
    Y = X.clone()
    O.muonh_post_orthogonalize(Y, U, float(lr), float(wd), float(eps))
    assert _rel(Y, GOLD["upd_muonh"]) < 2e-3          # bf16 rounding of U*s*lr in the reference's op order
    Y = X.clone()
    O.muon_post_orthogonalize(Y, U, float(lr), O.adjust_lr(float(lr), (64, 80), "spectral_norm"), float(wd))
    assert _rel(Y, GOLD["upd_plain"]) < 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["wide", "tall", "square"])
@pytest.mark.parametrize("table", ["simple", "quintic"])
def test_hip_ns_matches_golden(gpu_device, name, table):
    import archscale_amd.optim.newton_schulz_hip as H
    G = torch.from_numpy(GOLD[f"ns_in_{name}"]).to(torch.bfloat16).to(gpu_device)
    got = H.newton_schulz(G, O.coefficient_schedule(table, 5), 1e-7, prec="bsplit" if table == "simple" else "bf16")
    assert _rel(got, GOLD[f"ns_out_{name}_{table}"]) <= 1e-2


@pytest.mark.gpu
def test_hip_updates_match_golden(gpu_device):
    from archscale_amd.optim.muon import Muon
    lr, wd, eps = (float(v) for v in GOLD["upd_hyper"])
    U = torch.from_numpy(GOLD["upd_u"]).to(torch.bfloat16)
    for use_muonh, key in ((True, "upd_muonh"), (False, "upd_plain")):
        p = torch.nn.Parameter(torch.from_numpy(GOLD["upd_x"]).float().to(gpu_device))
        # feed U through the hook, so that only momentum (zero state, mu = 0) and the update kernels are exercised
        opt = Muon([p], lr=lr, mu=0.0, weight_decay=wd, epsilon=eps, nesterov=False, use_muonh=use_muonh,
                   newton_schulz_func=lambda X, epsilon: U.to(gpu_device))
        p.grad = torch.ones_like(p)
        opt.step()
        assert _rel(p.detach(), GOLD[key]) < 1e-5
