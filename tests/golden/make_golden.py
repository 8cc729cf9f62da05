#!/usr/bin/env python3
"""Writes tests/golden/muon_golden.npz: small known-answer vectors for the Muon / MuonH path.

The reference ships no golden vectors for this path and none of its modules is imported here.  The expected
outputs come from formulas that are INDEPENDENT of the iteration being tested:
  * Newton-Schulz: U diag(p_5(..p_1(s/(|G|_F + eps)))) V^T from an fp64 SVD of the bf16-rounded input,
    p(s) = a s + b s^3 + c s^5 per coefficient row;
  * MuonH update: the fp64 closed form  r (x' - lr s U),  s = |x'|/|U|,  r = |x'|/|x' - lr s U|;
  * plain update: x (1 - lr wd) - lr_adj U.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

TABLES = {
    "simple": [(3.4445, -4.7750, 2.0315)] * 5,
    "quintic": [(4.0848, -6.8946, 2.9270), (3.9505, -6.3029, 2.6377), (3.7418, -5.5913, 2.3037),
                (2.8769, -3.1427, 1.2046), (2.8366, -3.0525, 1.2012)],
}


def ns_closed_form(G_bf16: torch.Tensor, rows, eps: float) -> torch.Tensor:
    G = G_bf16.to(torch.float64)
    U, S, Vh = torch.linalg.svd(G, full_matrices=False)
    s = S / (G.norm() + eps)
    for a, b, c in rows:
        s = a * s + b * s ** 3 + c * s ** 5
    return U @ torch.diag(s) @ Vh


def main():
    g = torch.Generator().manual_seed(20240521)
    out = {}
    for name, shape in (("wide", (48, 160)), ("tall", (160, 48)), ("square", (96, 96))):
        G = torch.randn(*shape, generator=g).to(torch.bfloat16)
        out[f"ns_in_{name}"] = G.float().numpy()          # exactly representable in bf16
        for table, rows in TABLES.items():
            out[f"ns_out_{name}_{table}"] = ns_closed_form(G, rows, 1e-7).numpy()
    X = (torch.randn(64, 80, generator=g) * 0.02).to(torch.float64)
    U = torch.randn(64, 80, generator=g).to(torch.bfloat16).to(torch.float64)
    lr, wd, eps = 0.02, 0.1, 1e-8
    xd = X * (1 - lr * wd)
    y = xd - lr * (xd.norm() / U.norm()) * U
    out["upd_x"], out["upd_u"] = X.numpy(), U.numpy()
    out["upd_muonh"] = (y * xd.norm() / y.norm()).numpy()
    out["upd_plain"] = (xd - lr * np.sqrt(64 / 80) * U).numpy()
    out["upd_hyper"] = np.array([lr, wd, eps])
    np.savez_compressed(os.path.join(HERE, "muon_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "muon_golden.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
