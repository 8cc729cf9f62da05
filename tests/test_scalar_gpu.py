"""AdamW / hyperball-AdamW / Lion multi-tensor HIP kernels (through the C ABI) against the CPU oracle.
fp32 state: element-wise agreement to fp32 round-off; bf16 state: within one bf16 ulp of the oracle's own rounding."""
import pytest
import torch

from oracle import scalar_oracle as S

pytestmark = pytest.mark.gpu

SHAPES = [(1000,), (64, 96), (3, 5, 7), (8192 * 2 + 8,), (33,)]


def _mk(dtype, seed):
    g = torch.Generator().manual_seed(seed)
    X = [(torch.randn(*s, generator=g)).to(dtype) for s in SHAPES]
    G = [(torch.randn(*s, generator=g) * 0.1).to(dtype) for s in SHAPES]
    M = [(torch.randn(*s, generator=g) * 0.05).to(dtype) for s in SHAPES]
    V = [(torch.rand(*s, generator=g) * 0.01).to(dtype) for s in SHAPES]
    return X, G, M, V


def _close(a, b, dtype):
    a, b = a.float().cpu(), b.float()
    if dtype == torch.float32:
        return torch.allclose(a, b, rtol=2e-5, atol=1e-6)
    return torch.allclose(a, b, rtol=1.6e-2, atol=1e-3)   # two bf16 roundings apart at most


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cautious", [False, True])
def test_adamw_lion_hyperball(gpu_device, dtype, cautious):
    from archscale_amd.optim import scalar_opts as H
    dev = gpu_device
    for algo in ("adamw", "lion", "hyperball"):
        X, G, M, V = _mk(dtype, 3)
        Xd, Gd, Md, Vd = ([t.clone().to(dev) for t in L] for L in (X, G, M, V))
        if algo == "adamw":
            for step in (1, 2):
                S.adamw_update_foreach(X, G, M, V, 1e-2, 0.9, 0.95, 0.1, step, 1e-8, cautious)
                H.adamw_update_foreach(Xd, Gd, Md, Vd, 1e-2, 0.9, 0.95, 0.1, step, 1e-8, cautious)
        elif algo == "lion":
            S.lion_update_foreach(X, G, M, 1e-2, 0.9, 0.99, 0.1, cautious)
            H.lion_update_foreach(Xd, Gd, Md, 1e-2, 0.9, 0.99, 0.1, cautious)
        else:
            S.hyperball_adamw_update_foreach(X, G, M, V, 1e-2, 0.9, 0.95, 0.1, 3, 1e-8, cautious)
            H.hyperball_adamw_update_foreach(Xd, Gd, Md, Vd, 1e-2, 0.9, 0.95, 0.1, 3, 1e-8, cautious)
        torch.cuda.synchronize()
        for i in range(len(SHAPES)):
            assert _close(Md[i], M[i], dtype), (algo, i)
            if algo != "lion":
                assert _close(Vd[i], V[i], dtype), (algo, i)
            if algo == "lion" and dtype == torch.bfloat16:
                # a sign can flip where the interpolated momentum is within rounding of zero; allow a handful
                bad = (Xd[i].float().cpu() - X[i].float()).abs() > 2e-2
                assert bad.float().mean().item() < 1e-2
            else:
                assert _close(Xd[i], X[i], dtype), (algo, i)


def test_hyperball_norm_and_zero_grad(gpu_device):
    from archscale_amd.optim import scalar_opts as H
    x = [torch.randn(128, 64, device=gpu_device), torch.randn(40, 40, device=gpu_device)]
    n0 = [t.norm().item() for t in x]
    g = [torch.randn_like(t) for t in x]
    g[1].zero_()
    m = [torch.zeros_like(t) for t in x]
    v = [torch.zeros_like(t) for t in x]
    x1 = x[1].clone()
    H.hyperball_adamw_update_foreach(x, g, m, v, 0.05, 0.9, 0.95, 0.0, 1, 1e-8)
    assert x[0].norm().item() == pytest.approx(n0[0], rel=1e-5)
    assert torch.allclose(x[1], x1, rtol=1e-6)     # zero direction: clamp path leaves the tensor alone
